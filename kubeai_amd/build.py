"""Build-on-demand of the in-tree HIP extensions.

`ensure_built(["_C_seq"])` compiles the named extensions (setup.py, gfx950)
when their shared object is missing or older than its sources, under a file
lock so concurrent first starts do not race. Programs that start a model
call it with the extensions that model's family needs and nothing more.
"""
from __future__ import annotations

import fcntl
import glob
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SRC_DIRS = {"_C": "csrc", "_C_seq": "csrc_seq"}


def _built_object(name: str):
    hits = glob.glob(os.path.join(ROOT, "kubeai_amd", name + ".*.so"))
    return hits[0] if hits else None


def _stale(name: str) -> bool:
    so = _built_object(name)
    if so is None:
        return True
    built = os.path.getmtime(so)
    src = os.path.join(ROOT, "kubeai_amd", _SRC_DIRS[name])
    for f in glob.glob(os.path.join(src, "*")):
        if f.endswith(("_hip.hip", "_hip.h")):
            continue  # generated
        if f.endswith((".hip", ".cpp", ".h")) and os.path.getmtime(f) > built:
            return True
    return False


def ensure_built(names, log=sys.stderr) -> None:
    todo = [n for n in names if _stale(n)]
    if not todo:
        return
    os.makedirs(os.path.join(ROOT, "build"), exist_ok=True)
    with open(os.path.join(ROOT, "build", ".ext.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        todo = [n for n in names if _stale(n)]  # another process may have built
        if not todo:
            return
        env = dict(os.environ, PYTORCH_ROCM_ARCH="gfx950",
                   KUBEAI_BUILD_ONLY=",".join(todo))
        print("building HIP extensions: " + ", ".join(todo), file=log, flush=True)
        subprocess.run(
            [sys.executable, "setup.py", "build_ext", "--inplace"],
            cwd=ROOT, env=env, check=True, stdout=log, stderr=log,
        )
