"""Build the kubeai_amd gfx950 HIP extension in-tree.

Usage:  PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

The .so lands inside kubeai_amd/ (kubeai_amd._C) so it travels with the
repo snapshot to GPU boxes. CPU-only boxes cross-compile fine (hipcc needs
no GPU present).
"""
import os
import glob

from setuptools import setup

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from torch.utils import cpp_extension  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))

# extension name -> source folder. KUBEAI_BUILD_ONLY=<name>[,<name>] builds a
# subset (a model family's first start compiles only what it needs).
EXTENSIONS = {
    "_C": os.path.join(ROOT, "kubeai_amd", "csrc"),
    "_C_seq": os.path.join(ROOT, "kubeai_amd", "csrc_seq"),
}
_only = [n for n in os.environ.get("KUBEAI_BUILD_ONLY", "").split(",") if n]
for _n in _only:
    if _n not in EXTENSIONS:
        raise SystemExit(f"unknown extension {_n!r}; known: {sorted(EXTENSIONS)}")


def _sources(csrc: str) -> list:
    sources = sorted(
        glob.glob(os.path.join(csrc, "*.cpp")) + glob.glob(os.path.join(csrc, "*.hip"))
    )
    # torch's hipify/ninja pipeline tracks no header dependencies for .hip
    # objects: a header edit would silently ship stale kernels. Touch every
    # .hip older than its headers so the pipeline rebuilds them.
    hdr_mtime = max(
        (
            os.path.getmtime(h)
            for h in glob.glob(os.path.join(csrc, "*.h"))
            if not h.endswith("_hip.h")
        ),
        default=0.0,
    )
    for src in list(sources):
        if (
            src.endswith(".hip")
            and not src.endswith("_hip.hip")
            and os.path.exists(src)
            and os.path.getmtime(src) < hdr_mtime
        ):
            os.utime(src, None)
            gen = src[:-4] + "_hip.hip"
            if os.path.exists(gen):
                os.remove(gen)
                sources = [s for s in sources if s != gen]
    # drop hipify artifacts: they are regenerated from their base source
    return [s for s in sources if os.path.exists(s) and not s.endswith("_hip.hip")]


setup(
    name="kubeai_amd_C",
    ext_modules=[
        cpp_extension.CUDAExtension(
            name="kubeai_amd." + name,
            sources=_sources(csrc),
            extra_compile_args={
                "cxx": ["-O3", "-std=c++17"],
                "nvcc": [
                    "-O3",
                    "-std=c++17",
                    "--offload-arch=gfx950",
                    # packed fp32 math is left to scalar instructions
                    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                ],
            },
        )
        for name, csrc in EXTENSIONS.items()
        if not _only or name in _only
    ],
    cmdclass={"build_ext": cpp_extension.BuildExtension},
)
