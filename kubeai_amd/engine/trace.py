"""Replay a recorded token stream through the engine, step by step, and write
the logits it produces. Nothing is sampled: every step says which sequences
run, which tokens each contributes and at which of them logits are wanted.

    python -m kubeai_amd.engine.trace --model DIR --dtype bfloat16|float32 \\
        --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": ["a"]}

All entries of a step are one packed batch through LLMEngine.step_fixed — the
engine's own model, scheduler bookkeeping, paged cache, state slots and
kernels. For a step with wanted rows, OUT/<step>.f32 receives them as
little-endian fp32 [rows, vocab] in entry order; after every step the line
"done <step>" is printed. The cache pool holds --max-tokens tokens (rounded
up to whole blocks) and --max-seqs state slots, so blocks and slots are
reused as sequences end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json + safetensors")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--out", required=True)
    p.add_argument("--max-tokens", type=int, required=True,
                   help="tokens the cache pool holds at any time")
    p.add_argument("--max-seqs", type=int, default=4,
                   help="sequences live at any time (state slots)")
    p.add_argument("--device", default="cuda",
                   help="cuda (default) or cpu (reference ops, development only)")
    args = p.parse_args(argv)

    import torch

    if args.device.startswith("cuda") and not torch.cuda.is_available():
        print("no GPU visible; pass --device cpu to run the reference ops",
              file=sys.stderr)
        return 4
    # float32 means true 32-bit products, never a reduced-precision mode
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")

    from kubeai_amd.engine import EngineConfig, LLMEngine

    block = 16
    eng = LLMEngine(
        EngineConfig(
            model=args.model,
            device=args.device,
            dtype=args.dtype,
            block_size=block,
            num_gpu_blocks=max(1, (args.max_tokens + block - 1) // block),
            max_num_seqs=args.max_seqs,
            max_model_len=1 << 30,
            max_num_batched_tokens=1 << 30,
            enable_prefix_caching=False,
            enable_graphs=False,
        )
    )
    os.makedirs(args.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [
            (e["id"], e["tokens"], e.get("want") or []) for e in step["entries"]
        ]
        rows = eng.step_fixed(entries, step.get("end") or [])
        rows = [r for r in rows if r.shape[0] > 0]
        if rows:
            data = torch.cat(rows).to(torch.float32).cpu().contiguous().numpy()
            tmp = os.path.join(args.out, ".%d.part" % step["step"])
            with open(tmp, "wb") as f:
                f.write(data.astype("<f4").tobytes())
            os.replace(tmp, os.path.join(args.out, "%d.f32" % step["step"]))
        print("done %d" % step["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
