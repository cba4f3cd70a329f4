"""Trace replay: feed given token ids through a model step by step and write the logits it is asked for.

    bin/trace_run --model PATH --dtype bfloat16|float32 --out DIR --max-tokens N [--device cuda|cpu]

Steps arrive on standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step are ONE forward of the engine (`Runner.step_entries`: portions of prompts beside
single tokens of other requests). A request is admitted at its first entry and may sit out steps; the
requests under "end" give their cache blocks and state slot back after the step. For a step with wanted
places, DIR/<step>.f32 holds their logits, little-endian float32 [wanted, vocab], in entry order; after
every step the line "done <step>" is printed. Nothing is sampled.

The model class follows the model: a folder with config.json + model.safetensors is a layer-list model
(engine/stack_runner.py), a GGUF file a `Runner`. The cache pool holds --max-tokens tokens (in blocks of 16),
and there are four sequence slots. float32 is refused (exit 3) for GGUF models, whose kernels are 16-bit.
The default device is the GPU and there is no fallback from it; `--device cpu` runs the torch twin of the
executor, the host-logic test vehicle.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

SLOTS = 4


def _ensure_built(stack: bool) -> None:
    """A fresh checkout has no built library: compile what this model's engine needs, and only that."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    import torch  # noqa: F401  (first: the native modules share the HIP runtime that torch ships)
    import build_native
    if stack:
        try:
            from . import _stack  # noqa: F401
        except ImportError:
            build_native.build_stack()
    else:
        try:
            from . import _C  # noqa: F401
        except ImportError:
            build_native.build()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default="cuda", choices=["cuda", "cpu"])
    ap.add_argument("--max-batch", type=int, default=512, help="rows per forward (longer steps run in parts)")
    a = ap.parse_args(argv)
    from .models.config import is_stack_model
    stack = is_stack_model(a.model)
    if not stack and a.dtype == "float32":
        print("trace_run: GGUF models run on 16-bit kernels only; float32 is refused", file=sys.stderr)
        return 3
    if a.device == "cuda":
        _ensure_built(stack)
    import numpy as np
    import torch
    if a.device == "cuda" and not torch.cuda.is_available():
        print("trace_run: no GPU visible (the engine's step runs on HIP kernels; --device cpu is the test twin)",
              file=sys.stderr)
        return 1
    dev = "cuda:0" if a.device == "cuda" else "cpu"
    os.makedirs(a.out, exist_ok=True)
    n_tok = max(16, a.max_tokens)
    if stack:
        from .engine.stack_runner import StackRunner
        r = StackRunner(a.model, device=dev, dtype=a.dtype, max_batch=a.max_batch, max_seqs=SLOTS, ctx=n_tok,
                        kv_tokens=n_tok, use_graphs=False)
    else:
        from .engine.runner import Runner
        r = Runner(a.model, device=dev, max_batch=a.max_batch, max_seqs=SLOTS, ctx=n_tok, kv_tokens=n_tok,
                   use_graphs=False)
    live: dict[str, int] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = []
        for e in st.get("entries", []):
            if e["id"] not in live:
                live[e["id"]] = r.new_sequence()
            entries.append((live[e["id"]], [int(t) for t in e["tokens"]], [int(i) for i in e.get("want", [])]))
        logits = r.step_entries(entries) if entries else None
        if logits is not None and logits.shape[0]:
            data = np.ascontiguousarray(logits.float().cpu().numpy(), dtype="<f4")
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif a.device == "cuda":
            torch.cuda.synchronize()
        for rid in st.get("end", []):
            if rid in live:
                r.free_sequence(live.pop(rid))
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
