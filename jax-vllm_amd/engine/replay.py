"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and owns no forward pass, cache or loader: it drives the framework's
model, step function, cache manager and kernels, the ones generation uses.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch.  For a step in which something is wanted,
``DIR/<step>.f32`` receives the logits at the wanted places, in the order of the entries
and of ``want``, as little-endian float32 ``[wanted, vocab]``.  After every step the line
``done <step>`` is printed and flushed.  Requests named in ``end`` give back what they
hold after the step.  The page pool is sized for ``--max-tokens`` tokens (each live
request's count rounded up to the page size), so pages are used again.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path


def _say(msg: str) -> None:
    print(f"[trace_run] {msg}", file=sys.stderr, flush=True)


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder that receives <step>.f32")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (per request rounded up to the page size)")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page (default 16)")
    p.add_argument("--max-num-seqs", type=int, default=8, help="state slots / live requests (default 8)")
    return p.parse_args(argv)


def main(argv=None, stdin=None, stdout=None) -> int:
    args = parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    t0 = time.time()
    _say("importing torch ...")
    import numpy as np
    import torch

    from ..config.engine import EngineConfig
    from ..ops import library
    from ..weights import load_model
    from .core import EngineCore
    from .entries import StepEntry

    if not torch.cuda.is_available():
        _say("no GPU visible: the engine has no CPU path")
        return 3
    library.core()  # compiles at the first call in a fresh checkout
    _say(f"loading {args.model} as {args.dtype} ({time.time() - t0:.0f}s)")
    model, _ = load_model(args.model, args.dtype, "cuda")
    pages = -(-args.max_tokens // args.block_size)
    cfg = EngineConfig(dtype=args.dtype, block_size=args.block_size, num_blocks=pages + 1,
                       max_num_seqs=args.max_num_seqs, max_model_len=max(args.max_tokens, args.block_size),
                       max_num_batched_tokens=max(args.max_tokens, 1), enable_prefix_cache=False,
                       use_hip_graphs=False)
    core = EngineCore(model, cfg)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    _say(f"ready: {pages} pages of {args.block_size} tokens ({time.time() - t0:.0f}s)")

    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            if not core.has_request(e["id"]):
                core.start_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e.get("want", [])))
        logits = core.run(entries)
        if logits.shape[0] > 0:
            arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            np.ascontiguousarray(arr).tofile(out_dir / f"{step}.f32")
        else:
            torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if core.has_request(rid):
                core.finish_request(rid)
        print(f"done {step}", file=stdout, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
