"""Trace replay: feeds given token ids through a model step by step and writes
logits.  It samples nothing and has no forward pass, cache or loader of its own:
it drives the engine's model, step function, cache manager and kernels.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object a line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, DIR/<step>.f32 receives the logits at
the wanted places (order of the entries, then of `want`) as little-endian
float32 [wanted, vocab].  After every step a line `done <step>` is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to a page)")
    ap.add_argument("--block-size", type=int, default=64, help="positions per cache page")
    ap.add_argument("--max-seqs", type=int, default=8, help="state slots (live requests)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)

    print("[trace_run] starting (the first import of torch on a fresh machine can take a minute)",
          file=sys.stderr, flush=True)
    import numpy as np
    import torch

    from .loading import load_model
    from .runner import ModelRunner, StepEntry

    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; this engine has no CPU path", file=sys.stderr)
        return 2
    os.makedirs(args.out, exist_ok=True)
    bs = args.block_size
    model = load_model(args.model, args.dtype, args.device)
    runner = ModelRunner(model, block_size=bs, num_pages=max(1, -(-args.max_tokens // bs)),
                         max_seqs=args.max_seqs)
    print(f"[trace_run] model loaded: {len(model.blocks)} layers, {args.dtype}, "
          f"{runner.manager.n_free_pages()} pages of {bs}", file=sys.stderr, flush=True)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid, toks = e["id"], e["tokens"]
            if rid not in runner.manager and not runner.admit(rid):
                print(f"trace_run: step {step}: no free slot for request {rid!r}", file=sys.stderr)
                return 3
            if not runner.reserve(rid, len(toks)):
                print(f"trace_run: step {step}: out of cache pages for request {rid!r} "
                      f"(--max-tokens {args.max_tokens})", file=sys.stderr)
                return 3
            entries.append(StepEntry(rid, toks, list(e.get("want", []))))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(args.out, f"{step}.f32"))
        for rid in rec.get("end", []):
            runner.release(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
