"""Trace replay: feed given token ids through the engine step by step and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry continues (or starts) the request ``id`` with its next tokens; all entries of a
step run as one batch through ``Engine.step``, the same model, cache and kernels generation
uses.  ``want`` lists the places among an entry's tokens whose logits are written, in the order
of the entries, to ``<out>/<step>.f32`` as little-endian float32 [wanted, vocab].  Requests
named in ``end`` give back what they hold after the step.  After each step ``done <step>`` is
printed and flushed.  Nothing is sampled.  The reference has no such tool; its nearest
relative is the perplexity loop that feeds a window block by block and reads every row
(reference: src/zedinfer/engine.cpp:575,643-665).
"""
from __future__ import annotations

import argparse
import json
import os
import sys


PAGE_SIZE = 16          # divides the 64-token rounding of --max-tokens
MAX_LIVE = 8


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at once (each rounded up to 64)")
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    os.makedirs(args.out, exist_ok=True)

    import numpy as np
    import torch
    from ..config import SchedulerConfig
    from ..engine import Engine, StepEntry

    pages = -(-args.max_tokens // PAGE_SIZE)
    sched = SchedulerConfig(num_kv_blocks=pages, kv_block_size=PAGE_SIZE, max_batch_requests=MAX_LIVE,
                            max_batch_tokens=max(args.max_tokens, 1), max_seq_len=max(args.max_tokens, 1))
    print(f"[trace_run] loading {args.model} as {args.dtype}", file=sys.stderr, flush=True)
    engine = Engine.from_folder(args.model, args.dtype, sched)
    print(f"[trace_run] ready: {pages} pages of {PAGE_SIZE} tokens per cache group", file=sys.stderr, flush=True)

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in live:
                live[rid] = engine.open(rid)
            entries.append(StepEntry(live[rid], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if entries:
            logits = engine.step(entries, copy=False)
            if logits is not None:
                arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if rid in live:
                engine.close(live.pop(rid))
        sys.stdout.write(f"done {step}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
