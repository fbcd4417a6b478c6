"""Trace replay: feed given token ids through the engine step by step and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
              [--kv-block-size P] [--num-kv-blocks B] [--max-live R]

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry continues (or starts) the request ``id`` with its next tokens; all entries of a
step run as one batch through ``Engine.step``, the same model, cache and kernels generation
uses.  ``want`` lists the places among an entry's tokens whose logits are written, in the order
of the entries, to ``<out>/<step>.f32`` as little-endian float32 [wanted, vocab].  Requests
named in ``end`` give back what they hold after the step.  After each step ``done <step>`` is
printed and flushed.  Nothing is sampled.

The cache pool is made for ``--max-tokens`` tokens (every live request's count rounded up to a
multiple of 64, or of the page size when that is larger), in pages of ``--kv-block-size`` tokens
(default 16); ``--num-kv-blocks`` gives the number of pages outright and ``--max-live`` the most
requests live at a time (default 8).  A trace may carry the same geometry itself, as a line before
its first step, which then wins over the options:

    {"geometry": {"kv_block_size": 8, "num_kv_blocks": 40, "max_live": 4}}

When the input ends, a line for each cache group on standard error says how many pages the pool has
and how many were handed out in all (more than the pool has: pages were used again).

The reference has no such tool; its nearest
relative is the perplexity loop that feeds a window block by block and reads every row
(reference: src/zedinfer/engine.cpp:575,643-665).
"""
from __future__ import annotations

import argparse
import json
import os
import sys


ROUND_TO = 64           # --max-tokens counts every live request rounded up to a multiple of this


def pool_pages(max_tokens: int, page_size: int) -> int:
    """Pages that hold ``max_tokens`` tokens when every request's count was rounded up to a multiple of
    ROUND_TO (of the page size when that is larger) and every request has pages of its own."""
    if page_size >= ROUND_TO:
        return -(-max_tokens // page_size)
    return -(-max_tokens // ROUND_TO) * (-(-ROUND_TO // page_size))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at once (each rounded up to 64)")
    ap.add_argument("--kv-block-size", type=int, default=16, help="tokens a page of the cache holds (default 16)")
    ap.add_argument("--num-kv-blocks", type=int, default=0,
                    help="pages of the cache pool (default: what --max-tokens needs)")
    ap.add_argument("--max-live", type=int, default=8, help="most requests live at a time (default 8)")
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    if args.kv_block_size <= 0 or args.num_kv_blocks < 0 or args.max_live <= 0:
        ap.error("--kv-block-size and --max-live must be positive, --num-kv-blocks not negative")
    os.makedirs(args.out, exist_ok=True)

    import torch
    from ..config import SchedulerConfig
    from ..engine import Engine, StepEntry

    geometry = {"kv_block_size": args.kv_block_size, "num_kv_blocks": args.num_kv_blocks, "max_live": args.max_live}
    engine = None

    def make_engine():
        ps = int(geometry["kv_block_size"])
        pages = int(geometry["num_kv_blocks"]) or pool_pages(args.max_tokens, ps)
        room = max(args.max_tokens, pages * ps, 1)
        sched = SchedulerConfig(num_kv_blocks=pages, kv_block_size=ps, max_batch_requests=int(geometry["max_live"]),
                                max_batch_tokens=room, max_seq_len=room)
        print(f"[trace_run] loading {args.model} as {args.dtype}", file=sys.stderr, flush=True)
        eng = Engine.from_folder(args.model, args.dtype, sched)
        print(f"[trace_run] ready: {pages} pages of {ps} tokens per cache group, up to {geometry['max_live']} "
              f"live requests", file=sys.stderr, flush=True)
        return eng

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        if "geometry" in rec:
            if engine is not None:
                raise SystemExit("trace_run: the geometry line must come before the first step")
            unknown = set(rec["geometry"]) - set(geometry)
            if unknown:
                raise SystemExit(f"trace_run: unknown geometry key(s) {sorted(unknown)}; known: {sorted(geometry)}")
            geometry.update({k: int(v) for k, v in rec["geometry"].items()})
            continue
        if engine is None:
            engine = make_engine()
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
    if engine is not None:
        for gi, g in enumerate(engine.cache.groups):
            print(f"[trace_run] cache group {gi} ({g.kind}): {g.pool.total} pages, {g.pool.takes} handed out",
                  file=sys.stderr, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
