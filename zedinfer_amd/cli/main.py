"""Command lines in the manner of the reference's examples: ``ping`` (one prompt, generated
tokens), ``bench`` (one request's prefill and decode speed) and ``batch_bench`` (throughput of a
batch), plus ``random_model``, which writes a model folder with seeded random weights.

Option names and meanings are the reference's where it has them (reference:
examples/ping.cpp:29-115, examples/bench.cpp:23-60,86-145, examples/batch_bench.cpp:27-60,101-180).
``--nvidia`` is accepted and ignored: there is one backend.  Text prompts need a tokenizer, which
this engine does not hold: ``ping`` takes token ids (``--prompt-ids``), or text (``--prompt``) when a
tokenizer.json is supplied, which the `tokenizers` package then reads.
"""
from __future__ import annotations

import argparse
import os
import random
import sys
import time
from typing import List, Optional


def _common(p: argparse.ArgumentParser) -> None:
    p.add_argument("model_path", help="Path to the model directory (config.json + *.safetensors)")
    p.add_argument("--nvidia", action="store_true", help="accepted for compatibility; the GPU is always used")
    p.add_argument("--gpu-memory-utilization", type=float, default=0.9,
                   help="Fraction of GPU memory for KV cache (0.0-1.0)")
    p.add_argument("--dtype", choices=["bf16", "fp32", "bfloat16", "float32"], default="bf16")
    p.add_argument("--random-weights", action="store_true",
                   help="model_path holds only config.json (or is a .json file); weights are drawn from --seed")
    p.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    p.add_argument("--num-kv-blocks", type=int, default=0, help="pages per cache group (0: from free memory)")
    p.add_argument("--kv-block-size", type=int,
                   default=int(os.environ.get("ZEDINFER_KV_BLOCK_SIZE", "16")), help="tokens per page")
    p.add_argument("--max-batch-tokens", type=int, default=2048)
    p.add_argument("--max-prefill-tokens", type=int, default=512)
    p.add_argument("--max-batch-requests", type=int, default=64)
    p.add_argument("--max-seq-len", type=int, default=16384)


def _logging(p: argparse.ArgumentParser, name: str):
    from .logging_options import add_logging_arguments
    add_logging_arguments(p, f"logs/{name}.log")


def _init_logging(args) -> bool:
    from .logging_options import init_logger
    try:
        init_logger(args)
        return True
    except ValueError as e:
        print(e, file=sys.stderr)
        return False


def _sampling(p: argparse.ArgumentParser) -> None:
    p.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    p.add_argument("--top-k", type=int, default=0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--repetition-penalty", type=float, default=1.0)


def _engine(args, step_tokens: Optional[List[int]] = None):
    """The serving engine the options describe.  ``step_tokens``: the program's steps of many tokens bring these
    numbers of tokens only, so the engine measures its choices for them instead of for every size."""
    from ..config import SchedulerConfig, load_config
    from ..engine import Engine, InferenceEngine
    sched = SchedulerConfig(max_batch_tokens=args.max_batch_tokens, max_batch_requests=args.max_batch_requests,
                            max_prefill_tokens=args.max_prefill_tokens,
                            gpu_memory_utilization=args.gpu_memory_utilization, kv_block_size=args.kv_block_size,
                            num_kv_blocks=args.num_kv_blocks, max_seq_len=args.max_seq_len)
    t0 = time.perf_counter()
    if args.random_weights:
        arch, cfg = load_config(args.model_path)
        eng = Engine.from_config(cfg, arch.name, args.dtype, args.seed, sched)
    else:
        eng = Engine.from_folder(args.model_path, args.dtype, sched)
    import logging
    log = logging.getLogger("zedinfer_amd")
    log.info("Engine initialized in %.0f ms (%d pages of %d tokens)", (time.perf_counter() - t0) * 1000,
             eng.cache.num_pages, eng.cache.page_size)
    sizes = None
    if step_tokens is not None:
        sizes = sorted({eng.model.step_rows(n, "mixed") for n in step_tokens if n > 1}, reverse=True)
    ie = InferenceEngine(eng, warm_up_sizes=sizes, freeze_gc=os.environ.get("ZEDINFER_GC_FREEZE", "1") not in ("", "0"))
    log.debug("choices made at warm-up: %s", eng.rt.choices)
    return ie


def load_tokenizer(path: str):
    """A tokenizer from a tokenizer.json file, through the `tokenizers` package: a text front-end beside the
    engine, which itself takes and gives token ids (the reference holds its own tokenizer:
    src/frontend/tokenizer/base.hpp:17-20)."""
    if not os.path.isfile(path):
        raise OSError(f"no tokenizer file at {path}")
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def ping(argv: Optional[List[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="ping", description="Generate from one prompt")
    _common(p)
    _sampling(p)
    p.add_argument("--prompt-ids", default="1,2,3,4,5,6,7,8",
                   help="prompt as comma-separated token ids (the engine holds no tokenizer)")
    p.add_argument("--prompt", default=None,
                   help="prompt as text, for a model folder that holds a tokenizer.json (or with --tokenizer): encoded "
                        "with the `tokenizers` package, the generated ids are decoded too")
    p.add_argument("--tokenizer", default=None, help="a tokenizer.json file (default: the one in the model folder)")
    p.add_argument("--max-new-tokens", "--max-tokens", type=int, default=0, dest="max_new_tokens",
                   help="Maximum number of new tokens to generate (0 = unlimited)")
    p.add_argument("--stream", action="store_true", help="Print token ids as they are generated")
    p.add_argument("--ignore-eos", action="store_true")
    _logging(p, "ping")
    args = p.parse_args(argv)
    if not _init_logging(args):
        return 1
    if args.max_new_tokens < 0:
        print("--max-new-tokens/--max-tokens must be >= 0", file=sys.stderr)
        return 1
    from ..engine import GenerationConfig
    tokenizer = None
    if args.prompt is not None:
        try:
            tokenizer = load_tokenizer(args.tokenizer or os.path.join(args.model_path, "tokenizer.json"))
        except (OSError, ImportError, ValueError) as e:
            print(f"--prompt needs a tokenizer: {e}", file=sys.stderr)
            return 1
    if tokenizer is not None:
        ids = tokenizer.encode(args.prompt).ids
    else:
        ids = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
    # one prompt: its full portions and the last one are the only steps of many tokens
    ie = _engine(args, [min(len(ids), args.max_prefill_tokens), len(ids) % max(args.max_prefill_tokens, 1)])
    cb = (lambda t: print(t, end=" ", flush=True)) if args.stream else None
    cfg = GenerationConfig(max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k,
                           top_p=args.top_p, repetition_penalty=args.repetition_penalty, seed=args.seed,
                           ignore_eos=args.ignore_eos, stream=args.stream, stream_callback=cb)
    res = ie.generate_tokens(ids, cfg)
    if args.stream:
        print()
    print("output_ids:", ",".join(str(t) for t in res.output_ids))
    if tokenizer is not None:
        print("output_text:", tokenizer.decode(list(res.output_ids)))
    print("finish_reason:", res.finish_reason)
    print(res.stats.summary())
    return 0


def bench(argv: Optional[List[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="bench", description="Prefill and decode speed of one request")
    _common(p)
    p.add_argument("-p", "--prefill-len", type=int, default=128)
    p.add_argument("-d", "--decode-len", "--max-tokens", type=int, default=128, dest="decode_len")
    p.add_argument("-r", "--rounds", type=int, default=3)
    _logging(p, "bench")
    args = p.parse_args(argv)
    if not _init_logging(args):
        return 1
    if args.decode_len <= 0:
        print("--decode-len/--max-tokens must be > 0 for benchmark runs", file=sys.stderr)
        return 1
    from ..engine.profiler import Profiler
    args.max_batch_tokens = max(args.max_batch_tokens, args.prefill_len)
    ie = _engine(args, [args.prefill_len])          # the prompt enters in one step
    prof = Profiler(ie.engine)
    prof.warmup(args.prefill_len, args.decode_len)
    tp = td = 0.0
    for i in range(args.rounds):
        a, b = prof.profile(args.prefill_len, args.decode_len)
        tp, td = tp + a, td + b
        print(f"Round {i + 1}: prefill={a:.2f}ms, decode={b:.2f}ms", file=sys.stderr)
    ap_, ad = tp / args.rounds, td / args.rounds
    print("\n================ Performance Report ================")
    print(f"Config : prefill={args.prefill_len}, decode={args.decode_len}, rounds={args.rounds}")
    print(f"Prefill: {ap_:8.2f} ms | {args.prefill_len / ap_ * 1000.0:8.2f} tok/s")
    print(f"Decode : {ad:8.2f} ms | {args.decode_len / ad * 1000.0:8.2f} tok/s")
    print("====================================================")
    return 0


def batch_bench(argv: Optional[List[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="batch_bench", description="Throughput of a batch of requests")
    _common(p)
    _sampling(p)
    p.add_argument("-b", "--batch-size", type=int, default=4)
    p.add_argument("-p", "--prefill-len", type=int, default=128)
    p.add_argument("-d", "--decode-len", "--max-tokens", type=int, default=128, dest="decode_len")
    p.add_argument("-r", "--rounds", type=int, default=1)
    p.add_argument("--no-warmup", action="store_true",
                   help="count the first batch too (it records the decode graphs and measures the matrix products' "
                        "way round once; the reference has no such first-time costs and no warm-up round)")
    _logging(p, "batch_bench")
    args = p.parse_args(argv)
    if not _init_logging(args):
        return 1
    if args.decode_len <= 0:
        print("--decode-len/--max-tokens must be > 0 for benchmark runs", file=sys.stderr)
        return 1
    from ..engine import GenerationConfig, InferenceRequest
    from ..engine.profiler import Profiler
    ie = _engine(args)
    print("\n============ Single-Request Baseline ============")
    prof = Profiler(ie.engine)
    prof.warmup(min(args.prefill_len, args.max_batch_tokens), args.decode_len)    # first calls load and allocate
    a, b = prof.profile(min(args.prefill_len, args.max_batch_tokens), args.decode_len)
    print(f"Prefill: {a:8.2f} ms | {args.prefill_len / a * 1000.0:8.2f} tok/s")
    print(f"Decode : {b:8.2f} ms | {args.decode_len / b * 1000.0:8.2f} tok/s  (per request)")
    print("\n============ Batch Benchmark ============")
    print(f"Config: batch_size={args.batch_size}, prefill={args.prefill_len}, decode={args.decode_len}, "
          f"rounds={args.rounds}")
    rng = random.Random(12345)
    V = ie.engine.vocab_size
    lo, hi = (100, min(30000, V - 1)) if V > 200 else (0, V - 1)
    total_ms, total_tokens = 0.0, 0
    loop = ie.serving_loop()
    for r in range(0 if args.no_warmup else -1, args.rounds):
        reqs = []
        t0 = time.perf_counter()
        for i in range(args.batch_size):
            cfg = GenerationConfig(max_new_tokens=args.decode_len, temperature=args.temperature, top_k=args.top_k,
                                   top_p=args.top_p, repetition_penalty=args.repetition_penalty,
                                   seed=args.seed + i + 1 if args.temperature > 0 else 0, ignore_eos=True)
            reqs.append(loop.submit_async(InferenceRequest([rng.randint(lo, hi) for _ in range(args.prefill_len)], cfg)))
        loop.run_loop()
        ms = (time.perf_counter() - t0) * 1000.0
        failed = [q for q in reqs if q.error]
        if failed:
            print(f"{len(failed)} request(s) failed: {failed[0].error}", file=sys.stderr)
        n = sum(len(q.output_ids) for q in reqs)
        if r < 0:
            print(f"Warm-up (not counted): {args.batch_size} requests, {n} tokens generated, {ms:.2f} ms")
            continue
        total_ms, total_tokens = total_ms + ms, total_tokens + n
        print(f"Round {r + 1}: {args.batch_size} requests, {n} tokens generated, {ms:.2f} ms")
    avg_ms, avg_tok = total_ms / args.rounds, total_tokens / args.rounds
    print("\n============ Batch Performance Report ============")
    print(f"Batch size     : {args.batch_size} requests")
    print(f"Avg total time : {avg_ms:8.2f} ms")
    print(f"Avg tokens/batch: {avg_tok:8.0f}")
    print(f"Throughput     : {avg_tok / avg_ms * 1000.0:8.2f} tok/s  (total, all requests)")
    print(f"Per-request    : {avg_ms / args.batch_size:8.2f} ms  (avg wall time per request)")
    print("===================================================")
    return 0


def random_model(argv: Optional[List[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="random_model",
                                description="Write config.json and model.safetensors with seeded random weights")
    p.add_argument("config", help="a config.json (or a folder holding one)")
    p.add_argument("out", help="folder to write")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--std", type=float, default=0.02)
    p.add_argument("--noisy-norms", action="store_true", help="norm weights 1 + N(0, std) instead of 1")
    args = p.parse_args(argv)
    import torch
    from ..config import load_config
    from ..models import expected_weights
    from ..weights import write_model_folder
    arch, cfg = load_config(args.config)
    fc = arch.forward_config(cfg)
    dt = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    write_model_folder(args.out, cfg, expected_weights(fc), args.seed, dt, args.std, args.noisy_norms)
    print(f"wrote {args.out} ({arch.name}, seed {args.seed}, {args.dtype})")
    return 0


COMMANDS = {"ping": ping, "bench": bench, "batch_bench": batch_bench, "random_model": random_model}


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] not in COMMANDS:
        print("usage: python -m zedinfer_amd.cli.main {" + ",".join(COMMANDS) + "} ...", file=sys.stderr)
        return 2
    return COMMANDS[argv[0]](argv[1:])


if __name__ == "__main__":
    sys.exit(main())
