#!/usr/bin/env python3
"""The headline benchmark: decode tokens a second of the Qwen2.5-1.5B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
    python bench.py --shape 7B --mix 64                    (continuous batching of 64 requests)
    python bench.py --shape 32B --prompt-len 8192 --prefill-len 16384 --steps 32 --warmup 8

A step is one decode step of the serving loop (schedule, model, sampling) with ``batch`` running
requests that each hold a 2,048-token prompt.  Prints ONE JSON line.  Besides the decode speed it
reports a 2,048-token prefill (tokens a second and the fraction of the bf16 matrix peak), the
decode step against the HBM roofline (bytes that must be read: every weight once and the cache of
the live requests), decode at batch 1, 64, 128 and 256, and (under "further") the same architecture at the
Qwen2.5-7B sizes: decode at batch 8 and 64 requests batched continuously.  Weights are seeded random, token ids seeded
uniform random in [100, vocab-100] as in the reference's own benchmark
(reference: src/zedinfer/profiler.cpp:79-84, docs/perf/benchmark_v0.1.0.md:3-11).
"""
import argparse
import gc
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen2.5-1.5B: the benchmark model
SHAPE = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=1536, intermediate_size=8960,
             vocab_size=151936, max_position_embeddings=32768, num_hidden_layers=28, num_attention_heads=12,
             num_key_value_heads=2, head_dim=128, rope_theta=1000000.0, rms_norm_eps=1e-6,
             tie_word_embeddings=True, use_sliding_window=False, torch_dtype="bfloat16")
# Other shapes of the same architecture, for measurements beside the headline (--shape)
SHAPES = {
    "1.5B": {},
    "7B": dict(hidden_size=3584, intermediate_size=18944, vocab_size=152064, num_hidden_layers=28,
               num_attention_heads=28, num_key_value_heads=4, tie_word_embeddings=False),
    "32B": dict(hidden_size=5120, intermediate_size=27648, vocab_size=152064, num_hidden_layers=64,
                num_attention_heads=40, num_key_value_heads=8, tie_word_embeddings=False),
}
FULL_LAYERS = 28
PROMPT = 2048
CONTEXT = 4096
HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
CHOICES = {}       # decisions the engine made in its warm-up (Engine.warm_up), printed with the result


def matmul_params_per_layer(c):
    H, I = c["hidden_size"], c["intermediate_size"]
    qd, kvd = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return H * (qd + 2 * kvd) + qd * H + 3 * H * I


def decode_bytes(c, layers, batch, ctx_tokens_total, el):
    """Bytes one decode step has to read: every weight it uses once (layers, norms, biases, the output
    head) and the keys and values of all live tokens."""
    H = c["hidden_size"]
    qd, kvd = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    per_layer = matmul_params_per_layer(c) + (qd + 2 * kvd) + 2 * H
    # the output head is read once; an untied input table is only gathered from
    weights = (layers * per_layer + c["vocab_size"] * H + H) * el
    kv = ctx_tokens_total * 2 * layers * kvd * el
    return weights + kv


def prefill_flops(c, layers, T):
    lin = 2 * T * layers * matmul_params_per_layer(c) + 2 * c["vocab_size"] * c["hidden_size"]
    att = 4 * c["num_attention_heads"] * c["head_dim"] * (T * (T + 1) // 2) * layers
    return lin + att


def rand_ids(rng, n, vocab):
    return [rng.randrange(100, vocab - 100) for _ in range(n)]


def measure_decode(engine_factory, batch, steps, warmup, vocab, prompt_len=PROMPT, warm_up_sizes=None):
    """tokens a second and ms a step of `steps` decode steps with `batch` running requests that each
    hold a prompt of `prompt_len` tokens.  `warm_up_sizes`: the numbers of rows the serving engine measures its
    choices for before (None: every size its steps can bring)."""
    import torch
    from zedinfer_amd import GenerationConfig, InferenceRequest
    from zedinfer_amd.engine import InferenceEngine
    ie = InferenceEngine(engine_factory(), warm_up_sizes=warm_up_sizes, freeze_gc=True)
    loop = ie.serving_loop()
    rng = random.Random(1234 + batch)
    reqs = [loop.submit_async(InferenceRequest(rand_ids(rng, prompt_len, vocab),
                                               GenerationConfig(max_new_tokens=warmup + steps + 2 * batch + 32,
                                                                ignore_eos=True)))
            for _ in range(batch)]
    while loop.pending_count() or any(r.phase.value != "decode" for r in reqs):
        loop.step()
    # set-up, like the prompts before: a kind of step is captured as a graph once it has come a few times
    # (Engine.graph_after); the warm-up and the timed steps are steps of the serving loop's steady state
    for _ in range(2 * ie.engine.graph_after + 2):
        if ie.engine.graph_replays > 0:
            break
        loop.step()
    for _ in range(warmup):
        loop.step()
    ctx0 = sum(r.seq.length for r in reqs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loop.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.seq.length for r in reqs)
    assert all(not r.error for r in reqs), [r.error for r in reqs if r.error][:1]
    assert ctx1 - ctx0 == batch * steps
    for r in reqs:
        r.cancelled = True
    loop.run_loop()
    return batch * steps / dt, dt / steps * 1000.0, (ctx0 + ctx1) / 2.0


def decode_point(engine_factory, shape, layers, batch, steps, warmup, prompt_len, el, warm_up_sizes=None):
    """A decode measurement as a record: tokens a second, ms a step, and the step against the HBM roofline."""
    tps, ms_step, ctx_mid = measure_decode(engine_factory, batch, steps, warmup, shape["vocab_size"], prompt_len,
                                           warm_up_sizes=warm_up_sizes)
    achieved = decode_bytes(shape, layers, batch, ctx_mid, el) / (ms_step / 1000.0) / 1e9
    return {"value": round(tps, 2), "unit": "tok/s", "ms_per_step": round(ms_step, 4), "batch": batch, "seq_len": prompt_len,
            "steps": steps, "roofline_achieved_gbs": round(achieved, 1), "roofline_frac": round(achieved / HBM_PEAK_GBS, 4)}


def long_context_points(base_engine, shape, layers, el, args, contexts=(16384, 32768), batch=8):
    """Decode at batch 8 with prompts of 16,384 and 32,768 tokens (the cache of the live requests is then most of
    what a step reads), on another cache pool of an engine that holds the weights already."""
    import torch
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.parts.rows import many_rows as many_rows_size_at_least
    out = {}
    steps, warm = min(args.steps, 32), min(args.warmup, 8)
    for ctx in contexts:
        gc.collect()
        torch.cuda.empty_cache()
        tokens = ctx + warm + steps + 2 * batch + 64

        def make():
            return base_engine().with_cache(SchedulerConfig(
                num_kv_blocks=batch * (-(-tokens // 16)) + 16, kv_block_size=16, max_batch_requests=batch,
                max_batch_tokens=ctx + batch, max_prefill_tokens=ctx, max_seq_len=2 * ctx))
        out[f"decode_b{batch}_ctx{ctx}"] = decode_point(make, shape, layers, batch, steps, warm, ctx, el,
                                                         warm_up_sizes=[many_rows_size_at_least(ctx + 64), ctx])
    return out


def measure_mix(engine_factory, requests, vocab, new_tokens=256, lo=128, hi=4096):
    """Continuous batching: `requests` prompts of lengths uniform in [lo, hi], all queued at once,
    `new_tokens` greedy tokens each; generated tokens a second over the whole run, prompt tokens a
    second, and the wall time (reference: examples/batch_bench.cpp:168-171)."""
    import torch
    from zedinfer_amd import GenerationConfig, InferenceRequest
    from zedinfer_amd.engine import InferenceEngine
    # every size's choices measured before the clock starts: the figure is a server's steady state (left to itself
    # the engine measures a size when its first step comes, which a long run does not notice and this one would)
    ie = InferenceEngine(engine_factory(), warm_up_sizes="all", freeze_gc=True)
    loop = ie.serving_loop()
    rng = random.Random(4321)
    warm = loop.submit_async(InferenceRequest(rand_ids(rng, hi, vocab), GenerationConfig(max_new_tokens=8, ignore_eos=True)))
    loop.run_loop()
    assert not warm.error, warm.error
    lens = [rng.randint(lo, hi) for _ in range(requests)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reqs = [loop.submit_async(InferenceRequest(rand_ids(rng, n, vocab),
                                               GenerationConfig(max_new_tokens=new_tokens, ignore_eos=True))) for n in lens]
    loop.run_loop()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert all(not r.error and len(r.output_ids) == new_tokens for r in reqs), [r.error for r in reqs if r.error][:1]
    return requests * new_tokens / dt, sum(lens) / dt, dt, sum(lens)


def measure_prefill(engine_factory, vocab, rounds=3, tokens=PROMPT, warm=2):
    import torch
    from zedinfer_amd import ops
    from zedinfer_amd.engine import StepEntry
    eng = engine_factory()
    # which of two equivalent orientations the library's gate/up product takes at this many rows is
    # measured here, before the clock starts, and reported with the result
    rows = eng.model.step_rows(tokens, "mixed")      # the step runs padded to this many rows
    CHOICES.update({" ".join(str(x) for x in k): v for k, v in eng.warm_up([rows]).items()
                    if len(k) > 1 and k[1] == rows})          # this step's own; a serving engine holds one set a size
    rng = random.Random(77)
    times = []
    for i in range(rounds + warm):
        seq = eng.open(("prefill", i), tokens)
        ids = rand_ids(rng, tokens, vocab)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.step([StepEntry(seq, ids, [tokens - 1])], copy=False)
        ops.argmax(logits).tolist()
        times.append(time.perf_counter() - t0)
        eng.close(seq)
    return sum(times[warm:]) / rounds * 1000.0


def further_7b(args):
    """Decode at batch 8 (2,048-token prompts) and 64 requests batched continuously, at the Qwen2.5-7B sizes:
    each figure with its sizes and, for the decode step, its fraction of the HBM roofline."""
    import torch
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine
    shape = dict(SHAPE, **SHAPES["7B"])
    cfg = Qwen2Config.from_dict(shape)
    L, el, batch, steps, warm = shape["num_hidden_layers"], 2, 8, min(args.steps, 48), min(args.warmup, 8)
    holder = {}

    def decode_engine():
        tokens = PROMPT + warm + steps + 2 * batch + 64
        sched = SchedulerConfig(num_kv_blocks=batch * (-(-tokens // 16)) + 16, kv_block_size=16, max_batch_requests=batch,
                                max_batch_tokens=PROMPT + batch, max_prefill_tokens=PROMPT, max_seq_len=8192)
        holder["e"] = Engine.from_config(cfg, "Qwen2ForCausalLM", args.dtype, seed=0, sched=sched)
        return holder["e"]
    tps, ms_step, ctx_mid = measure_decode(decode_engine, batch, steps, warm, cfg.vocab_size, PROMPT)
    need = decode_bytes(shape, L, batch, ctx_mid, el)
    achieved = need / (ms_step / 1000.0) / 1e9
    res = {"config": {"model": "Qwen2.5-7B shape", "num_layers": L, "layers_run": L, "hidden": cfg.hidden_size,
                      "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                      "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "tied_head": False,
                      "kv_page_tokens": 16, "context_len": 8192, "dtype": args.dtype},
           "decode_b8": {"value": round(tps, 2), "unit": "tok/s", "ms_per_step": round(ms_step, 4), "seq_len": PROMPT,
                         "steps": steps, "roofline_achieved_gbs": round(achieved, 1),
                         "roofline_frac": round(achieved / HBM_PEAK_GBS, 4)}}

    def mix_engine():
        sched = SchedulerConfig(num_kv_blocks=64 * (-(-(4096 + 256 + 64) // 16)) + 16, kv_block_size=16,
                                max_batch_requests=64, max_batch_tokens=2048 + 64, max_prefill_tokens=2048, max_seq_len=8192)
        return holder["e"].with_cache(sched)
    res["long_context"] = long_context_points(lambda: holder["e"], shape, L, el, args)
    gen, pre, secs, ptoks = measure_mix(mix_engine, 64, cfg.vocab_size)
    res["mix64"] = {"value": round(gen, 1), "unit": "generated tok/s", "requests": 64, "prompt_tokens": ptoks,
                    "prompt_lens": "uniform 128..4096", "new_tokens_each": 256, "prefill_chunk": 2048,
                    "seconds": round(secs, 3), "prompt_tok_s": round(pre, 1)}
    return res


def further_32b(args):
    """Decode at batch 8, 1 and 64 with 8,192-token prompts and the prefill of one 16,384-token prompt in one step, at
    the Qwen2.5-32B sizes (64 layers, 65 GB of weights; batch 64 holds 139 GB of keys and values and takes half a
    minute to prefill; reference method: examples/batch_bench.cpp:101-180)."""
    import torch
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine
    shape = dict(SHAPE, **SHAPES["32B"])
    cfg = Qwen2Config.from_dict(shape)
    L, el, batch, prompt, long_prompt = shape["num_hidden_layers"], 2, 8, 8192, 16384
    steps, warm = min(args.steps, 24), min(args.warmup, 4)
    holder = {}

    def decode_engine():
        tokens = prompt + warm + steps + 2 * batch + 64
        sched = SchedulerConfig(num_kv_blocks=batch * (-(-tokens // 16)) + 16, kv_block_size=16, max_batch_requests=batch,
                                max_batch_tokens=prompt + batch, max_prefill_tokens=prompt, max_seq_len=2 * prompt)
        holder["e"] = Engine.from_config(cfg, "Qwen2ForCausalLM", args.dtype, seed=0, sched=sched)
        return holder["e"]
    # the prompts enter whole, alone or beside the requests that decode already: the two sizes of such steps
    from zedinfer_amd.parts.rows import many_rows as many_rows_size_at_least
    tps, ms_step, ctx_mid = measure_decode(decode_engine, batch, steps, warm, cfg.vocab_size, prompt,
                                           warm_up_sizes=[many_rows_size_at_least(prompt + 64), prompt])
    need = decode_bytes(shape, L, batch, ctx_mid, el)
    achieved = need / (ms_step / 1000.0) / 1e9
    res = {"config": {"model": "Qwen2.5-32B shape", "num_layers": L, "layers_run": L, "hidden": cfg.hidden_size,
                      "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                      "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "tied_head": False,
                      "kv_page_tokens": 16, "context_len": 2 * prompt, "dtype": args.dtype},
           "decode_b8": {"value": round(tps, 2), "unit": "tok/s", "ms_per_step": round(ms_step, 4), "seq_len": prompt,
                         "steps": steps, "roofline_achieved_gbs": round(achieved, 1),
                         "roofline_frac": round(achieved / HBM_PEAK_GBS, 4)}}
    torch.cuda.empty_cache()
    one, _, _ = measure_decode(lambda: holder["e"].with_cache(SchedulerConfig(
        num_kv_blocks=(prompt + warm + steps + 128) // 16 + 16, kv_block_size=16, max_batch_requests=1,
        max_batch_tokens=prompt + 1, max_prefill_tokens=prompt, max_seq_len=2 * prompt)), 1, steps, warm, cfg.vocab_size,
        prompt, warm_up_sizes=[prompt])
    res["decode_b1"] = {"value": round(one, 2), "unit": "tok/s", "seq_len": prompt}
    gc.collect()
    torch.cuda.empty_cache()
    many, st64 = 64, min(args.steps, 16)
    tokens64 = prompt + warm + st64 + 2 * many + 64
    if many * tokens64 * 2 * L * cfg.num_key_value_heads * cfg.head_dim * el <= 0.9 * torch.cuda.mem_get_info()[0]:
        res["decode_b64"] = decode_point(lambda: holder["e"].with_cache(SchedulerConfig(
            num_kv_blocks=many * (-(-tokens64 // 16)) + 16, kv_block_size=16, max_batch_requests=many,
            max_batch_tokens=prompt + many, max_prefill_tokens=prompt, max_seq_len=2 * prompt)), shape, L, many, st64, warm,
            prompt, el, warm_up_sizes=[many_rows_size_at_least(prompt + 64), prompt, many])
    else:
        res["decode_b64"] = None        # the requests' keys and values do not fit beside the weights
    gc.collect()
    torch.cuda.empty_cache()

    def prefill_engine():
        sched = SchedulerConfig(num_kv_blocks=long_prompt // 16 + 16, kv_block_size=16, max_batch_requests=1,
                                max_batch_tokens=long_prompt + 1, max_prefill_tokens=long_prompt, max_seq_len=2 * long_prompt)
        return holder["e"].with_cache(sched)
    pms = measure_prefill(prefill_engine, cfg.vocab_size, rounds=2, tokens=long_prompt)
    fl = prefill_flops(shape, L, long_prompt)
    res["prefill_16384"] = {"value": round(long_prompt / pms * 1000.0, 1), "unit": "tok/s", "tokens": long_prompt,
                            "ms": round(pms, 2), "frac": round(fl / (pms / 1000.0) / MFMA_PEAK[args.dtype], 4)}
    return res


STAMP_NAMES = {0: "start", 1: "normed", 2: "q/k/v product done", 3: "at barrier 1", 4: "past barrier 1",
               5: "attention done, at barrier 2", 6: "past barrier 2", 13: "attention's output in LDS",
               7: "output product done, at barrier 3", 8: "past barrier 3", 12: "normed residual in LDS",
               9: "gate/up done, at barrier 4", 10: "past barrier 4", 14: "activation in LDS", 11: "end"}
STAMP_ORDER = [0, 1, 2, 3, 4, 5, 6, 13, 7, 8, 12, 9, 10, 14, 11]


def resident_layer_probe(args, shape):
    """Times ops.decode_layer (one launch a decoder layer) alone: `layers` layers of distinct random weights, one
    launch each, replayed as a graph, for `batch` requests at position `prompt_len`.  A library built with
    -DDL_TIMING also leaves the clock at the phases of the last launch; their spread over the workgroups is printed
    to stderr."""
    import math

    import torch
    from zedinfer_amd import ops
    n, ctx, L = args.batch, args.prompt_len, args.layers
    H, I = shape["hidden_size"], shape["intermediate_size"]
    nh, nkv = shape["num_attention_heads"], shape["num_key_value_heads"]
    d, ps, bt, dev = H // nh, 16, torch.bfloat16, "cuda"
    Qd, KVd = nh * d, nkv * d
    max_keys = ctx + 64
    if not ops.decode_layer_supported(bt, n, H, I, nh, nkv, d, d, ps, max_keys, 0):
        print(json.dumps({"resident_layer": None, "why": "the kernel does not take this shape"}))
        return 0
    W = [dict(wqkv=torch.randn(Qd + 2 * KVd, H, device=dev, dtype=bt) * 0.02, bias=torch.randn(Qd + 2 * KVd, device=dev, dtype=bt) * 0.1,
              wo=torch.randn(H, Qd, device=dev, dtype=bt) * 0.02, wgu=torch.randn(2 * I, H, device=dev, dtype=bt) * 0.02,
              wd=torch.randn(H, I, device=dev, dtype=bt) * 0.01, g=torch.ones(H, device=dev, dtype=bt)) for _ in range(L)]
    pages_each = -(-(ctx + 64) // ps)
    num_pages = n * pages_each + 1
    caches = [(torch.randn(num_pages, nkv, ps, d, device=dev, dtype=bt), torch.randn(num_pages, nkv, d, ps, device=dev, dtype=bt))
              for _ in range(L)]
    table = (torch.arange(n * pages_each, dtype=torch.int32).view(n, pages_each) + 1).to(dev)
    pos = torch.full((n,), ctx, dtype=torch.int32, device=dev)
    slots = (table[:, ctx // ps].long() * ps + ctx % ps).to(torch.int32)
    ws = torch.empty(ops.decode_layer_workspace(n, H, I, nh, nkv, d, max_keys, 0), dtype=torch.uint8, device=dev)
    words = ops.decode_layer_sync_words()
    sync = torch.zeros(words, dtype=torch.int32, device=dev)
    err = torch.zeros(1, dtype=torch.int32).pin_memory()
    rope = ops.rope_table(pos, ops.rope_inv_freq(d, shape["rope_theta"], torch.device(dev)))
    resid = torch.randn(n, H, device=dev)

    def step():
        for w, (kc, vc) in zip(W, caches):
            ops.decode_layer(resid, w["g"], w["g"], 1e-6, 1e-6, False, w["wqkv"], w["bias"], w["wo"], w["wgu"], w["wd"], rope,
                             slots, kc, vc, pos, table, nh, nkv, d, 1 / math.sqrt(d), max_keys, 0, ws, sync, err)
    step()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for _ in range(max(args.warmup, 1)):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        g.replay()
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) / args.steps * 1e6
    weights = L * 2 * ((Qd + 2 * KVd) * H + H * Qd + 3 * I * H)
    cache = L * n * ctx * 2 * KVd * 2
    print(json.dumps({"resident_layer": {"us_per_layer": round(us / L, 2), "us_per_step": round(us, 1), "layers": L,
                                         "batch": n, "context": ctx, "shape": args.shape,
                                         "GB/s": round((weights + cache) / us / 1e3, 1), "wait_ran_out": int(err[0])}}))
    stamps = ops.decode_layer_stamps()
    if stamps:
        st = sync[words - 256 * 2 * stamps:].view(torch.int64).view(256, stamps).cpu().double()
        rel = (st - st[:, 0].min()) / 100.0           # the clock runs at 100 MHz: microseconds
        for i in STAMP_ORDER:
            col = rel[:, i][st[:, i] > 0]
            if col.numel():
                print(f"{STAMP_NAMES[i]:36s} first {col.min():7.2f}  median {col.median():7.2f}  last {col.max():7.2f} us",
                      file=sys.stderr)
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the model has (reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--shape", default="1.5B", choices=sorted(SHAPES), help="layer sizes of Qwen2.5-<shape>")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="tokens every decoding request holds at the start")
    ap.add_argument("--prefill-len", type=int, default=PROMPT, help="tokens of the timed prefill")
    ap.add_argument("--mix", type=int, default=0, metavar="R",
                    help="instead: continuous batching of R requests, prompts uniform in [128, 4096], 256 greedy "
                         "tokens each, prompts cut at 2,048 tokens a step")
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 / 128 / 256 points")
    ap.add_argument("--no-further", action="store_true", help="skip the figures at the 7B and 32B sizes")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiling) and print its figures")
    ap.add_argument("--resident-layer", action="store_true",
                    help="instead: time the one-launch decoder layer (ops.decode_layer) alone, --layers launches a step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine

    full_layers = SHAPES[args.shape].get("num_hidden_layers", FULL_LAYERS)
    if args.layers == FULL_LAYERS and args.shape != "1.5B":
        args.layers = full_layers
    shape = dict(SHAPE, **SHAPES[args.shape])
    shape["num_hidden_layers"] = args.layers
    if args.resident_layer:
        return resident_layer_probe(args, shape)
    cfg = Qwen2Config.from_dict(shape)
    el = 2 if args.dtype == "bf16" else 4
    weights_cache = {}

    def factory(batch, prompt=args.prompt_len):
        def make():
            context = max(CONTEXT, 2 * prompt)
            # pages for what the requests will hold, not for the whole context: 64 long requests must fit
            tokens = min(context, prompt + args.warmup + args.steps + 2 * batch + 64)
            pages = batch * (-(-tokens // 16)) + 16
            sched = SchedulerConfig(num_kv_blocks=pages, kv_block_size=16, max_batch_requests=max(batch, 1),
                                    max_batch_tokens=prompt + batch, max_prefill_tokens=prompt, max_seq_len=context)
            if "w" not in weights_cache:
                e = Engine.from_config(cfg, "Qwen2ForCausalLM", args.dtype, seed=0, sched=sched)
                weights_cache["w"] = e
                return e
            # share the first engine's weights: same model, another cache pool
            return weights_cache["w"].with_cache(sched)
        return make

    V = cfg.vocab_size
    PF = args.prefill_len
    if args.mix:
        def mix_engine():
            sched = SchedulerConfig(num_kv_blocks=args.mix * (-(-(4096 + 256 + 64) // 16)) + 16, kv_block_size=16,
                                    max_batch_requests=args.mix, max_batch_tokens=2048 + args.mix,
                                    max_prefill_tokens=2048, max_seq_len=8192)
            return Engine.from_config(cfg, "Qwen2ForCausalLM", args.dtype, seed=0, sched=sched)
        gen, pre, secs, ptoks = measure_mix(mix_engine, args.mix, V)
        print(json.dumps({"metric": f"continuous batching, generated tok/s (Qwen2.5-{args.shape} shape)",
                          "value": round(gen, 1), "unit": "tok/s", "requests": args.mix, "prompt_tokens": ptoks,
                          "new_tokens_each": 256, "seconds": round(secs, 3), "prompt_tok_s": round(pre, 1),
                          "dtype": args.dtype, "layers_run": args.layers, "num_layers": full_layers}))
        return 0
    if args.prefill_only:
        pms = measure_prefill(factory(1, PF), V, tokens=PF)
        fl = prefill_flops(shape, args.layers, PF)
        print(json.dumps({"prefill": {"value": round(PF / pms * 1000.0, 1), "tokens": PF, "ms": round(pms, 3),
                                      "frac": round(fl / (pms / 1000.0) / MFMA_PEAK[args.dtype], 4)},
                          "choices": CHOICES}))
        return 0
    tps, ms_step, ctx_mid = measure_decode(factory(args.batch), args.batch, args.steps, args.warmup, V, args.prompt_len)
    need = decode_bytes(shape, args.layers, args.batch, ctx_mid, el)
    achieved = need / (ms_step / 1000.0) / 1e9
    out = {
        "metric": f"decode tok/s at batch {args.batch}, {args.prompt_len:,}-token prompts (Qwen2.5-{args.shape} shape)",
        "value": round(tps, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: seeded random weights, seeded uniform-random token ids",
        "config": {"model": f"Qwen2.5-{args.shape} shape", "global_batch": args.batch, "seq_len": args.prompt_len,
                   "context_len": max(CONTEXT, 2 * args.prompt_len), "parallelism": "single GPU", "num_layers": full_layers,
                   "layers_run": args.layers, "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "tied_head": bool(shape["tie_word_embeddings"]),
                   "kv_page_tokens": 16, "sampling": "greedy"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        torch.cuda.empty_cache()
        pms = measure_prefill(factory(1, PF), V, tokens=PF)
        fl = prefill_flops(shape, args.layers, PF)
        out["prefill"] = {"value": round(PF / pms * 1000.0, 1), "tokens": PF, "ms": round(pms, 3),
                          "frac": round(fl / (pms / 1000.0) / MFMA_PEAK[args.dtype], 4)}
        points = {}
        per_token = 2 * args.layers * cfg.num_key_value_heads * cfg.head_dim * el      # cache bytes of one token
        for b, st in ((1, min(args.steps, 64)), (64, min(args.steps, 32)), (128, min(args.steps, 24)), (256, min(args.steps, 16))):
            gc.collect()
            torch.cuda.empty_cache()
            tokens = args.prompt_len + args.warmup + args.steps + 2 * b + 64
            if b * tokens * per_token > 0.9 * torch.cuda.mem_get_info()[0]:
                points[f"decode_b{b}"] = None       # the requests' keys and values do not fit beside the weights
                continue
            t, _, _ = measure_decode(factory(b), b, st, min(args.warmup, 8), V, args.prompt_len)
            points[f"decode_b{b}"] = round(t, 2)
        # the reference's own short run (its bench -p 128): a prompt step of this size replays as a graph
        # from its third time on, so two steps warm up
        torch.cuda.empty_cache()
        short = measure_prefill(factory(1, 128), V, tokens=128, warm=2)
        points["prefill_128"] = round(128 / short * 1000.0, 1)
        out["points"] = points
        def flat(prefix, results):
            """Further measurements as flat numbers of `points` (what is deeper is lost in the record)."""
            for name, r in results.items():
                if isinstance(r, dict) and "value" in r:
                    points[prefix + name] = r["value"]
                    if "roofline_frac" in r:
                        points[prefix + name + "_roofline_frac"] = r["roofline_frac"]
        if not args.no_further:
            out["long_context"] = long_context_points(lambda: weights_cache["w"], shape, args.layers, el, args)
            flat("", out["long_context"])
        if args.shape == "1.5B" and args.layers == FULL_LAYERS and not args.no_further:
            # the same architecture at the Qwen2.5-7B sizes: decode at batch 8 and the continuous-batching mix
            weights_cache.clear()
            torch.cuda.empty_cache()
            out["further"] = further_7b(args)
            flat("7b_", out["further"].get("long_context", {}))
            flat("7b_", {k: v for k, v in out["further"].items() if k != "long_context"})
            gc.collect()
            torch.cuda.empty_cache()
            out["further_32b"] = further_32b(args)
            flat("32b_", out["further_32b"])
    out["choices"] = CHOICES
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
