"""Generation through the entry points: greedy tokens against the plain implementation, continuous
batching with chunked prefill, sampling against the plain sampler, the command lines."""
import os
import subprocess
import sys

import pytest
import torch

import tiny_configs
import traces
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module", params=["A", "B"])
def tiny(request, tmp_path_factory):
    name = request.param
    folder = tiny_configs.write_tiny(str(tmp_path_factory.mktemp(f"gen{name}")), name)
    cfg, w = plain.load_folder(folder)
    return dict(name=name, folder=folder, cfg=cfg, weights=w)


def engine(tiny, dtype="float32", **kw):
    from zedinfer_amd import InferenceEngine, SchedulerConfig
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    sc = dict(num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4)
    sc.update(kw)
    return InferenceEngine.create(tiny["folder"], dtype, SchedulerConfig(**sc))


def test_greedy_generation_matches_plain(tiny):
    """The tiny workloads: prompts of 5/17/33 tokens (A) and 1/31/64/100 (B), 16 greedy tokens each."""
    from zedinfer_amd import GenerationConfig
    lens = [5, 17, 33] if tiny["name"] == "A" else [1, 31, 64, 100]
    V = tiny["cfg"]["vocab_size"]
    ie = engine(tiny)
    for i, n in enumerate(lens):
        prompt = traces.random_tokens(V, n, seed=i)
        want = plain.greedy_generate(tiny["cfg"], tiny["weights"], prompt, 16)
        res = ie.generate_tokens(prompt, GenerationConfig(max_new_tokens=16, ignore_eos=True))
        assert res.output_ids == want and res.finish_reason == "length"
        assert res.stats.prompt_tokens == n and res.stats.generated_tokens == 16
    assert not ie.engine.cache.live


def test_window_ignored_gives_full_attention_logits(tmp_path, monkeypatch):
    """With ZEDINFER_IGNORE_SLIDING_WINDOW a configuration that asks for a window attends over all keys,
    which is what the reference computes for it; the plain implementation without a window agrees."""
    from zedinfer_amd.engine import StepEntry
    monkeypatch.setenv("ZEDINFER_IGNORE_SLIDING_WINDOW", "1")
    folder = tiny_configs.write_tiny(str(tmp_path / "c"), "C")
    cfg, w = plain.load_folder(folder)
    toks = traces.random_tokens(cfg["vocab_size"], 70, seed=9)
    ref = plain.forward(dict(cfg, use_sliding_window=False), w, toks)
    windowed = plain.forward(cfg, w, toks)
    assert float((ref[40:] - windowed[40:]).abs().max()) > 1e-3
    e = engine(dict(name="C", folder=folder)).engine
    assert len(e.cache.groups) == 1 and e.cache.groups[0].kind == "full"
    s = e.open("r")
    got = torch.cat([e.step([StepEntry(s, toks[:50], list(range(50)))]),
                     *[e.step([StepEntry(s, [t], [0])]) for t in toks[50:]]]).cpu()
    assert float((got - ref).abs().max()) < 2e-4


def test_continuous_batching_equals_one_by_one(tiny):
    """Chunked prefill (24 tokens a step) mixed with decoding of earlier requests gives every request
    the tokens it gets alone."""
    from zedinfer_amd import GenerationConfig
    lens = [1, 31, 64, 100, 7, 50]
    V = tiny["cfg"]["vocab_size"]
    prompts = [traces.random_tokens(V, n, seed=10 + i) for i, n in enumerate(lens)]
    ie = engine(tiny, max_prefill_tokens=24, max_batch_tokens=32, max_batch_requests=3)
    results = ie.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))
    for prompt, res in zip(prompts, results):
        assert res.output_ids == plain.greedy_generate(tiny["cfg"], tiny["weights"], prompt, 12)
    ie.engine.cache.check()
    assert not ie.engine.cache.live and ie.engine.steps_run > 12


def test_long_decoding(tiny):
    """200 tokens decoded one by one from a short prompt: logits at every step against the plain run
    of the final sequence."""
    from zedinfer_amd.engine import StepEntry
    V = tiny["cfg"]["vocab_size"]
    toks = traces.random_tokens(V, 230, seed=5)
    ref = plain.forward(tiny["cfg"], tiny["weights"], toks)
    ie = engine(tiny)
    e = ie.engine
    s = e.open("long")
    got = [e.step([StepEntry(s, toks[:30], list(range(30)))])]
    for t in toks[30:]:
        got.append(e.step([StepEntry(s, [t], [0])]))
    e.close(s)
    got = torch.cat(got).cpu()
    assert float((got - ref).abs().max()) < 2e-4


def test_first_tokens_of_a_sequence(tiny):
    """Position 0 alone, then position 1 alone: the smallest cases of the cache."""
    from zedinfer_amd.engine import StepEntry
    toks = [7, 9, 11]
    ref = plain.forward(tiny["cfg"], tiny["weights"], toks)
    e = engine(tiny).engine
    s = e.open("first")
    for i, t in enumerate(toks):
        lg = e.step([StepEntry(s, [t], [0])]).cpu()
        assert float((lg[0] - ref[i]).abs().max()) < 1e-4
    e.close(s)


def test_stop_token_ends_generation(tiny):
    from zedinfer_amd import GenerationConfig
    prompt = traces.random_tokens(tiny["cfg"]["vocab_size"], 9, seed=3)
    free = plain.greedy_generate(tiny["cfg"], tiny["weights"], prompt, 8)
    ie = engine(tiny)
    ie.serving_loop().scheduler.stop_token_ids = {free[3]}
    res = ie.generate_tokens(prompt, GenerationConfig(max_new_tokens=8))
    first = free.index(free[3])
    assert res.finish_reason == "stop" and res.output_ids == free[:first + 1]


def test_steps_queued_ahead_give_the_same_tokens(tiny):
    """Steps that are queued before the step before them has finished (their decoding requests' tokens are read
    on the device; portions of prompts ride along) against a loop that waits for every step: requests of different lengths, greedy and
    sampled, one that ends on a stop token while a step ahead already computes for it, one that arrives
    while the others decode, and prompts that enter in portions.  Every request gets the same tokens and
    the same reason to end, and no page is lost."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, InferenceRequest, SchedulerConfig
    from zedinfer_amd.engine import ServingLoop
    V = tiny["cfg"]["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    prompts = [traces.random_tokens(V, n, seed=40 + i) for i, n in enumerate([9, 31, 50, 3, 20])]

    def configs():
        return [GenerationConfig(max_new_tokens=30, ignore_eos=True),
                GenerationConfig(max_new_tokens=30),                                    # ends on the stop token
                GenerationConfig(max_new_tokens=17, temperature=0.8, top_k=20, seed=5, ignore_eos=True),
                GenerationConfig(max_new_tokens=2, ignore_eos=True),
                GenerationConfig(max_new_tokens=25, temperature=0.6, top_p=0.9, seed=6, ignore_eos=True)]

    def run(look_ahead, stops):
        ie = InferenceEngine.create(tiny["folder"], "float32", SchedulerConfig(
            num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4, max_prefill_tokens=24, max_batch_tokens=32))
        loop = ServingLoop(ie.engine, stops, look_ahead=look_ahead)
        cf = configs()
        reqs = [loop.submit_async(InferenceRequest(p, c)) for p, c in zip(prompts[:4], cf[:4])]
        for _ in range(9):
            loop.step()
        reqs.append(loop.submit_async(InferenceRequest(prompts[4], cf[4])))     # arrives while the others decode
        loop.run_loop()
        assert all(r.done and not r.error for r in reqs)
        ie.engine.cache.check()
        assert not ie.engine.cache.live
        return [(r.result.output_ids, r.result.finish_reason) for r in reqs], (loop.steps_ahead, loop.prompt_steps_ahead)

    free, _ = run(False, [])
    stop = free[1][0][11]           # a token the second request makes on its way
    want, (none_ahead, _) = run(False, [stop])
    got, (ahead, with_prompts) = run(True, [stop])
    assert none_ahead == 0 and ahead > 10 and with_prompts > 0
    assert want[1][1] == "stop" and len(want[1][0]) <= 12
    assert got == want


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_get_the_same_tokens_with_steps_queued_ahead(tiny, seed):
    """Random requests (prompts from 1 to 200 tokens that enter in portions, greedy and sampled, some that end on
    stop tokens, arriving while others run, few pages so that some wait) through a loop that queues steps ahead and
    one that waits for every step, in 32 bits, where a token's logits do not depend on what else is in its step:
    the same tokens and reasons to end for everyone, and no page lost."""
    import random
    from zedinfer_amd import GenerationConfig, InferenceEngine, InferenceRequest, SchedulerConfig
    from zedinfer_amd.engine import ServingLoop
    V = tiny["cfg"]["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    rng = random.Random(seed)
    lens = [rng.choice([1, 5, 20, 64, 65, 130, 200]) for _ in range(9)]
    prompts = [traces.random_tokens(V, n, seed=seed * 50 + i) for i, n in enumerate(lens)]
    cfgs = [dict(max_new_tokens=rng.randint(1, 30), ignore_eos=rng.random() < 0.7, temperature=rng.choice([0.0, 0.0, 0.8]),
                 top_k=rng.choice([0, 10]), seed=rng.randint(1, 99)) for _ in lens]
    arrive = sorted(rng.randrange(0, 25) for _ in lens)
    sched = dict(num_kv_blocks=rng.choice([60, 90, 200]) * 16 // ps, kv_block_size=ps, max_batch_requests=rng.choice([2, 4, 8]),
                 max_prefill_tokens=rng.choice([24, 64, 512]), max_batch_tokens=rng.choice([72, 128, 520]), generation_reserve=32)
    outs, ahead = [], None
    for look_ahead in (False, True):
        ie = InferenceEngine.create(tiny["folder"], "float32", SchedulerConfig(**sched))
        loop = ServingLoop(ie.engine, [7, 11, 13], look_ahead=look_ahead)
        reqs, step, todo = [], 0, list(zip(arrive, prompts, cfgs))
        while todo or loop.scheduler.has_work():
            while todo and todo[0][0] <= step:
                _, p, c = todo.pop(0)
                reqs.append(loop.submit_async(InferenceRequest(p, GenerationConfig(**c))))
            loop.step()
            step += 1
            assert step < 5000
        ie.engine.cache.check()
        assert not ie.engine.cache.live
        outs.append([(r.error, r.result.finish_reason if r.result else None, r.result.output_ids if r.result else None)
                     for r in reqs])
        ahead = loop.steps_ahead
    assert ahead > 0 and outs[0] == outs[1]


def test_steps_queued_ahead_without_graphs(tiny, monkeypatch):
    """The same with decode steps launched kernel by kernel (no graphs): the tokens of a step queued
    ahead are copied into the step's batch on the device."""
    from zedinfer_amd import GenerationConfig
    monkeypatch.setenv("ZEDINFER_DISABLE_GRAPHS", "1")
    V = tiny["cfg"]["vocab_size"]
    prompts = [traces.random_tokens(V, n, seed=60 + i) for i, n in enumerate([9, 31, 3])]
    ie = engine(tiny)
    assert not ie.engine.use_graphs
    results = ie.generate(prompts, GenerationConfig(max_new_tokens=14, ignore_eos=True))
    assert ie.serving_loop().steps_ahead > 5 and ie.engine.graph_replays == 0
    for p, r in zip(prompts, results):
        assert r.output_ids == plain.greedy_generate(tiny["cfg"], tiny["weights"], p, 14)


def test_steps_queued_ahead_with_the_serving_kernels(tiny, tmp_path):
    """A bfloat16 checkpoint, greedy, steps queued ahead and replayed as graphs: every token a request
    gets is the best, or within rounding of the best, at its place in the plain run of its sequence."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, InferenceRequest, SchedulerConfig
    V = tiny["cfg"]["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    folder = tiny_configs.write_tiny(str(tmp_path), tiny["name"], dtype=torch.bfloat16)
    cfg, w = plain.load_folder(folder)
    prompts = [traces.random_tokens(V, n, seed=50 + i) for i, n in enumerate([9, 31, 3])]
    ie = InferenceEngine.create(folder, "bfloat16", SchedulerConfig(num_kv_blocks=64, kv_block_size=ps,
                                                                    max_batch_requests=4))
    loop = ie.serving_loop()
    reqs = [loop.submit_async(InferenceRequest(p, GenerationConfig(max_new_tokens=n, ignore_eos=True)))
            for p, n in zip(prompts, (24, 17, 30))]
    loop.run_loop()
    assert loop.steps_ahead > 10 and ie.engine.graph_replays > 10
    for p, r in zip(prompts, reqs):
        out = r.result.output_ids
        assert len(out) == r.config.max_new_tokens
        ref = plain.forward(cfg, w, p + out[:-1])
        for i, t in enumerate(out):
            row = ref[len(p) - 1 + i]
            assert float(row.max() - row[t]) <= 0.03 * float(row.abs().max()), (i, t, int(row.argmax()))
    ie.engine.cache.check()
    assert not ie.engine.cache.live


@pytest.mark.parametrize("seed", [0, 1])
def test_requests_arriving_and_cancelled_while_the_loop_runs(tiny, seed):
    """Requests of random lengths arrive while others decode, a pool so small that admission has to
    wait for pages, some requests cancelled on the way: every request that finishes has the tokens it
    gets alone, a cancelled one a prefix of them, and every page and slot is back at the end."""
    import random
    from zedinfer_amd import GenerationConfig, InferenceRequest
    rng = random.Random(100 + seed)
    V = tiny["cfg"]["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    ie = engine(tiny, num_kv_blocks=(160 + 16) // ps + 6, max_prefill_tokens=24, max_batch_tokens=40,
                max_batch_requests=4, generation_reserve=16)      # the reserve covers every request's new tokens: admission waits, nothing fails
    loop = ie.serving_loop()
    todo = []
    for i in range(18):
        prompt = traces.random_tokens(V, rng.choice([1, 2, 3, 9, 17, 33, 48, 70]), seed=200 + 50 * seed + i)
        todo.append((rng.randrange(0, 40), prompt, rng.randrange(1, 15)))
    todo.sort(key=lambda x: x[0])
    cancel_at = {3: rng.randrange(5, 30), 8: rng.randrange(10, 45), 12: rng.randrange(20, 60)}
    reqs, step = [], 0
    while todo or loop.scheduler.has_work():
        while todo and todo[0][0] <= step:
            _, prompt, n = todo.pop(0)
            reqs.append(loop.submit_async(InferenceRequest(prompt, GenerationConfig(max_new_tokens=n, ignore_eos=True))))
        for i, at in cancel_at.items():
            if at == step and i < len(reqs):
                reqs[i].cancelled = True
        loop.step()
        step += 1
        assert step < 2000
    assert len(reqs) == 18 and loop.steps_ahead > 0
    finished = 0
    for i, q in enumerate(reqs):
        assert q.done and q.error is None, (i, q.error)
        want = plain.greedy_generate(tiny["cfg"], tiny["weights"], q.input_ids, q.config.max_new_tokens)
        if q.cancelled and len(q.output_ids) < len(want):
            assert q.output_ids == want[:len(q.output_ids)], i
        else:
            assert q.output_ids == want, i
            finished += 1
    assert finished >= 15
    ie.engine.cache.check()
    assert not ie.engine.cache.live


def test_out_of_pages_fails_the_request_not_the_engine(tiny):
    from zedinfer_amd import GenerationConfig
    ie = engine(tiny, num_kv_blocks=4)
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    with pytest.raises(RuntimeError, match="Cannot admit"):
        ie.generate_tokens(list(range(1, 5 * ps)), GenerationConfig(max_new_tokens=4))
    res = ie.generate_tokens([1, 2, 3], GenerationConfig(max_new_tokens=4, ignore_eos=True))
    assert len(res.output_ids) == 4


def test_sampling_kernel_against_plain_sampler():
    """Same logits, same uniform draw: the kernel picks the token the plain sorted-order sampler picks."""
    from zedinfer_amd import ops
    g = torch.Generator().manual_seed(0)
    V = 1000
    cases = [(1.0, 0, 1.0, 1.0), (0.7, 0, 1.0, 1.0), (0.7, 5, 1.0, 1.0), (1.3, 0, 0.8, 1.0), (0.9, 50, 0.5, 1.0),
             (1.0, 1, 1.0, 1.0), (0.01, 0, 1.0, 1.0), (1.0, 0, 0.05, 1.0), (0.8, 20, 0.9, 1.7)]
    rows, params, us, hist = [], [], [], []
    for ci, c in enumerate(cases):
        for r in range(12):
            rows.append(torch.randn(V, generator=g) * 2.5)
            params.append(c)
            us.append(float(torch.rand((), generator=g)))
            hist.append([int(x) for x in torch.randint(0, V, (6,), generator=g)] + [int(rows[-1].argmax())] * 2)
    logits = torch.stack(rows).cuda()
    R = len(rows)
    dev = lambda v, dt: torch.tensor(v, dtype=dt, device="cuda")  # noqa: E731
    recent = torch.tensor(hist, dtype=torch.int32, device="cuda")
    out = ops.sample(logits, dev([p[0] for p in params], torch.float32), dev([p[1] for p in params], torch.int32),
                     dev([p[2] for p in params], torch.float32), dev([p[3] for p in params], torch.float32),
                     dev(us, torch.float32), recent, dev([len(h) for h in hist], torch.int32)).tolist()
    mismatches = 0
    for i in range(R):
        T, k, p, pen = params[i]
        probs, idx = plain.truncated_distribution(rows[i], T, k, p, pen, hist[i])
        c = torch.cumsum(probs, 0)
        hit = (us[i] < c).nonzero()
        want = int(idx[int(hit[0])] if len(hit) else idx[-1])
        assert out[i] in idx.tolist(), f"row {i}: token {out[i]} is outside the kept set"
        mismatches += out[i] != want
    assert mismatches == 0
    # top_k = 1, a tiny top_p and a tiny temperature are all argmax (reference: tests/sampler/test_sampler.cpp:157-202)
    am = torch.argmax(logits, -1).tolist()
    for i, c in enumerate(params):
        if c in [(1.0, 1, 1.0, 1.0), (0.01, 0, 1.0, 1.0)]:
            assert out[i] == am[i]


def test_sampling_in_the_engine_is_seeded_per_request(tiny):
    """Temperature 0.7 with a fixed seed: the same request samples the same tokens alone and in a
    mixed batch with chunked prefill; another seed gives other tokens."""
    from zedinfer_amd import GenerationConfig, InferenceRequest
    V = tiny["cfg"]["vocab_size"]
    prompts = [traces.random_tokens(V, n, seed=20 + i) for i, n in enumerate([1, 31, 64, 100])]
    cfg = lambda s: GenerationConfig(max_new_tokens=10, temperature=0.7, seed=s, ignore_eos=True)  # noqa: E731
    alone = [engine(tiny).generate_tokens(p, cfg(100 + i)).output_ids for i, p in enumerate(prompts)]
    ie = engine(tiny, max_prefill_tokens=24, max_batch_tokens=40)
    loop = ie.serving_loop()
    reqs = [loop.submit_async(InferenceRequest(p, cfg(100 + i))) for i, p in enumerate(prompts)]
    loop.run_loop()
    assert [r.output_ids for r in reqs] == alone
    other = engine(tiny).generate_tokens(prompts[3], cfg(999)).output_ids
    assert other != alone[3]
    greedy = engine(tiny).generate_tokens(prompts[3], GenerationConfig(max_new_tokens=10, ignore_eos=True)).output_ids
    assert greedy == plain.greedy_generate(tiny["cfg"], tiny["weights"], prompts[3], 10)


def test_generation_config_of_the_model_folder_is_the_default(tiny, tmp_path, monkeypatch):
    """do_sample in the folder's generation_config.json: a request that sets no sampling option samples
    with the file's values, one that asks for argmax is greedy, ZEDINFER_FORCE_ARGMAX makes all greedy
    (reference: src/zedinfer/engine.cpp:49-126, scheduler.cpp:576-600)."""
    import json
    import shutil
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    monkeypatch.delenv("ZEDINFER_FORCE_ARGMAX", raising=False)
    folder = str(tmp_path / "model")
    shutil.copytree(tiny["folder"], folder)
    with open(os.path.join(folder, "generation_config.json"), "w") as f:
        json.dump(dict(do_sample=True, temperature=0.8, top_k=30, seed=9), f)
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    sc = lambda: SchedulerConfig(num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4)  # noqa: E731
    prompt = traces.random_tokens(tiny["cfg"]["vocab_size"], 21, seed=8)
    greedy = plain.greedy_generate(tiny["cfg"], tiny["weights"], prompt, 12)
    ie = InferenceEngine.create(folder, "float32", sc())
    assert ie.default_sampling.temperature == 0.8 and not ie.default_sampling.greedy
    got = ie.generate_tokens(prompt, GenerationConfig(max_new_tokens=12, ignore_eos=True)).output_ids
    own = engine(tiny).generate_tokens(prompt, GenerationConfig(max_new_tokens=12, temperature=0.8, top_k=30, seed=9,
                                                               ignore_eos=True)).output_ids
    assert got == own and got != greedy
    assert ie.generate_tokens(prompt, GenerationConfig(max_new_tokens=12, use_argmax=True, ignore_eos=True)
                              ).output_ids == greedy
    monkeypatch.setenv("ZEDINFER_FORCE_ARGMAX", "1")
    forced = InferenceEngine.create(folder, "float32", sc())
    assert forced.generate_tokens(prompt, GenerationConfig(max_new_tokens=12, ignore_eos=True)).output_ids == greedy


def test_command_lines(tiny, tmp_path):
    env = dict(os.environ, PYTHONPATH=ROOT)
    run = lambda *a: subprocess.run([sys.executable, *a], capture_output=True, text=True, env=env, timeout=300,  # noqa: E731
                                    cwd=str(tmp_path))
    ps = str(tiny_configs.PAGE_SIZES[tiny["name"]])
    prompt = traces.random_tokens(tiny["cfg"]["vocab_size"], 9, seed=3)
    r = run(os.path.join(ROOT, "bin", "ping"), tiny["folder"], "--dtype", "fp32", "--prompt-ids",
            ",".join(map(str, prompt)), "--max-new-tokens", "5", "--ignore-eos", "--num-kv-blocks", "32",
            "--kv-block-size", ps, "--log-file", str(tmp_path / "p.log"), "--log-level", "debug")
    assert r.returncode == 0, r.stderr
    want = plain.greedy_generate(tiny["cfg"], tiny["weights"], prompt, 5)
    assert "output_ids: " + ",".join(map(str, want)) in r.stdout and "finish_reason: length" in r.stdout
    logged = (tmp_path / "p.log").read_text()
    assert "Engine initialized" in logged and "Engine initialized" in r.stderr and "choices made at warm-up" in logged
    r = run(os.path.join(ROOT, "bin", "bench"), tiny["folder"], "-p", "32", "-d", "8", "-r", "1",
            "--num-kv-blocks", "32", "--kv-block-size", ps, "--no-log-to-console")
    assert r.returncode == 0 and "Prefill:" in r.stdout and "tok/s" in r.stdout, r.stderr
    assert "Engine initialized" not in r.stderr and "Engine initialized" in (tmp_path / "logs" / "bench.log").read_text()
    r = run(os.path.join(ROOT, "bin", "bench"), tiny["folder"], "--log-append", "--log-overwrite")
    assert r.returncode == 1 and "mutually exclusive" in r.stderr
    r = run(os.path.join(ROOT, "bin", "batch_bench"), tiny["folder"], "-b", "3", "-p", "20", "-d", "6",
            "--num-kv-blocks", "64", "--kv-block-size", ps, "--random-weights", "--seed", "4")
    assert r.returncode == 0 and "Throughput" in r.stdout and "18 tokens generated" in r.stdout, r.stderr + r.stdout


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16w"])
def test_decode_graphs_replay_what_eager_steps_compute(tiny, dtype, tmp_path):
    """Steps of single decoded tokens are captured as graphs and replayed.  Every replay is checked
    against an engine that launches eagerly, with eager prompt portions, closes and new requests
    (reused pages, other batch sizes) between the replays.  "bfloat16w": a bfloat16 checkpoint, whose
    decode steps take the few-rows products and the one-kernel attention with its per-step table."""
    from zedinfer_amd.engine import StepEntry
    V = tiny["cfg"]["vocab_size"]
    if dtype == "bfloat16w":
        folder16 = tiny_configs.write_tiny(str(tmp_path / "bf16"), tiny["name"], dtype=torch.bfloat16)
        tiny = dict(tiny, folder=folder16, weights=plain.load_folder(folder16)[1])
        dtype = "bfloat16"
    fast, slow = engine(tiny, dtype).engine, engine(tiny, dtype).engine
    assert fast.use_graphs
    fast.graph_after = 2                           # a kind of step is captured the second time it comes
    slow.use_graphs = slow.use_tapes = False       # every step part by part
    toks = {r: traces.random_tokens(V, 150, seed=60 + i) for i, r in enumerate("abcd")}
    fed = {r: 0 for r in toks}
    seqs = {}

    def both(plan):
        """plan: [(request, number of tokens)]; returns the two engines' logits."""
        outs = []
        for eng in (fast, slow):
            entries = []
            for r, n in plan:
                if (eng, r) not in seqs:
                    seqs[(eng, r)] = eng.open(r)
                entries.append(StepEntry(seqs[(eng, r)], toks[r][fed[r]:fed[r] + n], list(range(n))))
            outs.append(eng.step(entries))
        for r, n in plan:
            fed[r] += n
        assert torch.equal(outs[0], outs[1]), plan
        return outs[0]

    both([("a", 20), ("b", 7)])
    for _ in range(6):
        both([("a", 1), ("b", 1)])
    both([("c", 33), ("a", 1)])                 # a mixed step runs eagerly
    for _ in range(5):
        both([("a", 1), ("b", 1), ("c", 1)])
    for eng in (fast, slow):
        eng.close(seqs.pop((eng, "b")))
    both([("d", 40)])                           # takes the pages b gave back
    for _ in range(30):
        both([("a", 1), ("c", 1), ("d", 1)])    # crosses page edges; the same graph serves all of them
    for _ in range(4):
        both([("d", 1)])
    assert fast.graph_replays >= 30 and slow.graph_replays == 0
    # and the replayed logits are the plain implementation's
    last = both([("d", 1)])
    ref = plain.forward(tiny["cfg"], tiny["weights"], toks["d"][:fed["d"]])
    tol = 2e-4 if dtype == "float32" else 0.06 * float(ref.abs().max())
    assert float((last[0].cpu() - ref[fed["d"] - 1]).abs().max()) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16w"])
def test_prompt_portions_replay_as_graphs(tiny, dtype, tmp_path):
    """A step that is one portion of one prompt is padded to a multiple of 64 tokens and, from the third
    step of a shape on, replayed as a graph.  Every step is checked against an engine that launches
    eagerly and does not pad: portions of different lengths that share a graph, alone, two in a step and
    beside decoded tokens, with and without a wanted row, decode steps (graphs of their own) and a step that
    takes no graph between them, and at the end the caches, which
    the padding must not have touched: decoding on gives the plain implementation's logits."""
    from zedinfer_amd.engine import StepEntry
    V = tiny["cfg"]["vocab_size"]
    if dtype == "bfloat16w":
        folder16 = tiny_configs.write_tiny(str(tmp_path / "bf16"), tiny["name"], dtype=torch.bfloat16)
        tiny = dict(tiny, folder=folder16, weights=plain.load_folder(folder16)[1])
        dtype = "bfloat16"
    fast, slow = engine(tiny, dtype, num_kv_blocks=1000).engine, engine(tiny, dtype, num_kv_blocks=1000).engine
    assert fast.use_graphs
    slow.use_graphs = slow.use_tapes = False       # every step part by part
    toks = {r: traces.random_tokens(V, 1800, seed=80 + i) for i, r in enumerate("abcd")}
    fed = {r: 0 for r in toks}
    seqs = {}
    scale = [1.0]

    def both(plan, want_last=True):
        outs = []
        for eng in (fast, slow):
            entries = []
            for r, n in plan:
                if (eng, r) not in seqs:
                    seqs[(eng, r)] = eng.open(r)
                entries.append(StepEntry(seqs[(eng, r)], toks[r][fed[r]:fed[r] + n], [n - 1] if want_last else []))
            outs.append(eng.step(entries))
        for r, n in plan:
            fed[r] += n
            assert fed[r] <= len(toks[r])
        if outs[1] is None:
            assert outs[0] is None
        else:
            # float32: 64 rows and more take the norm kernel with a wavefront a row, which adds in another
            # order than the one for few rows; bfloat16: the library's product may round 128 rows otherwise
            # than 100
            scale[0] = max(scale[0], float(outs[1].abs().max()))
            assert float((outs[0] - outs[1]).abs().max()) <= (2e-5 if dtype == "float32" else 0.03) * scale[0], plan
        return outs[0]

    for n, want in ((100, False), (70, True), (120, False), (65, True), (128, True), (9, True)):
        for r in "abcd":
            both([(r, n)], want)
        both([("a", 1), ("b", 1), ("c", 1)])              # a decode graph between them
    before = fast.prompt_graph_replays
    for i in range(8):               # a portion beside decoded tokens: recorded the fourth time, then replayed
        both([("a", 1), ("d", 40 + 3 * i), ("b", 1)])
    assert fast.prompt_graph_replays >= before + 4
    before = fast.prompt_graph_replays
    for i in range(12):              # two portions and a decoded token: the padded total is what counts
        both([("a", 6 + i), ("b", 1), ("c", 20 - i)])
    assert fast.prompt_graph_replays >= before + 3          # (a wider block table on the way starts a new graph)
    both([("a", 30), ("d", 3)])                           # an entry of three tokens: launched kernel by kernel
    for r in "bcd":
        both([(r, 77)], True)
    assert fast.prompt_graph_replays >= 14 and slow.prompt_graph_replays == 0
    for _ in range(3):
        last = both([("a", 1), ("b", 1), ("c", 1), ("d", 1)])
    ref = plain.forward(tiny["cfg"], tiny["weights"], toks["d"][:fed["d"]])
    tol = 2e-4 if dtype == "float32" else 0.06 * float(ref.abs().max())
    assert float((last[3].cpu() - ref[fed["d"] - 1]).abs().max()) < tol
    for eng in (fast, slow):
        eng.cache.check()


def test_graphs_that_are_dropped_and_recorded_again(tiny):
    """With room for two shapes of each kind, steps of four shapes in turn drop recorded graphs and record
    them again; every step equals the eager engine's."""
    from zedinfer_amd.engine import StepEntry
    V = tiny["cfg"]["vocab_size"]
    fast, slow = engine(tiny, num_kv_blocks=300).engine, engine(tiny, num_kv_blocks=300).engine
    slow.use_graphs = slow.use_tapes = False       # every step part by part
    fast.graph_limit = fast.prompt_graph_limit = 2
    fast.graph_after = 2                           # a kind of step is captured the second time it comes
    toks = {r: traces.random_tokens(V, 900, seed=90 + i) for i, r in enumerate("abc")}
    fed = {r: 0 for r in toks}
    seqs = {(eng, r): eng.open(r) for eng in (fast, slow) for r in toks}

    def both(plan):
        outs = [eng.step([StepEntry(seqs[(eng, r)], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in plan])
                for eng in (fast, slow)]
        for r, n in plan:
            fed[r] += n
        assert float((outs[0] - outs[1]).abs().max()) <= 2e-5 * max(1.0, float(outs[1].abs().max())), plan

    for _ in range(3):
        for plan in ([("a", 1)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 1)], [("b", 1), ("c", 1)]):
            for _ in range(3):
                both(plan)
        for plan in ([("a", 10)], [("b", 70)], [("a", 1), ("c", 9)], [("c", 70)]):
            for _ in range(3):
                both(plan)
    assert len(fast._graphs) <= 2 and len(fast._prompt_graphs) <= 2
    assert fast.graph_replays >= 10 and fast.prompt_graph_replays >= 5


def test_steps_of_many_rows_come_in_the_sizes_the_warm_up_measured(tmp_path):
    """A serving engine on bfloat16 weights that is told to measure everything at once measures the library's algorithms for its many-rows
    products at every multiple of 64 rows a step can bring; portions of prompts beside decoding requests then run
    with their decoding entries filled up to a multiple of 64, so every such step's rows are among the measured
    sizes; the tokens are the plain implementation's.  Left to itself an engine measures nothing when it is made
    and every size when its first step is about to run."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    from zedinfer_amd.parts.rows import sizes_between
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "B", dtype=torch.bfloat16, std=tiny_configs.SHARP_STD)
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["B"]
    sched = SchedulerConfig(num_kv_blocks=160, kv_block_size=ps, max_batch_requests=4, max_prefill_tokens=192,
                            max_batch_tokens=256)
    ie = InferenceEngine.create(folder, "bfloat16", sched, warm_up_sizes="all")
    eng = ie.engine
    measured = {k[1] for k in eng.rt.choices if k[0] == "library_product"}
    assert measured == set(sizes_between(eng.model.step_rows, "mixed", 128, 192 + 4 + 64)) == {320, 256, 192, 128}
    prompts = [traces.random_tokens(cfg["vocab_size"], n, seed=70 + i) for i, n in enumerate([250, 200, 130, 70])]
    results = ie.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))
    mixed = [k for k in eng._prompt_graphs if k[1] > 0]             # (entries, decoding entries, tokens of the portions, ...)
    assert mixed and all(k[1] % 64 == 0 and (k[2] + k[1]) in measured for k in mixed), mixed
    # bfloat16 may break a near tie the other way: every token that was generated must be, for the plain
    # implementation fed the same tokens, the best or within the bfloat16 tolerance of the best
    for prompt, res in zip(prompts, results):
        assert len(res.output_ids) == 12
        ref = plain.forward(cfg, w, list(prompt) + res.output_ids)[len(prompt) - 1:-1]
        taken = ref[torch.arange(12), torch.tensor(res.output_ids)]
        assert bool((taken >= ref.max(dim=1).values - 0.06 * float(ref.abs().max())).all()), (taken, ref.max(dim=1).values)
    eng.cache.check()
    # left to itself: nothing when it is made, the sizes of the steps that came afterwards, and the same tokens
    lazy = InferenceEngine.create(folder, "bfloat16", sched)
    assert lazy.engine.tune_when_scheduled and not [k for k in lazy.engine.rt.choices if k[0] == "library_product"]
    again = lazy.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))
    came = {k[1] for k in lazy.engine.rt.choices if k[0] == "library_product"}
    ran = {k[2] + k[1] for k in lazy.engine._prompt_graphs}
    assert came and came <= measured and {r for r in ran if r > 64} <= came, (came, ran)
    assert [r.output_ids for r in again] == [r.output_ids for r in results]


def test_one_kernel_decode_attention_equals_the_two_kernel_path(tiny, monkeypatch, tmp_path):
    """Pure decode steps of few tokens rotate, store and attend in one kernel.  With that path switched
    off the same steps give the same logits (the caches hold the same keys and values, so later steps
    agree too), across page edges and with sequences of different lengths."""
    from zedinfer_amd.engine import StepEntry
    from zedinfer_amd.parts.mixers import Attention
    V = tiny["cfg"]["vocab_size"]
    # a bfloat16 checkpoint: weights stored in 32 bits would stay so and take the plain kernels
    folder16 = tiny_configs.write_tiny(str(tmp_path / "bf16"), tiny["name"], dtype=torch.bfloat16)
    tiny16 = dict(tiny, folder=folder16, weights=plain.load_folder(folder16)[1])
    one, two = engine(tiny16, "bfloat16").engine, engine(tiny16, "bfloat16").engine
    for eng in (one, two):
        eng.use_graphs = eng.use_tapes = False       # every step part by part: the calls are counted
    toks = {r: traces.random_tokens(V, 120, seed=70 + i) for i, r in enumerate("abc")}
    fed = {r: 0 for r in toks}
    seqs = {(e, r): e.open(r) for e in (one, two) for r in toks}
    calls = {"fused": 0}
    from zedinfer_amd import ops
    real = ops.attention_decode_fused

    def counted(*a, **k):
        calls["fused"] += 1
        return real(*a, **k)
    monkeypatch.setattr(ops, "attention_decode_fused", counted)

    def both(plan):
        outs = []
        for eng in (one, two):
            monkeypatch.setattr(Attention, "FUSED_DECODE_MAX_TOKENS", 16 if eng is one else 0)
            outs.append(eng.step([StepEntry(seqs[(eng, r)], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in plan]))
        for r, n in plan:
            fed[r] += n
        scale = float(outs[1].abs().max())
        assert float((outs[0] - outs[1]).abs().max()) <= 0.02 * scale, plan
        return outs

    both([("a", 37), ("b", 5), ("c", 1)])
    before = calls["fused"]
    for _ in range(40):
        both([("a", 1), ("b", 1), ("c", 1)])
    layers = tiny["cfg"]["num_hidden_layers"]
    assert calls["fused"] - before == 40 * layers       # only the first engine, every layer
    last = both([("b", 1)])[0]
    ref = plain.forward(tiny["cfg"], tiny16["weights"], toks["b"][:fed["b"]])
    assert float((last[0].cpu() - ref[fed["b"] - 1]).abs().max()) < 0.06 * float(ref.abs().max())
    # a launch of more workgroups (tokens x key/value heads x chunks of the keys) than the limit takes the
    # separate kernels: with the limit below this step's launch nothing is fused, and the logits agree as before
    nkv = tiny["cfg"]["num_key_value_heads"]
    assert 3 * nkv * ops.attention_decode_chunks(256) <= Attention.FUSED_DECODE_WORKGROUPS_PER_UNIT * ops.compute_units() == 512
    monkeypatch.setattr(Attention, "FUSED_DECODE_MAX_WORKGROUPS", 3 * nkv - 1)
    before = calls["fused"]
    both([("a", 1), ("b", 1), ("c", 1)])
    assert calls["fused"] == before
    both([("b", 1)])
    assert calls["fused"] == before + layers


@pytest.mark.parametrize("requests", [20, 70, 136])
def test_decode_graphs_with_the_library_product(tiny, requests, monkeypatch, tmp_path):
    """More than 16 decoding requests on a bfloat16 checkpoint: 17..64 rows take the second few-rows
    kernel, more than 64 the library's product (also for the float32 logits), inside the captured graph;
    the rotary launch is its own again and the attention takes every token of the step.  Every replay is
    checked against eager launches, with eager prompt steps between them, and the last step against the
    plain implementation; the calls are counted to show which product ran (weights stored in 32 bits
    would go to the plain product instead, which this test is not about)."""
    from zedinfer_amd.engine import StepEntry
    from zedinfer_amd.ops import _lib
    from tolerances import bf16_within
    V = tiny["cfg"]["vocab_size"]
    folder16 = tiny_configs.write_tiny(str(tmp_path / "bf16"), tiny["name"], dtype=torch.bfloat16,
                                       std=tiny_configs.SHARP_STD)
    tiny16 = dict(tiny, folder=folder16, weights=plain.load_folder(folder16)[1])
    fast = engine(tiny16, "bfloat16", max_batch_requests=requests + 4, num_kv_blocks=8 * requests).engine
    slow = engine(tiny16, "bfloat16", max_batch_requests=requests + 4, num_kv_blocks=8 * requests).engine
    slow.use_graphs = slow.use_tapes = False       # every step part by part
    # steps with prompt portions run as they are in both engines (padded to a graph's shape they would take
    # other kernels and round differently, and so would every later step that reads what they stored)
    fast.prompt_graph_max_tokens = 0
    fast.use_tapes = False
    names = [f"r{i}" for i in range(requests)]
    toks = {r: traces.random_tokens(V, 40, seed=80 + i) for i, r in enumerate(names)}
    seqs = {(e, r): e.open(r) for e in (fast, slow) for r in names}
    fed = {r: 0 for r in names}
    calls = {}
    real_call = _lib.call

    def counted_call(name, *a):
        calls[name] = calls.get(name, 0) + 1
        return real_call(name, *a)
    monkeypatch.setattr(_lib, "call", counted_call)

    def both(plan):
        outs = []
        for eng in (fast, slow):
            outs.append(eng.step([StepEntry(seqs[(eng, r)], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in plan]))
        for r, n in plan:
            fed[r] += n
        assert torch.equal(outs[0], outs[1]), (plan[0], len(plan))
        return outs[0]

    both([(r, 5 + i % 4) for i, r in enumerate(names)])
    calls.clear()
    for step in range(12):
        last = both([(r, 1) for r in names])
        if step == 0:
            first = dict(calls)
        if step % 4 == 1:
            both([(names[0], 3), (names[1], 1)])      # an eager mixed step between the replays
    assert fast.graph_replays >= 8
    # which kernels a decode step of this many rows took (counted over the step's two engines)
    assert first.get("zi_gemm_generic", 0) == 0, first
    assert first.get("zi_attention_decode", 0) > 0 and first.get("zi_attention_decode_fused", 0) == 0, first
    if requests <= 64:
        assert first.get("zi_gemm_skinny", 0) > 0 and first.get("zi_gemm_lt", 0) == 0, first
    else:
        assert first.get("zi_gemm_lt", 0) > 0, first
    worst = mean = scale = 0.0
    for i, r in enumerate(names):
        ref = plain.forward(tiny["cfg"], tiny16["weights"], toks[r][:fed[r]])[-1]
        d = (last[i].cpu() - ref).abs()
        worst, mean, scale = max(worst, float(d.max())), mean + float(d.mean()) / requests, max(scale, float(ref.abs().max()))
    print(f"{requests} requests: worst {worst:.3e} mean {mean:.3e} of scale {scale:.3e}; calls of a step {first}")
    assert bf16_within(worst, mean, scale)
