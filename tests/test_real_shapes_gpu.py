"""Two layers of the Qwen2.5-1.5B, 7B and 32B layer shapes (real widths, head counts and groups; a smaller
vocabulary and two layers so that the plain implementation stays affordable on the CPU) against the plain
implementation: a prompt in portions, then decoded tokens, alone and beside a second request.  In float32,
in bfloat16 with the float32 checkpoint (weights stored in 32 bits stay so) and in bfloat16 with a bfloat16
checkpoint ("bfloat16w"): the serving kernels (few-rows products and their cuts along k, partial sums, the
one-kernel decode attention, prompt attention, the library product) at the shapes they serve.  At these
widths N(0, 0.02) weights already make attention peaked: a pass without rotation or scale leaves the bfloat16
tolerance several times over (tests/test_tolerances.py shows it for the 1.5B sizes)."""
import pytest
import torch

import traces
from plain import qwen2_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST

pytestmark = pytest.mark.gpu

SHAPES = {
    "1.5B": dict(hidden_size=1536, intermediate_size=8960, num_attention_heads=12, num_key_value_heads=2,
                 head_dim=128, tie_word_embeddings=True),
    "7B": dict(hidden_size=3584, intermediate_size=18944, num_attention_heads=28, num_key_value_heads=4,
               head_dim=128, tie_word_embeddings=False),
    "32B": dict(hidden_size=5120, intermediate_size=27648, num_attention_heads=40, num_key_value_heads=8,
                head_dim=128, tie_word_embeddings=False),
}


@pytest.fixture(scope="module", params=list(SHAPES))
def model(request, tmp_path_factory):
    from zedinfer_amd.config import Qwen2Config
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    cfgd = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=4099, max_position_embeddings=4096,
                num_hidden_layers=2, rope_theta=1000000.0, rms_norm_eps=1e-6, use_sliding_window=False,
                torch_dtype="float32", eos_token_id=4098, **SHAPES[request.param])
    cfg = Qwen2Config.from_dict(cfgd)
    folder = str(tmp_path_factory.mktemp("real" + request.param))
    write_model_folder(folder, cfg, expected_weights(qwen2_forward_config(cfg)), seed=7, dtype=torch.float32,
                       noisy_norms=True)
    pcfg, w = plain.load_folder(folder)
    reqs = {"p": traces.random_tokens(4099, 330, seed=1), "q": traces.random_tokens(4099, 97, seed=2)}
    ref = {rid: plain.forward(pcfg, w, toks) for rid, toks in reqs.items()}
    del w
    folder16 = str(tmp_path_factory.mktemp("real16" + request.param))
    write_model_folder(folder16, cfg, expected_weights(qwen2_forward_config(cfg)), seed=7, dtype=torch.bfloat16,
                       noisy_norms=True)
    _, w16 = plain.load_folder(folder16)
    ref16 = {rid: plain.forward(pcfg, w16, toks) for rid, toks in reqs.items()}
    return dict(folder=folder, requests=reqs, reference=ref, folder16=folder16, reference16=ref16)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16w"])
def test_real_layer_shapes_match_plain(model, dtype):
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    folder, reference = model["folder"], model["reference"]
    if dtype == "bfloat16w":
        folder, reference, dtype = model["folder16"], model["reference16"], "bfloat16"
    engine = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=40, kv_block_size=16,
                                                               max_batch_requests=4))
    reqs = model["requests"]
    p, q = reqs["p"], reqs["q"]
    want = lambda n: list(range(n))   # noqa: E731
    steps = [
        {"step": 0, "entries": [{"id": "p", "tokens": p[:200], "want": want(200)}], "end": []},
        {"step": 1, "entries": [{"id": "p", "tokens": p[200:270], "want": want(70)},
                                {"id": "q", "tokens": q[:65], "want": want(65)}], "end": []},
        {"step": 2, "entries": [{"id": "p", "tokens": p[270:273], "want": want(3)},
                                {"id": "q", "tokens": q[65:66], "want": [0]}], "end": []},
    ]
    fp, fq = 273, 66
    while fq < len(q):          # both decode, token by token; q ends first and p goes on alone
        steps.append({"step": len(steps), "entries": [{"id": "p", "tokens": p[fp:fp + 1], "want": [0]},
                                                      {"id": "q", "tokens": q[fq:fq + 1], "want": [0]}],
                      "end": ["q"] if fq == len(q) - 1 else []})
        fp, fq = fp + 1, fq + 1
    while fp < len(p):
        steps.append({"step": len(steps), "entries": [{"id": "p", "tokens": p[fp:fp + 1], "want": [0]}],
                      "end": ["p"] if fp == len(p) - 1 else []})
        fp += 1
    out = traces.run_in_process(engine, steps)
    worst, mean, scale, rows, where = traces.compare(steps, out, reference, reqs)
    print(f"[{dtype}] rows={rows} worst={worst:.3e} mean={mean:.3e} scale={scale:.3e} at {where}")
    assert rows == len(p) + len(q)
    if dtype == "float32":
        assert worst <= 3e-4 * max(1.0, scale), where
    else:
        assert engine.graph_replays > 10
        assert worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale, where


def test_wide_prompt_tiles_give_the_same_logits(model, monkeypatch):
    """The prompt kernel's tiles of 128 queries (taken by the planner for steps that fill the chip) against its
    tiles of 64, through the engine: a query's walk over its keys does not depend on the tile it rides in, so the
    logits agree bit for bit, portions beside each other and at a page's edge included."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.parts.mixers import AttentionPlanner
    reqs = model["requests"]
    p, q = reqs["p"], reqs["q"]
    want = lambda n: list(range(n))   # noqa: E731
    steps = [
        {"step": 0, "entries": [{"id": "p", "tokens": p[:200], "want": want(200)}], "end": []},
        {"step": 1, "entries": [{"id": "p", "tokens": p[200:329], "want": want(129)},
                                {"id": "q", "tokens": q[:65], "want": want(65)}], "end": ["p", "q"]},
    ]
    seen, outs = [], []
    plan = AttentionPlanner.plan

    def recording(self, hb):
        made = plan(self, hb)
        seen.append(made.sizes["tile"])
        return made

    monkeypatch.setattr(AttentionPlanner, "plan", recording)
    monkeypatch.setattr(AttentionPlanner, "FILL_ALONE", 10 ** 9)
    for fill in (None, 1):           # what the chip's size gives (one and a half workgroups a compute unit), then any step
        monkeypatch.setattr(AttentionPlanner, "FILL", fill)
        engine = Engine.from_folder(model["folder16"], "bfloat16",
                                    SchedulerConfig(num_kv_blocks=40, kv_block_size=16, max_batch_requests=4))
        assert engine.planners[0].wide_tile == 128
        seen.clear()
        outs.append(traces.run_in_process(engine, steps))
        assert set(seen) == ({64} if fill is None else {128}), seen
    for s in (0, 1):
        assert torch.equal(torch.as_tensor(outs[0][s]), torch.as_tensor(outs[1][s])), s
    worst, mean, scale, rows, where = traces.compare(steps, outs[1], model["reference16"], reqs)
    assert rows == 329 + 65
    assert worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale, where
    # and in workgroups of four wavefronts (what large steps take): another rounding, the same tolerance
    monkeypatch.setattr(AttentionPlanner, "FILL_ALONE", 1)
    engine = Engine.from_folder(model["folder16"], "bfloat16",
                                SchedulerConfig(num_kv_blocks=40, kv_block_size=16, max_batch_requests=4))
    alone = traces.run_in_process(engine, steps)
    worst, mean, scale, rows, where = traces.compare(steps, alone, model["reference16"], reqs)
    assert rows == 329 + 65
    assert worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale, where


def test_graphs_that_hold_the_library_product_replay_right_at_real_widths(model):
    """Steps whose many-rows products are the library's, with the algorithms a warm-up chose by timing, captured
    as HIP graphs at the real widths and replayed several times with other work between the replays: prompt
    portions of 200 tokens (run as 256 rows, one row wanted) and 96 requests decoding together.  Every replay is
    held against the plain implementation, the decode steps also bit for bit against an engine that launches
    every step part by part (a library algorithm that clears its workspace with a memset node, or anything
    else that a graph does not repeat, would show from the second replay on)."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    pcfg, w16 = plain.load_folder(model["folder16"])
    p = model["requests"]["p"]
    sched = SchedulerConfig(num_kv_blocks=400, kv_block_size=16, max_batch_requests=100)
    fast, slow = (Engine.from_folder(model["folder16"], "bfloat16", sched) for _ in range(2))
    slow.use_graphs = slow.use_tapes = False
    fast.graph_after = 2                            # a kind of step is captured the second time it comes
    fast.warm_up([256])

    def within(got, ref):
        d = (got.float().cpu() - ref).abs()
        scale = float(ref.abs().max())
        return float(d.max()) <= BF16_REL_WORST * scale and float(d.mean()) <= BF16_REL_MEAN * scale

    # ---- prompt portions: the first step of the shape runs part by part, the second is captured, the rest replay
    other = fast.open("other")
    fast.step([StepEntry(other, p[:40], [])])
    for i in range(5):
        toks = p[20 * i:20 * i + 200]
        seq = fast.open(("prompt", i))
        got = fast.step([StepEntry(seq, toks, [199])])
        assert within(got[0], plain.forward(pcfg, w16, toks)[199]), i
        fast.close(seq)
        fast.step([StepEntry(other, p[40 + i:41 + i], [0])])          # eager work of another shape between the replays
        torch.cuda.synchronize()
    assert fast.prompt_graph_replays >= 3
    fast.close(other)
    # ---- 96 requests decode together: more than 64 rows, the library's product inside the decode graph (a number
    # of requests that the engine runs as it is: fewer would be filled up to it in the engine that records)
    names = [f"d{i}" for i in range(96)]
    seqs = {(e, r): e.open(r) for e in (fast, slow) for r in names}
    # (the prompts enter part by part in both engines: padded to a graph's shape the products would have other
    # numbers of rows, round differently, and so would every later step that reads what was stored)
    fast.use_graphs = fast.use_tapes = False
    for e in (fast, slow):
        e.step([StepEntry(seqs[(e, r)], p[i:i + 8], []) for i, r in enumerate(names)])
    fast.use_graphs = fast.use_tapes = True
    before = fast.graph_replays
    for k in range(6):
        outs = [e.step([StepEntry(seqs[(e, r)], p[i + 8 + k:i + 9 + k], [0]) for i, r in enumerate(names)]) for e in (fast, slow)]
        assert torch.equal(outs[0], outs[1]), k
        torch.cuda.synchronize()
    assert fast.graph_replays >= before + 4 and slow.graph_replays == 0
    for i in (0, 33, 95):
        assert within(outs[0][i], plain.forward(pcfg, w16, p[i:i + 14])[13]), i
    for e in (fast, slow):
        for r in names:
            e.close(seqs[(e, r)])
        e.cache.check()
