"""The engine against the plain implementation: each request alone and whole; most of it in one
step and the last 32 tokens one by one; portions of changing size; and mixed batches with so few
pages that they are used again.  In float32 and in bfloat16, on three tiny configurations; bfloat16
both with the float32 checkpoint (weights stored in 32 bits stay so) and with a bfloat16 checkpoint
("bfloat16w"), which is what the serving kernels for bfloat16 weights take.

Every variant runs a second time with "sharp" weights (a trailing "s": matrices of width
tiny_configs.SHARP_STD instead of 0.02).  With the narrow weights attention is nearly uniform and a
forward pass without rotation, or without the 1/sqrt(d), stays inside the bfloat16 tolerance; with the
sharp ones either moves the logits by their whole size while bfloat16 rounding stays below 2 % of it
(tests/test_tolerances.py holds that on the CPU)."""

import pytest
import torch

import tiny_configs
import traces
from plain import qwen2_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 100, 70, 64, 90, 41, 128, 77], "B": [1, 31, 64, 100, 47, 90, 120, 66, 35, 80],
           "C": [1, 31, 64, 100, 47, 90, 120, 66, 35, 80]}


@pytest.fixture(scope="module", params=["A", "B", "C"])
def tiny(request, tmp_path_factory):
    name = request.param
    folder = tiny_configs.write_tiny(str(tmp_path_factory.mktemp(f"tiny{name}")), name)
    cfg, w = plain.load_folder(folder)
    reqs = {f"r{i}": traces.random_tokens(cfg["vocab_size"], n, seed=100 + i) for i, n in enumerate(LENGTHS[name])}
    ref = {rid: plain.forward(cfg, w, toks) for rid, toks in reqs.items()}
    folder16 = tiny_configs.write_tiny(str(tmp_path_factory.mktemp(f"tiny{name}bf16")), name, dtype=torch.bfloat16)
    _, w16 = plain.load_folder(folder16)
    ref16 = {rid: plain.forward(cfg, w16, toks) for rid, toks in reqs.items()}
    out = dict(name=name, folder=folder, cfg=cfg, weights=w, requests=reqs, reference=ref,
               folder16=folder16, reference16=ref16)
    # the sharp variants: the same sizes and requests, wider weights
    sharp = tiny_configs.write_tiny(str(tmp_path_factory.mktemp(f"tiny{name}s")), name, std=tiny_configs.SHARP_STD)
    sharp16 = tiny_configs.write_tiny(str(tmp_path_factory.mktemp(f"tiny{name}sbf16")), name, dtype=torch.bfloat16,
                                      std=tiny_configs.SHARP_STD)
    for key, f in (("", sharp), ("16", sharp16)):
        wf = plain.load_folder(f)[1]
        out["sharp_folder" + key] = f
        out["sharp_reference" + key] = {rid: plain.forward(cfg, wf, toks) for rid, toks in reqs.items()}
    return out


DTYPES = ["float32", "bfloat16", "bfloat16w", "float32s", "bfloat16s", "bfloat16ws"]


def variant(tiny, dtype):
    """(model folder, engine dtype, reference logits) of a dtype parameter."""
    pre = ""
    if dtype.endswith("s"):
        pre, dtype = "sharp_", dtype[:-1]
    if dtype == "bfloat16w":
        return tiny[pre + "folder16"], "bfloat16", tiny[pre + "reference16"]
    return tiny[pre + "folder"], dtype, tiny[pre + "reference"]


def make_engine(tiny, dtype, pages):
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    folder, engine_dtype, _ = variant(tiny, dtype)
    return Engine.from_folder(folder, engine_dtype,
                              SchedulerConfig(num_kv_blocks=pages, kv_block_size=ps, max_batch_requests=4))


def check(tiny, dtype, steps, outputs):
    worst, mean, scale, rows, where = traces.compare(steps, outputs, variant(tiny, dtype)[2], tiny["requests"])
    print(f"[{tiny['name']} {dtype}] rows={rows} worst={worst:.3e} mean={mean:.3e} scale={scale:.3e} at {where}")
    assert rows > 0
    if dtype.startswith("float32"):
        assert worst <= F32_TOL * max(1.0, scale), f"first/worst difference at (step, request, position) {where}"
    else:
        assert worst <= BF16_REL_WORST * scale, f"worst difference at {where}"
        assert mean <= BF16_REL_MEAN * scale


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", ["whole", "last32", "portions", "mixed", "mixed_few_wanted"])
def test_engine_matches_plain(tiny, dtype, shape):
    steps = {"whole": traces.whole, "last32": traces.last_decoded, "portions": traces.portions,
             "mixed": traces.mixed,
             "mixed_few_wanted": lambda reqs: traces.few_wanted(traces.mixed(reqs, decode_tail=24, seed=3), seed=3)
             }[shape](tiny["requests"])
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    pages = traces.max_live_tokens(steps) // ps      # as few pages as the replay tool would have
    engine = make_engine(tiny, dtype, pages)
    out = traces.run_in_process(engine, steps)
    if shape.startswith("mixed"):
        # pages were given back and taken again: more pages handed out than the pool has
        assert all(g.pool.takes > g.pool.total for g in engine.cache.groups)
    check(tiny, dtype, steps, out)


@pytest.mark.parametrize("dtype", ["float32s", "bfloat16ws"])
@pytest.mark.parametrize("seed,max_live", [(1, 4), (2, 4), (3, 9)])
def test_random_steps_match_plain(tiny, dtype, seed, max_live):
    """Mixed steps of up to ``max_live`` requests with the wanted places of every entry drawn at random (all, the
    last, none, a few in any order and perhaps twice) and the entries of a step shuffled: which kind of step the
    engine makes of each (recorded, padded, part by part) follows from that, and every wanted row is the plain
    implementation's."""
    import random
    rng = random.Random(seed)
    steps = traces.random_wanted(traces.mixed(tiny["requests"], max_live=max_live, seed=seed,
                                              decode_tail=rng.choice([3, 12, 40]), max_portion=rng.choice([24, 70, 150])), seed=seed)
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    folder, engine_dtype, _ = variant(tiny, dtype)
    engine = Engine.from_folder(folder, engine_dtype, SchedulerConfig(num_kv_blocks=traces.max_live_tokens(steps, round_to=ps) // ps + 1,
                                                                      kv_block_size=ps, max_batch_requests=max_live))
    engine.graph_after = 2
    out = traces.run_in_process(engine, steps)
    check(tiny, dtype, steps, out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16w", "bfloat16ws"])
def test_replay_tool(tiny, dtype, tmp_path):
    """The same mixed trace through bin/trace_run as a child process."""
    steps = traces.mixed(tiny["requests"], seed=3)
    folder, engine_dtype, _ = variant(tiny, dtype)
    out = traces.run_tool(folder, engine_dtype, steps, str(tmp_path / "out"), traces.max_live_tokens(steps))
    check(tiny, dtype, steps, out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16ws"])
def test_replay_tool_when_few_rows_are_wanted(tiny, dtype, tmp_path):
    """A mixed trace with a long decoding tail in which every entry wants the logits of its last token at most
    and some want none, through bin/trace_run: steps that write nothing still print their `done` line, and the
    files of the others hold the wanted rows only."""
    steps = traces.few_wanted(traces.mixed(tiny["requests"], seed=7, decode_tail=20), seed=7, none=0.25)
    assert any(not any(e["want"] for e in st["entries"]) for st in steps)       # a step that wants nothing
    folder, engine_dtype, _ = variant(tiny, dtype)
    out = traces.run_tool(folder, engine_dtype, steps, str(tmp_path / "out"), traces.max_live_tokens(steps))
    assert sorted(out) == [st["step"] for st in steps if any(e["want"] for e in st["entries"])]
    check(tiny, dtype, steps, out)


@pytest.mark.parametrize("how", ["options", "trace"])
def test_replay_tool_with_the_configuration_s_own_pages(tiny, how, tmp_path):
    """The pool geometry given to the tool, on the command line or as the trace's first line: the page
    size of the configuration (8 for B and C), at most four live requests, and so few pages that the
    tool reports more handed out than the pool has."""
    import re
    steps = traces.mixed(tiny["requests"], seed=5)
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    folder, engine_dtype, _ = variant(tiny, "bfloat16ws")
    need = traces.max_live_tokens(steps)
    log = str(tmp_path / "stderr.txt")
    if how == "options":
        out = traces.run_tool(folder, engine_dtype, steps, str(tmp_path / "out"), need,
                              options=["--kv-block-size", ps, "--max-live", 4], stderr_to=log)
    else:
        out = traces.run_tool(folder, engine_dtype, steps, str(tmp_path / "out"), need,
                              geometry={"kv_block_size": ps, "num_kv_blocks": need // ps, "max_live": 4}, stderr_to=log)
    check(tiny, "bfloat16ws", steps, out)
    said = open(log).read()
    assert f"{need // ps} pages of {ps} tokens" in said and "up to 4 live requests" in said
    groups = re.findall(r"cache group \d+ \(\w+\): (\d+) pages, (\d+) handed out", said)
    assert groups and all(int(total) == need // ps and int(takes) > int(total) for total, takes in groups), said


@pytest.mark.parametrize("dtype", ["float32", "bfloat16w"])
def test_a_step_that_fails_leaves_nothing_behind(tiny, dtype):
    """A step that cannot run to its end (a token the model does not have, in a prompt portion or among decoding
    requests; pages that run out for a later entry) gives back the pages and promises it had taken, changes no
    request's length, and the requests go on to the plain implementation's logits afterwards."""
    from zedinfer_amd.cache import OutOfPages
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    folder, edtype, ref = variant(tiny, dtype)
    V = tiny["cfg"]["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[tiny["name"]]
    toks = {r: tiny["requests"][r] for r in ("r3", "r4")}           # 100 and 70 (47) tokens
    pages = -(-len(toks["r3"]) // ps) + -(-len(toks["r4"]) // ps) + 1
    eng = Engine.from_folder(folder, edtype, SchedulerConfig(num_kv_blocks=pages, kv_block_size=ps, max_batch_requests=3))
    a, b = eng.open("a"), eng.open("b")
    fed = {"a": 0, "b": 0}
    ids = {"a": toks["r3"], "b": toks["r4"]}

    def state():
        pool = eng.cache.groups[0].pool
        return (a.length, b.length, list(a.pages[0]), list(b.pages[0]), list(a.promised), list(b.promised), pool.num_held,
                pool.committed)

    def good(seq, name, n):
        out = eng.step([StepEntry(seq, ids[name][fed[name]:fed[name] + n], [n - 1])])
        fed[name] += n
        scale = float(ref["r3" if name == "a" else "r4"].abs().max())
        want = ref["r3" if name == "a" else "r4"][fed[name] - 1]
        assert float((out[0].cpu() - want).abs().max()) <= (F32_TOL if dtype == "float32" else BF16_REL_WORST) * max(scale, 1.0)

    good(a, "a", 20)
    good(b, "b", 9)
    for _ in range(3):                       # decode steps of the two together: their shape gets a tape
        out = eng.step([StepEntry(a, ids["a"][fed["a"]:fed["a"] + 1], [0]), StepEntry(b, ids["b"][fed["b"]:fed["b"] + 1], [0])])
        fed["a"] += 1
        fed["b"] += 1
    before = state()
    # a bad token in a portion that needs new pages, beside a decoding request
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.step([StepEntry(a, ids["a"][fed["a"]:fed["a"] + 30] + [V + 5], [30]), StepEntry(b, ids["b"][fed["b"]:fed["b"] + 1], [0])])
    assert state() == before
    # a bad token among decoding requests of a shape that has run before
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.step([StepEntry(a, [ids["a"][fed["a"]]], [0]), StepEntry(b, [-1], [0])])
    assert state() == before
    # pages run out for the second entry after the first has grown
    c = eng.open("c")
    with pytest.raises(OutOfPages):
        eng.step([StepEntry(a, ids["a"][fed["a"]:fed["a"] + 40], [39]), StepEntry(c, list(range(1, 60 * ps)), [0])])
    assert state() == before and c.length == 0 and not any(p >= 0 for p in c.pages[0])
    eng.close(c)
    eng.cache.check()
    good(a, "a", 30)
    good(b, "b", 1)
    good(a, "a", 1)
    eng.close(a)
    eng.close(b)
    eng.cache.check()
    assert eng.cache.groups[0].pool.num_held == 0
