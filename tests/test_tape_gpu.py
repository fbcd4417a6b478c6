"""The step tape: library calls recorded once and made again from native code.  The tape alone (recorded
operators on buffers whose contents change), then the engine: steps that run from tapes against the same
steps part by part, bit for bit, and against the plain implementation."""
import pytest
import torch

import tiny_configs
import traces
from plain import qwen2_plain as plain
from tolerances import F32_TOL, bf16_within

pytestmark = pytest.mark.gpu


def test_a_tape_repeats_its_calls_on_new_contents():
    from zedinfer_amd import ops
    from zedinfer_amd.ops.tape import Recording
    torch.manual_seed(0)
    n, H, N = 6, 200, 136
    x = torch.randn(n, H, device="cuda").bfloat16()
    w = (torch.randn(N, H, device="cuda") * 0.05).bfloat16()
    g = torch.randn(H, device="cuda").bfloat16()
    resid = torch.randn(n, H, device="cuda")
    normed, y = torch.empty_like(x), torch.empty(n, N, device="cuda", dtype=torch.float32)

    def step():
        ops.add_rms_norm(resid, x, g, 1e-5, out=normed)          # resid += x; normed = norm(resid) * g
        ops.linear(normed, w, out=y)

    keep = resid.clone()
    step()                                   # workspaces get their sizes
    resid.copy_(keep)
    with Recording(torch.device("cuda", 0)) as rec:
        step()
    assert rec.allocations == 0 and [c[0] for c in rec.calls] == ["zi_add_rmsnorm", "zi_gemm_skinny"]
    tape = rec.tape()
    assert tape.length == 2
    first = y.clone()
    for seed in (1, 2):                      # new contents in the same buffers
        torch.manual_seed(seed)
        x.copy_(torch.randn(n, H, device="cuda").bfloat16())
        resid.copy_(torch.randn(n, H, device="cuda"))
        keep = resid.clone()
        tape.run()
        got, got_resid = y.clone(), resid.clone()
        resid.copy_(keep)
        step()
        assert torch.equal(got, y) and torch.equal(got_resid, resid) and not torch.equal(got, first)


def test_a_tape_refuses_what_it_cannot_hold():
    import ctypes
    from zedinfer_amd.ops import _lib
    from zedinfer_amd.ops.tape import Recording, Tape
    with pytest.raises(_lib.KernelLibraryError, match="not an entry point"):
        Tape([("zi_gemm_lt_choose", (1, 0, 0, 1, 1, 1, 1, 1, 1, 1, 0))])
    lib = _lib.load()
    handle = ctypes.c_void_p(lib.zi_tape_new())
    words = (ctypes.c_int64 * 3)(1, 2, 3)
    with pytest.raises(_lib.KernelLibraryError, match="takes 9 arguments, 3 were recorded"):
        _lib.call("zi_tape_record", handle, b"zi_embedding", ctypes.cast(words, ctypes.c_void_p), 3)
    lib.zi_tape_free(handle)
    # a call that fails on replay is reported with its place in the tape
    with Recording() as rec:
        pass
    assert rec.tape() is None
    bad = Tape([("zi_add", (ctypes.c_void_p(0), 1, ctypes.c_void_p(0), 1, ctypes.c_void_p(0), 1, 0, ctypes.c_void_p(0))),
                ("zi_add", (ctypes.c_void_p(0), 99, ctypes.c_void_p(0), 1, ctypes.c_void_p(0), 1, 8, ctypes.c_void_p(0)))])
    with pytest.raises(_lib.KernelLibraryError, match="call 1 of a tape of 2"):
        bad.run()
    with pytest.raises(RuntimeError, match="already"):
        with Recording():
            with Recording():
                pass


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_steps_from_tapes_equal_steps_part_by_part(name, dtype, tmp_path, monkeypatch):
    """Three requests with prompts of 128 tokens in portions of 64 (a shape that recurs: its second step is
    recorded, the later ones run from the tape), then decoded together token by token, on an engine that runs
    from tapes alone (no graphs) and on one that runs every step part by part: the same bits, and both within
    the tolerance of the plain implementation.  Portions that are multiples of the padding step are taken so
    that both engines launch the same kernels."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), name, dtype=store, std=tiny_configs.SHARP_STD)
    cfg, w = plain.load_folder(folder)
    V = cfg["vocab_size"]
    ps = tiny_configs.PAGE_SIZES[name]

    def make(tapes):
        e = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=3 * (200 // ps + 2), kv_block_size=ps,
                                                              max_batch_requests=4))
        e.use_graphs = False
        e.use_tapes = tapes
        return e
    taped, plainly = make(True), make(False)
    assert taped.model.tape_safe()
    toks = {r: traces.random_tokens(V, 150, seed=60 + i) for i, r in enumerate("abc")}
    seqs = {(e, r): e.open(r) for e in (taped, plainly) for r in toks}
    fed = {r: 0 for r in toks}

    def both(plan):
        outs = [e.step([StepEntry(seqs[(e, r)], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in plan])
                for e in (taped, plainly)]
        for r, n in plan:
            fed[r] += n
        assert torch.equal(outs[0], outs[1]), plan
        return outs[0]

    for r in "abc":
        both([(r, 64)])
    for r in "abc":
        both([(r, 64)])
    runs_after_prompts = taped.tape_runs
    assert runs_after_prompts >= 2              # the third request's portions, at the least
    for _ in range(22):
        last = both([(r, 1) for r in "abc"])
    assert taped.tape_runs >= runs_after_prompts + 15 and plainly.tape_runs == 0
    worst = mean = scale = 0.0
    for i, r in enumerate("abc"):
        ref = plain.forward(cfg, w, toks[r][:fed[r]])[-1]
        d = (last[i].cpu() - ref).abs()
        worst, mean, scale = max(worst, float(d.max())), mean + float(d.mean()) / 3, max(scale, float(ref.abs().max()))
    if dtype == "float32":
        assert worst <= F32_TOL * max(1.0, scale)
    else:
        assert bf16_within(worst, mean, scale)
    for e in (taped, plainly):
        for r in toks:
            e.close(seqs[(e, r)])
        e.cache.check()
    # without tapes and graphs nothing is padded and nothing recorded
    monkeypatch.setenv("ZEDINFER_DISABLE_TAPES", "1")
    off = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=32, kv_block_size=ps, max_batch_requests=4))
    assert not off.use_tapes


def test_a_step_that_allocates_is_not_taped(tmp_path, monkeypatch):
    """A part that takes device memory while a step runs (against what ``tape_safe`` promises) is noticed when the
    step is recorded: the recording is dropped, the shape marked, and its steps go on part by part, with the
    right results."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.parts.feed_forward import SwiGLU
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "A")
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["A"]
    e = Engine.from_folder(folder, "float32", SchedulerConfig(num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4))
    e.use_graphs = False
    real = SwiGLU.forward
    kept = []

    def leaky(self, x):
        kept.append(torch.empty(1024, device=x.device))        # a fresh allocation every call
        return real(self, x)
    monkeypatch.setattr(SwiGLU, "forward", leaky)
    toks = traces.random_tokens(cfg["vocab_size"], 40, seed=1)
    ref = plain.forward(cfg, w, toks)
    seq = e.open("r")
    e.step([StepEntry(seq, toks[:8], [7])])
    for i in range(8, 40):
        got = e.step([StepEntry(seq, toks[i:i + 1], [0])]).cpu()
        assert float((got[0] - ref[i]).abs().max()) < F32_TOL * max(1.0, float(ref.abs().max()))
    assert e.tape_runs == 0 and any(dg.no_tape for dg in e._graphs.values())


def test_a_step_with_work_that_is_no_library_call_is_not_taped(tmp_path, monkeypatch):
    """A part that does device work through a torch operator that takes no memory (against what ``tape_safe``
    promises) leaves nothing on the tape for it.  A new tape is therefore run once on its own step, from workspaces
    made NaN, and must repeat the step's logits: this one does not, the shape is marked, and its steps go on part
    by part with the right results.  Without the part's extra work the same steps do run from tapes."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.parts.norms import RMSNorm
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "A")
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["A"]
    toks = traces.random_tokens(cfg["vocab_size"], 40, seed=2)

    def run(engine):
        engine.use_graphs = False
        seq = engine.open("r")
        rows = [engine.step([StepEntry(seq, toks[:8], [7])]).cpu()]
        for i in range(8, 40):
            rows.append(engine.step([StepEntry(seq, toks[i:i + 1], [0])]).cpu())
        engine.close(seq)
        return torch.cat(rows)

    sched = SchedulerConfig(num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4)
    plain_engine = Engine.from_folder(folder, "float32", sched)
    straight = run(plain_engine)
    assert plain_engine.tape_runs > 20
    from zedinfer_amd import ops

    def through_a_copy(self, resid, delta):
        """The library's norm into another workspace, then a torch copy into the one the next part reads: the copy
        takes no memory and is on no tape, so a replay would leave the last step's rows there."""
        out = self.rt.buffer("norm_out", (resid.shape[0], self.dim), self.rt.dtype)
        tmp = self.rt.buffer("norm_elsewhere", (resid.shape[0], self.dim), self.rt.dtype)
        ops.add_rms_norm(resid, delta, self.weight, self.eps, out=tmp, add_one=self.add_one)
        out.copy_(tmp)
        return out
    monkeypatch.setattr(RMSNorm, "add_forward", through_a_copy)
    e = Engine.from_folder(folder, "float32", sched)
    got = run(e)
    assert torch.equal(got, straight)
    assert e.tape_runs == 0 and all(dg.no_tape for dg in e._graphs.values())


def test_generation_from_tapes_alone(tmp_path, monkeypatch):
    """The serving loop (continuous batching, chunked prefill, steps queued ahead) with graphs switched off: the
    recurring steps run from tapes, and every request gets the plain implementation's greedy tokens."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    monkeypatch.setenv("ZEDINFER_DISABLE_GRAPHS", "1")
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "B")
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["B"]
    ie = InferenceEngine.create(folder, "float32", SchedulerConfig(num_kv_blocks=96, kv_block_size=ps, max_batch_requests=3,
                                                                   max_prefill_tokens=64, max_batch_tokens=80))
    assert not ie.engine.use_graphs and ie.engine.use_tapes
    prompts = [traces.random_tokens(cfg["vocab_size"], n, seed=20 + i) for i, n in enumerate([130, 64, 7, 128, 50])]
    results = ie.generate(prompts, GenerationConfig(max_new_tokens=24, ignore_eos=True))
    for prompt, res in zip(prompts, results):
        assert res.output_ids == plain.greedy_generate(cfg, w, prompt, 24)
    assert ie.engine.tape_runs > 20 and ie.engine.graph_replays == 0
    ie.engine.cache.check()
    assert not ie.engine.cache.live


def test_a_large_step_is_brought_up_to_a_measured_size(tmp_path):
    """Beyond 4,096 rows the sizes that a serving engine measures lie 128 rows apart: a step of 4,170 prompt tokens
    beside one decoding request (4,224 + 64 rows) gets 64 more padding tokens behind the portion.  Nothing of a
    request changes by that: the logits of the step and of the decode steps after it are the plain
    implementation's."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.parts.rows import many_rows as many_rows_size_at_least
    assert [many_rows_size_at_least(n) for n in (4096, 4097, 4288, 8192, 8200)] == [4096, 4224, 4352, 8192, 8448]
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "A")
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["A"]
    e = Engine.from_folder(folder, "float32", SchedulerConfig(num_kv_blocks=4400 // ps + 8, kv_block_size=ps, max_batch_requests=4,
                                                              max_seq_len=8192))
    e.use_graphs = False
    long_toks = traces.random_tokens(cfg["vocab_size"], 4174, seed=5)
    short_toks = traces.random_tokens(cfg["vocab_size"], 36, seed=6)
    a, b = e.open("a"), e.open("b")
    e.step([StepEntry(b, short_toks[:30], [])])
    got = e.step([StepEntry(a, long_toks[:4170], [4169]), StepEntry(b, short_toks[30:31], [0])]).cpu()
    keys = [k for k in e._prompt_graphs if k[1] > 0]
    assert keys == [k for k in keys if k[2] == 4288 and k[0] == 65], list(e._prompt_graphs)
    ref_a, ref_b = plain.forward(cfg, w, long_toks), plain.forward(cfg, w, short_toks)
    tol = F32_TOL * max(1.0, float(ref_a.abs().max()), float(ref_b.abs().max()))
    assert float((got[0] - ref_a[4169]).abs().max()) < tol and float((got[1] - ref_b[30]).abs().max()) < tol
    for i in range(4):
        got = e.step([StepEntry(a, long_toks[4170 + i:4171 + i], [0]), StepEntry(b, short_toks[31 + i:32 + i], [0])]).cpu()
        assert float((got[0] - ref_a[4170 + i]).abs().max()) < tol and float((got[1] - ref_b[31 + i]).abs().max()) < tol
    assert a.length == 4174 and b.length == 35
    e.cache.check()


def test_portions_dealt_out_differently_share_a_tape(tmp_path):
    """Steps that agree in their tokens, entries and bounds, and in what the attention planner says its plan
    depends on (the tile and the number of tiles), share a recorded tape however the tokens are dealt out over
    the portions: the tile lists and the entries' starts are data, not shapes.  Four such steps in a row, the last
    two from the tape, against the plain implementation."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "A")
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["A"]
    e = Engine.from_folder(folder, "float32", SchedulerConfig(num_kv_blocks=3 * (832 // ps + 2), kv_block_size=ps, max_batch_requests=4))
    e.use_graphs = False
    toks = {r: traces.random_tokens(cfg["vocab_size"], 800, seed=30 + i) for i, r in enumerate("abx")}
    ref = {r: plain.forward(cfg, w, t) for r, t in toks.items()}
    seqs = {r: e.open(r) for r in toks}
    fed = {}
    for r, n in (("a", 520), ("b", 520), ("x", 20)):      # far enough in that the block tables keep their width
        e.step([StepEntry(seqs[r], toks[r][:n], [])])
        fed[r] = n
    tol = F32_TOL * max(1.0, max(float(v.abs().max()) for v in ref.values()))
    for na, nb in ((70, 60), (10, 100), (128, 50), (64, 65)):          # 128 + 64, 64 + 128, 128 + 64, 64 + 128 tokens as run
        plan = [("a", na), ("b", nb), ("x", 1)]
        got = e.step([StepEntry(seqs[r], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in plan]).cpu()
        for row, (r, n) in enumerate(plan):
            fed[r] += n
            assert float((got[row] - ref[r][fed[r] - 1]).abs().max()) < tol, (plan, r)
    mixed = [k for k in e._prompt_graphs if k[1] > 0]
    assert len(mixed) == 1 and mixed[0][2] == 192 and e.tape_runs >= 2, (mixed, e.tape_runs)
    # a step with another number of tokens is another shape
    e.step([StepEntry(seqs["a"], toks["a"][fed["a"]:fed["a"] + 6], [5]), StepEntry(seqs["x"], toks["x"][fed["x"]:fed["x"] + 1], [0])])
    assert len([k for k in e._prompt_graphs if k[1] > 0]) == 2
    e.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_fewer_and_fewer_requests_share_a_shape(tmp_path, dtype):
    """Requests end one by one: steps of 7, 6 and 5 decoding requests all run as 8 entries (the rest belong to no
    request), so they share one recorded shape; every request's logits are the plain implementation's, and the
    pages of a request that ended serve a new one."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.parts.rows import few_rows_entries as decode_entries_at_least
    assert [decode_entries_at_least(n) for n in (1, 2, 3, 5, 9, 16, 17, 33, 64, 65, 100, 128, 129, 256)] == \
        [1, 2, 4, 8, 16, 16, 32, 48, 64, 80, 112, 128, 160, 256]
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "C", dtype=store, std=tiny_configs.SHARP_STD)
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["C"]
    e = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=8 * (64 // ps + 1), kv_block_size=ps, max_batch_requests=8))
    e.use_graphs = False
    names = list("abcdefg")
    toks = {r: traces.random_tokens(cfg["vocab_size"], 40, seed=40 + i) for i, r in enumerate(names + ["h"])}
    ref = {r: plain.forward(cfg, w, t) for r, t in toks.items()}
    seqs, fed = {}, {}

    def prefill(r, n):
        seqs[r] = e.open(r)
        e.step([StepEntry(seqs[r], toks[r][:n], [])])
        fed[r] = n

    def decode(rs):
        got = e.step([StepEntry(seqs[r], toks[r][fed[r]:fed[r] + 1], [0]) for r in rs]).cpu()
        assert got.shape[0] == len(rs)
        for row, r in enumerate(rs):
            d = (got[row] - ref[r][fed[r]]).abs()
            scale = float(ref[r].abs().max())
            if dtype == "float32":
                assert float(d.max()) < F32_TOL * max(1.0, scale), (rs, r)
            else:
                assert bf16_within(float(d.max()), float(d.mean()), scale), (rs, r)
            fed[r] += 1

    for i, r in enumerate(names):
        prefill(r, 5 + i)
    live = list(names)
    for _ in range(3):
        for _ in range(3):
            decode(live)
        e.close(seqs.pop(live.pop(1)))
    assert len(live) == 4
    shapes = [k for k in e._graphs]
    assert len(shapes) == 1 and shapes[0][0] == 8, shapes
    assert e.tape_runs >= 6
    prefill("h", 9)                                     # takes pages that were given back
    for _ in range(4):
        decode(live + ["h"])
    assert len(e._graphs) == 1
    decode(live)                                        # four requests: a shape of its own
    assert sorted(k[0] for k in e._graphs) == [4, 8]
    e.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_decode_steps_that_want_some_rows_only(tmp_path, dtype, graphs):
    """Four requests decode; which of them want their logits changes from step to step (all, two of them, another
    two, one, none, all again).  Steps that want every row pick no rows at all, the others do: they are different
    kinds of steps although they have as many entries and, padded, as many wanted rows, and each wanted row is its
    own request's whichever kind ran before."""
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "A", dtype=store, std=tiny_configs.SHARP_STD)
    cfg, w = plain.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["A"]
    e = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=4 * (64 // ps + 1), kv_block_size=ps, max_batch_requests=4))
    e.use_graphs, e.graph_after = graphs, 2
    names = list("abcd")
    toks = {r: traces.random_tokens(cfg["vocab_size"], 48, seed=70 + i) for i, r in enumerate(names)}
    ref = {r: plain.forward(cfg, w, t) for r, t in toks.items()}
    seqs, fed = {}, {}
    for i, r in enumerate(names):
        seqs[r] = e.open(r)
        e.step([StepEntry(seqs[r], toks[r][:4 + i], [])])
        fed[r] = 4 + i
    # (a name twice: the request asks for its one row twice, and a step may then want more rows than it has entries)
    patterns = ["abcd", "abcd", "ac", "ac", "bd", "abcd", "c", "", "ac", "abd", "abcd", "bd", "bd", "bd", "abcd",
                "aabbcd", "aabbcd", "aaccd", "abcd", "bbbb", "bbbb"]
    for wanting in patterns:
        got = e.step([StepEntry(seqs[r], toks[r][fed[r]:fed[r] + 1], [0] * wanting.count(r)) for r in names])
        assert (got is None) == (not wanting) and (got is None or got.shape[0] == len(wanting))
        for row, r in enumerate(wanting):
            d = (got[row].cpu() - ref[r][fed[r]]).abs()
            scale = float(ref[r].abs().max())
            if dtype == "float32":
                assert float(d.max()) < F32_TOL * max(1.0, scale), (wanting, r)
            else:
                assert bf16_within(float(d.max()), float(d.mean()), scale), (wanting, r)
        for r in names:
            fed[r] += 1
    assert e.tape_runs + e.graph_replays > 0 and (e.graph_replays > 0) == graphs
