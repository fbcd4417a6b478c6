"""The kernels' walk over the paged cache, checked on the CPU.

zedinfer_amd/csrc/host/paging_model.cpp is compiled with the host compiler and runs the loops of the
decode attention, prompt attention and cache-store launches with the index arithmetic the kernels themselves
call (csrc/zi_paging.h): every index inside what it indexes, every visible key read once and from the page the
sequence holds for it, workspaces large enough and no place written twice.  The launches come from the cache
manager under random traffic (windows that give pages back, tables padded with -1, the padding entries and
padded portions that graph steps add); broken inputs must be reported."""
import ctypes
import os
import random
import shutil
import subprocess

import numpy as np
import pytest
import torch

from zedinfer_amd.cache import CacheManager, OutOfPages
from zedinfer_amd.parts import HostBatch
from zedinfer_amd.parts.mixers import attention_cache_request
from zedinfer_amd.parts.mixers import AttentionPlanner

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
I32 = ctypes.POINTER(ctypes.c_int)


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    lib = str(tmp_path_factory.mktemp("pm") / "paging_model.so")
    src = os.path.join(ROOT, "zedinfer_amd", "csrc", "host", "paging_model.cpp")
    subprocess.run([cxx, "-O1", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", lib, src], check=True)
    pm = ctypes.CDLL(lib)
    pm.pm_last_error.restype = ctypes.c_char_p
    for name in ("pm_decode_workspace", "pm_prefill_workspace"):
        getattr(pm, name).restype = ctypes.c_int64
    return pm


def ptr(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32).ctypes.data_as(I32)


def padded_tables(seqs, group, width):
    t = np.full((len(seqs), width), -1, dtype=np.int32)
    for i, s in enumerate(seqs):
        if s is not None:
            t[i, :len(s.pages[group])] = s.pages[group]
    return t


def pow2(n, floor):
    v = floor
    while v < n:
        v *= 2
    return v


def decode(pm, pos, tables, num_pages, nh, nkv, d, ps, window, max_chunks, slots=None, leave=False, workspace=None,
           tok_index=None, tok_seq=None):
    n = len(tok_index) if tok_index is not None else len(pos)
    ws = pm.pm_decode_workspace(n, nh, d) if workspace is None else workspace
    stats = (ctypes.c_int64 * 3)()
    rc = pm.pm_check_decode(n, ptr(tok_index), ptr(tok_seq), ptr(pos), ptr(tables), tables.shape[0], tables.shape[1],
                            num_pages, nh, nkv, d, ps, window, max_chunks, ctypes.c_int64(ws), int(leave), ptr(slots),
                            ctypes.c_int64(num_pages * ps), stats)
    return rc, pm.pm_last_error().decode(), list(stats)


def traffic(seed, window, pages=48, ps=16, requests=6):
    """A cache manager after random opens, growth and closes; returns it with its live sequences."""
    rng = random.Random(seed)
    kv = {0: attention_cache_request("full", 2, 32)}
    if window:
        kv[1] = attention_cache_request("window", 2, 32, window)
    m = CacheManager(kv, {}, pages, ps, requests, torch.bfloat16, None, max_step_tokens=64)
    live = []
    for step in range(60):
        if live and rng.random() < 0.15:
            m.close(live.pop(rng.randrange(len(live))))
        if len(live) < requests and rng.random() < 0.4:
            try:
                live.append(m.open(("r", seed, step)))
            except OutOfPages:
                pass
        for s in live:
            n = rng.choice([1, 1, 1, 2, 7, 24, 64, 100])
            try:
                m.ensure(s, s.length + n)
                m.commit(s, s.length + n)
            except OutOfPages:
                pass
    m.check()
    return m, [s for s in live if s.length > 0], rng


def growing(m, live):
    """The sequences that get a place for one more token."""
    out = []
    for s in live:
        try:
            m.ensure(s, s.length + 1)
            out.append(s)
        except OutOfPages:
            pass
    return out


@pytest.mark.parametrize("window", [0, 24, 100])
@pytest.mark.parametrize("seed", range(6))
def test_decode_walk_under_random_traffic(model, seed, window):
    m, live, rng = traffic(seed, window)
    if not live:
        return
    live = growing(m, live)             # every live sequence that can grow decodes one token
    if not live:
        return
    for g, group in enumerate(m.groups):
        ps, w = group.page_size, group.window
        seqs = list(live) + [None, None]                       # two padding entries of no request
        pos = np.array([s.length for s in live] + [0, 0], dtype=np.int32)
        slots = np.array([m.token_slots(s, g, s.length, 1)[0] for s in live] + [-1, -1], dtype=np.int32)
        width = pow2(max(len(s.pages[g]) for s in live), 8)
        tables = padded_tables(seqs, g, width)
        bound = pow2(int(pos.max()) + 1, 256)                  # the launch size a recorded step would have
        keys = min(bound, w) if w else bound
        chunks = model.pm_decode_chunks(keys)
        for leave in (False, True):
            rc, err, stats = decode(model, pos, tables, m.num_pages, 6, 2, 32, ps, w, chunks, slots, leave)
            assert rc == 0, err
            seen = sum(min(int(p) + 1, w) if w else int(p) + 1 for p in pos[:len(live)])
            assert stats[0] == 2 * seen and stats[2] == 0          # two kv heads read every visible key once
        # the rotary kernel's store of the same step
        st = (ctypes.c_int64 * 1)()
        rc = model.pm_check_store(len(pos), ptr(slots), ctypes.c_int64(m.num_pages * ps), m.num_pages, 2, 32, ps, st)
        assert rc == 0, model.pm_last_error()
        assert st[0] == len(live)
    # a subset of the tokens through an index list, with rows named by tok_seq (a mixed step's decoded tokens)
    g, ps = 0, m.groups[0].page_size
    pos = np.array([s.length for s in live], dtype=np.int32)
    tables = padded_tables(live, g, pow2(max(len(s.pages[g]) for s in live), 8))
    pick = np.array(sorted(rng.sample(range(len(live)), max(1, len(live) // 2))), dtype=np.int32)
    rc, err, _ = decode(model, pos, tables, m.num_pages, 4, 2, 32, ps, 0, model.pm_decode_chunks(int(pos.max()) + 1),
                        tok_index=pick, tok_seq=np.arange(len(live), dtype=np.int32))
    assert rc == 0, err


def test_decode_walk_reports_what_is_broken(model):
    m = CacheManager({0: attention_cache_request("full", 2, 32)}, {}, 64, 16, 4, torch.bfloat16, None, max_step_tokens=64)
    live = [m.open("a"), m.open("b")]
    for s, n in zip(live, (700, 40)):
        m.ensure(s, n)
        m.commit(s, n)
    live = growing(m, live)
    ps = m.groups[0].page_size
    pos = np.array([s.length for s in live], dtype=np.int32)
    slots = np.array([m.token_slots(s, 0, s.length, 1)[0] for s in live], dtype=np.int32)
    tables = padded_tables(live, 0, pow2(max(len(s.pages[0]) for s in live), 8))
    chunks = model.pm_decode_chunks(int(pos.max()) + 1)
    ok = decode(model, pos, tables, m.num_pages, 6, 2, 32, ps, 0, chunks, slots)
    assert ok[0] == 0, ok[1]
    longest = int(np.argmax(pos))
    broken = tables.copy()
    broken[longest, 0] = -1                                   # a page the sequence needs is gone
    rc, err, _ = decode(model, pos, broken, m.num_pages, 6, 2, 32, ps, 0, chunks, slots)
    assert rc != 0 and "page entry is -1" in err
    rc, err, _ = decode(model, pos, tables, m.num_pages, 6, 2, 32, ps, 0, chunks, slots, workspace=100)
    assert rc != 0 and "workspace" in err
    wrong = slots.copy()
    wrong[longest] += 1                                       # the new key would land beside its position
    rc, err, _ = decode(model, pos, tables, m.num_pages, 6, 2, 32, ps, 0, chunks, wrong)
    assert rc != 0 and "stores to page" in err
    rc, err, stats = decode(model, pos, tables, m.num_pages, 6, 2, 32, ps, 0, 1, slots)      # a launch sized too small
    assert rc == 0 and stats[2] > 0                           # those tokens get NaN, nothing else is touched
    st = (ctypes.c_int64 * 1)()
    twice = np.array([slots[0], slots[0]], dtype=np.int32)
    assert model.pm_check_store(2, ptr(twice), ctypes.c_int64(m.num_pages * ps), m.num_pages, 2, 32, ps, st) != 0
    assert b"two tokens" in model.pm_last_error()
    out = np.array([m.num_pages * ps], dtype=np.int32)
    assert model.pm_check_store(1, ptr(out), ctypes.c_int64(m.num_pages * ps), m.num_pages, 2, 32, ps, st) != 0


def prefill(pm, plan, hb, real, tables, num_pages, nh, nkv, d, ps, window, max_chunks, workspace=None, tile=64):
    """``tile``: 64, 128, or -128 for tiles of 128 queries in workgroups of four wavefronts (blocks of 64 keys)."""
    alone, tile = int(tile < 0), abs(tile)
    rows = hb.num_tokens
    ws = pm.pm_prefill_workspace(rows, nh, d, max_chunks) if workspace is None else workspace
    stats = (ctypes.c_int64 * 3)()
    rc = pm.pm_check_prefill(plan.sizes["num_tiles"], ptr(plan.arrays["tile_entry"]), ptr(plan.arrays["tile_off"]),
                             ptr(hb.entry_start), ptr(hb.entry_len), ptr(hb.entry_past), ptr(real), hb.num_entries,
                             ptr(tables), tables.shape[1], num_pages, nh, nkv, d, ps, window, rows, max_chunks,
                             ctypes.c_int64(ws), tile, alone, stats)
    return rc, pm.pm_last_error().decode(), list(stats)


@pytest.mark.parametrize("tile", [64, 128, -128])
@pytest.mark.parametrize("window", [0, 24, 100])
@pytest.mark.parametrize("seed", range(5))
def test_prefill_walk_under_random_traffic(model, seed, window, tile):
    """Portions of prompts after whatever the sequences hold, cut into tiles by the attention's own planner;
    once as they are, once padded to multiples of 64 tokens as recorded steps run them."""
    m, live, rng = traffic(seed + 20, window, pages=400, ps=8)
    if not live:
        return
    portions = []
    for s in live:
        n = rng.choice([5, 17, 64, 65, 130, 200])
        try:
            m.ensure(s, s.length + n)
            portions.append((s, n))
        except OutOfPages:
            pass
    if not portions:
        return
    for pad in (0, 64):
        lens = np.array([-(-n // pad) * pad if pad else n for _, n in portions], dtype=np.int32)
        real = np.array([n for _, n in portions], dtype=np.int32)
        starts = np.zeros(len(portions), dtype=np.int32)
        starts[1:] = np.cumsum(lens)[:-1]
        past = np.array([s.length for s, _ in portions], dtype=np.int32)
        hb = HostBatch(int(lens.sum()), len(portions), starts, lens, past, False)
        planner = AttentionPlanner(abs(tile), heads=6)
        planner.FILL = 1 if abs(tile) == 128 else planner.FILL   # take the wide tiles however small the step
        planner.FILL_ALONE = 1 if tile < 0 else 10 ** 9
        plan = planner.plan(hb)
        assert plan.sizes["num_long"] == int(lens.sum()) and plan.sizes["tile"] == abs(tile)
        assert plan.sizes["alone"] == (tile < 0)
        for g, group in enumerate(m.groups):
            tables = padded_tables([s for s, _ in portions], g, pow2(max(len(s.pages[g]) for s, _ in portions), 8))
            keys = plan.sizes["max_long_keys"]
            if group.window:
                keys = min(keys, group.window + 128 + 128) + 2047
            chunks = model.pm_prefill_chunks(keys)
            rc, err, stats = prefill(model, plan, hb, real, tables, m.num_pages, 6, 2, 32, group.page_size, group.window,
                                     chunks, tile=tile)
            assert rc == 0, err
            assert stats[0] > 0 and stats[2] == 0


@pytest.mark.parametrize("tile", [64, 128, -128])
def test_prefill_walk_of_a_long_prompt_and_what_is_broken(model, tile):
    """One portion that continues a long sequence: its tiles are cut along the keys every 2,048, and the cuts'
    partial results have places of their own in the workspace."""
    m = CacheManager({0: attention_cache_request("full", 2, 32)}, {}, 700, 8, 2, torch.bfloat16, None, max_step_tokens=2048)
    s = m.open("long")
    m.ensure(s, 4100)
    m.commit(s, 4100)
    m.ensure(s, 4100 + 300)
    hb = HostBatch(300, 1, np.array([0], dtype=np.int32), np.array([300], dtype=np.int32),
                   np.array([4100], dtype=np.int32), False)
    planner = AttentionPlanner(abs(tile), heads=4)
    planner.FILL = 1
    planner.FILL_ALONE = 1 if tile < 0 else 10 ** 9
    plan = planner.plan(hb)
    assert plan.sizes["tile"] == abs(tile) and plan.sizes["alone"] == (tile < 0)
    tables = padded_tables([s], 0, pow2(len(s.pages[0]), 8))
    chunks = model.pm_prefill_chunks(plan.sizes["max_long_keys"])
    assert chunks == 3
    rc, err, stats = prefill(model, plan, hb, None, tables, m.num_pages, 4, 2, 32, 8, 0, chunks, tile=tile)
    assert rc == 0, err
    assert stats[0] == sum(4100 + i + 1 for i in range(300)) and stats[1] == 300 * 4 * 3
    rc, err, _ = prefill(model, plan, hb, None, tables, m.num_pages, 4, 2, 32, 8, 0, chunks, workspace=1000, tile=tile)
    assert rc != 0 and "workspace" in err
    broken = tables.copy()
    broken[0, 300] = -1
    rc, err, _ = prefill(model, plan, hb, None, broken, m.num_pages, 4, 2, 32, 8, 0, chunks, tile=tile)
    assert rc != 0 and "page entry" in err
    rc, err, stats = prefill(model, plan, hb, None, tables, m.num_pages, 4, 2, 32, 8, 0, 2, tile=tile)    # sized for fewer cuts
    assert rc == 0 and stats[2] == plan.sizes["num_tiles"]


@pytest.mark.parametrize("tile", [64, 128, -128])
def test_prefill_walk_with_the_cut_of_long_prompts(model, tile):
    """Launches of 768 tiles x heads and more whose queries see more than 6,144 keys cut their tiles every 16,384
    keys instead of every 2,048 (they fill the chip without cuts, and every cut costs a merge): a portion behind 17,000 tokens walks its
    keys in two cuts, every (query, key) pair once, its block table entries within what the kernel stages; a
    portion behind 7,000 in one, with no workspace."""
    m = CacheManager({0: attention_cache_request("full", 2, 32)}, {}, 2300, 8, 2, torch.bfloat16, None, max_step_tokens=2048)
    assert model.pm_prefill_chunk_for(6144, 5000) == 2048 and model.pm_prefill_chunk_for(6145, 768) == 16384
    assert model.pm_prefill_chunk_for(30000, 767) == 2048
    for past, cuts in ((17000, 2), (7000, 1)):
        s = m.open(f"long{past}")
        m.ensure(s, past)
        m.commit(s, past)
        m.ensure(s, past + 300)
        hb = HostBatch(300, 1, np.array([0], dtype=np.int32), np.array([300], dtype=np.int32),
                       np.array([past], dtype=np.int32), False)
        planner = AttentionPlanner(abs(tile), heads=4)
        planner.FILL = 1
        planner.FILL_ALONE = 1 if tile < 0 else 10 ** 9
        plan = planner.plan(hb)
        tables = padded_tables([s], 0, pow2(len(s.pages[0]), 8))
        keys = plan.sizes["max_long_keys"]
        before = model.pm_set_prefill_chunk(model.pm_prefill_chunk_for(keys, 1000))       # as in a launch of many tiles
        try:
            assert before == 2048 and model.pm_prefill_chunks(keys) == cuts
            rc, err, stats = prefill(model, plan, hb, None, tables, m.num_pages, 4, 2, 32, 8, 0, cuts, tile=tile)
        finally:
            model.pm_set_prefill_chunk(before)
        assert rc == 0, err
        assert stats[0] == sum(past + i + 1 for i in range(300)) and stats[1] == (300 * 4 * cuts if cuts > 1 else 0)
        if past == 17000:
            # the same portion with a window of 7,000 keys: every tile's keys lie across the cut at 16,384
            window = 7000
            before = model.pm_set_prefill_chunk(16384)
            try:
                rc, err, stats = prefill(model, plan, hb, None, tables, m.num_pages, 4, 2, 32, 8, window, 2, tile=tile)
            finally:
                model.pm_set_prefill_chunk(before)
            assert rc == 0, err
            assert stats[0] == 300 * window and stats[1] == 300 * 4 * 2
        m.close(s)
