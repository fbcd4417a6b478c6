"""The plain C++ references of the operators (zedinfer_amd/csrc/host/reference_ops.cpp) against the plain Python
implementation, on the CPU: two implementations written apart from the same formulas must agree, on whole
sequences laid into a paged cache through shuffled block tables."""
import math
import random

import pytest
import torch

import reference_ops
from plain import qwen2_plain as plain


@pytest.fixture(scope="module")
def ref():
    r = reference_ops.load()
    if r is None:
        pytest.skip("no host C++ compiler")
    return r


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return torch.randn(*shape, generator=g) * scale


def close(a, b, tol=2e-6):
    scale = max(1.0, float(b.abs().max()))
    assert float((a.double() - b.double()).abs().max()) <= tol * scale


def test_embedding_and_its_loud_bad_id(ref):
    table = rnd(23, 10)
    out = ref.embedding(table, [3, 0, 22, 23, -1])
    assert torch.equal(out[:3], plain.embedding(torch.tensor([3, 0, 22]), table))
    assert torch.isnan(out[3:]).all()


@pytest.mark.parametrize("n,width,eps", [(3, 33, 1e-6), (1, 200, 1e-5), (5, 8, 0.1)])
def test_norms(ref, n, width, eps):
    x, w, delta = rnd(n, width, seed=1, scale=3.0), 1.0 + rnd(width, seed=2, scale=0.1), rnd(n, width, seed=3)
    close(ref.rms_norm(x, w, eps), plain.rms_norm(x.double(), w.double(), eps))
    close(ref.rms_norm(x, w, eps, add_one=True), plain.rms_norm(x.double(), 1.0 + w.double(), eps))
    resid, normed = ref.add_rms_norm(x, delta, w, eps)
    assert torch.equal(resid, x + delta)
    close(normed, plain.rms_norm((x + delta).double(), w.double(), eps))
    # the eps is inside the root: with a row of zeros the result is zero, not NaN
    assert float(ref.rms_norm(torch.zeros(1, width), w, eps).abs().max()) == 0.0


def test_linear_swiglu_argmax(ref):
    x, w, b = rnd(7, 33, seed=1), rnd(19, 33, seed=2), rnd(19, seed=3)
    close(ref.linear(x, w, b), plain.linear(x.double(), w.double(), b.double()))
    close(ref.linear(x, w), plain.linear(x.double(), w.double()))
    g, u = rnd(5, 40, seed=4, scale=4.0), rnd(5, 40, seed=5)
    close(ref.swiglu(g, u), plain.swiglu(g.double(), u.double()))
    logits = rnd(4, 50, seed=6)
    logits[1, 7] = logits[1, 30] = 9.0                  # equals: the lowest index
    logits[2, 0] = float("nan")                         # NaN never wins
    logits[3] = float("-inf")
    got = ref.argmax(logits).tolist()
    assert got[0] == plain.argmax_lowest_index(logits[0]) and got[1] == 7
    assert got[2] == int(torch.argmax(torch.nan_to_num(logits[2], nan=-1e30))) and got[3] == 0


@pytest.mark.parametrize("heads,d,theta,start", [(3, 16, 10000.0, 0), (2, 48, 1e6, 1000), (1, 6, 50.0, 7)])
def test_rotation(ref, heads, d, theta, start):
    n = 9
    x = rnd(n, heads, d, seed=1)
    pos = torch.arange(start, start + n, dtype=torch.int32)
    close(ref.rope_neox(x, pos, theta), plain.rope_neox(x.double(), pos, theta), 1e-5)
    # only the first dims rotate when rotary_dim is smaller; the pairing is then within those dims
    rd = d // 2 if (d // 2) % 2 == 0 else d // 2 + 1
    part = ref.rope_neox(x, pos, theta, rotary_dim=rd)
    close(part[..., :rd], plain.rope_neox(x[..., :rd].double(), pos, theta), 1e-5)
    assert torch.equal(part[..., rd:], x[..., rd:])
    # position 0 turns nothing
    assert torch.equal(ref.rope_neox(x, torch.zeros(n, dtype=torch.int32), theta), x)


@pytest.mark.parametrize("nh,nkv,d,ps,lens,window", [(4, 2, 16, 8, [37, 5, 20], 0), (3, 1, 24, 4, [30, 9], 7),
                                                     (6, 6, 8, 16, [16, 17, 1], 0), (5, 1, 10, 3, [25], 25)])
def test_attention_over_the_paged_cache(ref, nh, nkv, d, ps, lens, window):
    """Whole sequences go into the cache through shuffled tables (one store for all, as a step with several
    portions does); every token's attention equals the plain implementation's over its own sequence, whether all
    tokens are asked for at once (prompts) or a few (decoding), and a slot that was never stored is never read."""
    scale = 1.0 / math.sqrt(d)
    pages_each = [-(-n // ps) for n in lens]
    num_pages = sum(pages_each) + 3
    order = list(range(num_pages))
    random.Random(5).shuffle(order)
    width = max(pages_each) + 1
    tables = torch.full((len(lens), width), -1, dtype=torch.int32)
    at = 0
    for s, np_ in enumerate(pages_each):
        tables[s, :np_] = torch.tensor(order[at:at + np_], dtype=torch.int32)
        at += np_
    qs = [rnd(n, nh, d, seed=10 + s) for s, n in enumerate(lens)]
    ks = [rnd(n, nkv, d, seed=20 + s) for s, n in enumerate(lens)]
    vs = [rnd(n, nkv, d, seed=30 + s) for s, n in enumerate(lens)]
    seq = torch.tensor([s for s, n in enumerate(lens) for _ in range(n)], dtype=torch.int32)
    pos = torch.tensor([j for n in lens for j in range(n)], dtype=torch.int32)
    slots = torch.tensor([int(tables[s, j // ps]) * ps + j % ps for s, n in enumerate(lens) for j in range(n)], dtype=torch.int32)
    kc, vc = ref.empty_cache(num_pages, nkv, d, ps)
    k_all = torch.cat(ks)
    k_rot = ref.rope_neox(k_all, pos, 10000.0)
    ref.kv_store(kc, vc, k_rot, torch.cat(vs), slots)
    want = torch.cat([plain.causal_gqa_attention(plain.rope_neox(q.double(), torch.arange(n), 10000.0),
                                                 plain.rope_neox(k.double(), torch.arange(n), 10000.0), v.double(), scale,
                                                 window or None) for q, k, v, n in zip(qs, ks, vs, lens)])
    q_rot = ref.rope_neox(torch.cat(qs), pos, 10000.0)
    got = ref.paged_attention(q_rot, kc, vc, tables, seq, pos, scale, window)
    assert not torch.isnan(got).any()
    close(got, want, 1e-5)
    some = torch.tensor([len(pos) - 1, 0, lens[0] - 1, lens[0] // 2])
    few = ref.paged_attention(q_rot[some], kc, vc, tables, seq[some], pos[some], scale, window)
    assert torch.equal(few, got[some])
    # a table without the page a key lies in is an error, not a read of some other page
    broken = tables.clone()
    broken[0, 0] = -1
    with pytest.raises(RuntimeError, match="page 0 of the table is -1"):
        ref.paged_attention(q_rot[:1], kc, vc, broken, seq[:1], pos[:1], scale, window)


def test_store_skips_padding_and_refuses_slots_outside_the_pool(ref):
    kc, vc = ref.empty_cache(2, 1, 4, 2)
    k, v = rnd(3, 1, 4, seed=1), rnd(3, 1, 4, seed=2)
    ref.kv_store(kc, vc, k, v, [3, -1, 0])
    assert torch.equal(kc[1, 0, 1], k[0, 0]) and torch.equal(vc[1, 0, :, 1], v[0, 0])
    assert torch.equal(kc[0, 0, 0], k[2, 0]) and torch.equal(vc[0, 0, :, 0], v[2, 0])
    assert torch.isnan(kc[0, 0, 1]).all() and torch.isnan(kc[1, 0, 0]).all()
    with pytest.raises(RuntimeError, match="the pool has 2 pages"):
        ref.kv_store(kc, vc, k, v, [4, 0, 1])


@pytest.mark.parametrize("seed", range(6))
def test_sampling_picks_what_the_truncated_distribution_says(ref, seed):
    rng = random.Random(seed)
    V, R = 97, 8
    logits = rnd(R, V, seed=seed, scale=2.0)
    logits[0, 5] = logits[0, 50] = float(logits[0].max()) + 1.0        # equal probabilities: rising id
    temperature = [rng.choice([0.7, 1.0, 1.5]) for _ in range(R)]
    top_k = [rng.choice([0, 1, 5, 40, 200]) for _ in range(R)]
    top_p = [rng.choice([1.0, 0.9, 0.5, 0.05]) for _ in range(R)]
    penalty = [rng.choice([1.0, 1.3]) for _ in range(R)]
    uniform = [rng.random() for _ in range(R)]
    uniform[0] = 0.0
    recent = torch.tensor([[rng.randrange(V) for _ in range(6)] for _ in range(R)], dtype=torch.int32)
    recent_len = torch.tensor([rng.randrange(7) for _ in range(R)], dtype=torch.int32)
    temperature[-1] = 0.0                                              # greedy row
    got = ref.sample(logits, torch.tensor(temperature), torch.tensor(top_k), torch.tensor(top_p), torch.tensor(penalty),
                     torch.tensor(uniform), recent, recent_len).tolist()
    for r in range(R - 1):
        probs, ids = plain.truncated_distribution(logits[r], temperature[r], top_k[r], top_p[r], penalty[r],
                                                  recent[r, :int(recent_len[r])].tolist())
        run = torch.cumsum(probs.double(), 0)
        hit = (run > uniform[r]).nonzero()
        want = int(ids[int(hit[0])]) if len(hit) else int(ids[-1])
        # a draw that falls within rounding of a boundary may go either way: the neighbours are allowed then
        near = [int(ids[i]) for i in range(len(ids)) if abs(float(run[i]) - uniform[r]) < 1e-5]
        assert got[r] == want or got[r] in near, (r, got[r], want)
    assert got[0] == 5
    assert got[-1] == plain.argmax_lowest_index(logits[-1])
