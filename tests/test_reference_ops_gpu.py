"""Every kernel family beside its plain C++ reference (zedinfer_amd/csrc/host/reference_ops.cpp, compiled with the
host compiler): the kernel on the GPU and the reference on the CPU get the same inputs, rounded to the storage
type first, in 32 bits and in bfloat16."""
import math
import random

import pytest
import torch

import reference_ops
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from zedinfer_amd import ops as o
    o.load()
    return o


@pytest.fixture(scope="module")
def ref():
    r = reference_ops.load()
    if r is None:
        pytest.skip("no host C++ compiler")
    return r


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


def close(got, want, dtype, f32=2e-5, bf16=2e-2):
    t = f32 if dtype == torch.float32 else bf16
    torch.testing.assert_close(got.float().cpu(), want.float(), atol=t * max(1.0, float(want.abs().max())), rtol=t)


@pytest.mark.parametrize("dtype", DT)
def test_embedding_norms_activation_argmax(ops, ref, dtype):
    table = rnd(77, 200, dtype=dtype, seed=1)
    ids = torch.tensor([5, 76, 0, 33, 5], dtype=torch.int32, device="cuda")
    assert torch.equal(ops.embedding(ids, table, out_dtype=torch.float32).cpu(), ref.embedding(table, ids))
    for n, H, eps in ((3, 200, 1e-6), (70, 33 * 8, 1e-5)):
        x, w = rnd(n, H, dtype=dtype, scale=2.0, seed=2), (1.0 + rnd(H, scale=0.1, seed=3)).to(dtype)
        close(ops.rms_norm(x, w, eps), ref.rms_norm(x, w, eps), dtype)
        close(ops.rms_norm(x, w, eps, add_one=True), ref.rms_norm(x, w, eps, add_one=True), dtype)
        resid, delta = rnd(n, H, seed=4), rnd(n, H, dtype=dtype, seed=5)
        want_resid, want = ref.add_rms_norm(resid, delta, w, eps)
        got = ops.add_rms_norm(resid, delta, w, eps)                       # resid changes in place
        close(resid, want_resid, torch.float32)
        close(got, want, dtype)
    gate, up = rnd(9, 176, dtype=dtype, scale=3.0, seed=6), rnd(9, 176, dtype=dtype, seed=7)
    close(ops.swiglu(gate, up), ref.swiglu(gate, up), dtype)
    logits = rnd(6, 1000, dtype=dtype, seed=8)
    logits[2, 17] = logits[2, 900] = 50.0
    assert ops.argmax(logits).cpu().tolist() == ref.argmax(logits).tolist()


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M,N,K", [(3, 136, 72), (40, 200, 264), (70, 152, 136), (125, 264, 520), (200, 72, 1000),
                                   (160, 520, 64536)])
def test_products(ops, ref, dtype, M, N, K):
    """1..16 rows, 17..64 rows, 65..128 rows, the library's many rows and (a weight with many more columns than
    rows) the kernel for 129..256 rows in bfloat16; the plain product in 32 bits."""
    x, w, b = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, scale=0.1, seed=2), rnd(N, dtype=dtype, seed=3)
    close(ops.linear(x, w, b), ref.linear(x, w, b), dtype)
    close(ops.linear(x, w, out_dtype=torch.float32), ref.linear(x, w), dtype, bf16=2e-3)
    if dtype == torch.bfloat16 and ops.linear_sums_supported(x, w):
        # the same product as partial sums (the kernels for up to 64 and for 65..128 rows), added by the consumer
        close(ops.reduce_sums(ops.linear_sums(x, w), b, out_dtype=torch.float32), ref.linear(x, w, b), dtype, bf16=2e-3)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,d,rot,ps,window", [(6, 2, 48, 48, 8, 0), (4, 1, 64, 32, 16, 40), (12, 2, 128, 128, 16, 0)])
def test_rotation_store_and_attention(ops, ref, dtype, nh, nkv, d, rot, ps, window):
    """Three sequences' tokens are rotated and stored through shuffled tables by the kernel and by the reference;
    then a portion of one sequence beside single tokens of the others attends over what the kernel stored: the
    plain kernel in both types, the matrix-core prompt and decode kernels in bfloat16."""
    theta, lens = 5e4, [150, 70, 33]
    scale = 1.0 / math.sqrt(d)
    pages_each = [-(-n // ps) for n in lens]
    num_pages = sum(pages_each) + 2
    order = list(range(num_pages))
    random.Random(3).shuffle(order)
    tables = torch.full((3, max(pages_each) + 1), -1, dtype=torch.int32)
    at = 0
    for s, np_ in enumerate(pages_each):
        tables[s, :np_] = torch.tensor(order[at:at + np_], dtype=torch.int32)
        at += np_
    seq = torch.tensor([s for s, n in enumerate(lens) for _ in range(n)], dtype=torch.int32)
    pos = torch.tensor([j for n in lens for j in range(n)], dtype=torch.int32)
    slots = torch.tensor([int(tables[s, j // ps]) * ps + j % ps for s, n in enumerate(lens) for j in range(n)], dtype=torch.int32)
    n = int(pos.numel())
    qkv = rnd(n, (nh + 2 * nkv) * d, dtype=dtype, seed=1)
    q, k, v = qkv[:, :nh * d], qkv[:, nh * d:(nh + nkv) * d], qkv[:, (nh + nkv) * d:]
    # the reference's side first: the kernel rotates q in place
    q_ref = ref.rope_neox(q.reshape(n, nh, d), pos, theta, rotary_dim=rot)
    k_ref = ref.rope_neox(k.reshape(n, nkv, d), pos, theta, rotary_dim=rot)
    kc_ref, vc_ref = ref.empty_cache(num_pages, nkv, d, ps)
    ref.kv_store(kc_ref, vc_ref, k_ref, v.reshape(n, nkv, d), slots)
    kc = torch.full((num_pages, nkv, ps, d), float("nan"), dtype=dtype, device="cuda")
    vc = torch.full((num_pages, nkv, d, ps), float("nan"), dtype=dtype, device="cuda")
    ops.rope_kv_store(q, k, v, ops.rope_table(pos.cuda(), ops.rope_inv_freq(rot, theta, "cuda")), slots.cuda(), kc, vc,
                      nh, nkv, d)
    close(q.reshape(n, nh, d), q_ref, dtype, f32=5e-4)
    stored = ~torch.isnan(kc_ref)
    assert torch.equal(torch.isnan(kc).cpu(), ~stored) and torch.equal(torch.isnan(vc).cpu(), torch.isnan(vc_ref))
    close(torch.nan_to_num(kc), torch.nan_to_num(kc_ref), dtype, f32=5e-4)
    assert torch.equal(torch.nan_to_num(vc).float().cpu(), torch.nan_to_num(vc_ref))     # values are copied
    # queries: the last 40 tokens of the first sequence (a portion on top of 110 cached tokens) and the last token
    # of the other two; both sides read the cache the kernel made
    rows = list(range(lens[0] - 40, lens[0])) + [lens[0] + lens[1] - 1, n - 1]
    rows_t = torch.tensor(rows)
    qs = q[rows_t.cuda()].contiguous()
    tok_seq, tok_pos = seq[rows_t].contiguous(), pos[rows_t].contiguous()
    want = ref.paged_attention(qs.reshape(-1, nh, d), torch.nan_to_num(kc, nan=1e30).float().cpu(),
                               torch.nan_to_num(vc, nan=1e30).float().cpu(), tables, tok_seq, tok_pos, scale, window)
    assert float(want.abs().max()) < 1e3                                    # no slot that was never stored was read
    bt = tables.cuda()
    got = ops.attention(qs, kc, vc, tok_seq.cuda(), tok_pos.cuda(), bt, nh, nkv, d, scale, window)
    close(got.reshape(-1, nh, d), want, dtype)
    if dtype == torch.bfloat16:
        assert ops.attention_decode_supported(dtype, nh, nkv, d, ps) and ops.attention_prefill_supported(dtype, nh, nkv, d, ps)
        single = torch.tensor([40, 41, 0, 39], dtype=torch.int32, device="cuda")          # the two last tokens, and two of the portion
        out = torch.zeros_like(qs)
        ops.attention_decode(qs, kc, vc, tok_seq.cuda(), tok_pos.cuda(), bt, nh, nkv, d, scale, max(lens), window,
                             out=out, tok_index=single)
        close(out[single.long()].reshape(-1, nh, d), want[single.long().cpu()], dtype)
        dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
        out2 = torch.zeros_like(qs)
        ops.attention_prefill(qs, kc, vc, dev([0]), dev([0]), dev([0]), dev([40]), dev([lens[0] - 40]), bt, nh, nkv, d,
                              scale, window, out=out2)
        close(out2[:40].reshape(-1, nh, d), want[:40], dtype)


@pytest.mark.parametrize("seed", range(3))
def test_sampling(ops, ref, seed):
    rng = random.Random(seed)
    V, R = 1000, 12
    logits = rnd(R, V, scale=2.0, seed=seed)
    temperature = [rng.choice([0.7, 1.0, 1.5]) for _ in range(R)]
    temperature[-1] = 0.0
    top_k = [rng.choice([0, 1, 5, 40, 2000]) for _ in range(R)]
    top_p = [rng.choice([1.0, 0.9, 0.5, 0.05]) for _ in range(R)]
    penalty = [rng.choice([1.0, 1.3]) for _ in range(R)]
    uniform = [rng.random() for _ in range(R)]
    recent = torch.tensor([[rng.randrange(V) for _ in range(6)] for _ in range(R)], dtype=torch.int32)
    recent_len = torch.tensor([rng.randrange(7) for _ in range(R)], dtype=torch.int32)
    f = lambda v: torch.tensor(v, dtype=torch.float32)  # noqa: E731
    want = ref.sample(logits, f(temperature), torch.tensor(top_k), f(top_p), f(penalty), f(uniform), recent, recent_len).tolist()
    got = ops.sample(logits, f(temperature).cuda(), torch.tensor(top_k, dtype=torch.int32).cuda(), f(top_p).cuda(),
                     f(penalty).cuda(), f(uniform).cuda(), recent.cuda(), recent_len.cuda()).cpu().tolist()
    for r in range(R):
        if got[r] == want[r]:
            continue
        # a draw within rounding of a boundary of the running sum may fall to either neighbour
        probs, ids = plain.truncated_distribution(logits[r].cpu(), temperature[r], top_k[r], top_p[r], penalty[r],
                                                  recent[r, :int(recent_len[r])].tolist())
        run = torch.cumsum(probs.double(), 0)
        near = [int(ids[i]) for i in range(len(ids)) if abs(float(run[i]) - uniform[r]) < 1e-4 or
                (i > 0 and abs(float(run[i - 1]) - uniform[r]) < 1e-4)]
        assert got[r] in near and want[r] in near, (r, got[r], want[r])
