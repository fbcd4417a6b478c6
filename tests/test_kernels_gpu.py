"""Each HIP kernel alone against a plain float32 torch reference of the same op, at sizes other
than the tiny models' (widths that are no power of two, odd head counts, several page sizes)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]


def tol(dtype, f32=1e-5, bf16=2e-2):
    return dict(atol=f32, rtol=f32) if dtype == torch.float32 else dict(atol=bf16, rtol=bf16)


@pytest.fixture(scope="module")
def ops():
    from zedinfer_amd import ops as o
    o.load()
    assert o.library_path() is not None
    return o


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,H,V", [(1, 48, 100), (37, 1536, 3000), (5, 200, 77)])
def test_embedding(ops, dtype, n, H, V):
    table = rnd(V, H, dtype=dtype)
    ids = torch.randint(0, V, (n,), dtype=torch.int32, device="cuda")
    out = ops.embedding(ids, table, out_dtype=torch.float32)
    assert torch.equal(out, table[ids.long()].float())
    out2 = ops.embedding(ids, table)
    assert torch.equal(out2, table[ids.long()])


def test_embedding_bad_id_is_loud(ops):
    table = rnd(10, 32)
    ids = torch.tensor([3, 11], dtype=torch.int32, device="cuda")
    out = ops.embedding(ids, table)
    assert torch.isnan(out[1]).all() and not torch.isnan(out[0]).any()


@pytest.mark.parametrize("dtype", DT)
def test_gather_rows(ops, dtype):
    x = rnd(50, 72, dtype=dtype)
    idx = torch.tensor([49, 0, 7, 7], dtype=torch.int32, device="cuda")
    assert torch.equal(ops.gather_rows(x, idx), x[idx.long()])


@pytest.mark.parametrize("dtype", DT)
def test_add(ops, dtype):
    a, b = rnd(33, 100, dtype=dtype, seed=1), rnd(33, 100, dtype=dtype, seed=2)
    ref = (a.float() + b.float()).to(dtype)
    assert torch.equal(ops.add(a, b), ref)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,I", [(1, 176), (9, 8960), (70000, 8)])
def test_swiglu(ops, dtype, n, I):
    gu = rnd(n, 2 * I, dtype=dtype, scale=3.0)
    g, u = gu[:, :I], gu[:, I:]
    ref = (torch.nn.functional.silu(g.float()) * u.float())
    out = ops.swiglu(g, u)
    torch.testing.assert_close(out.float(), ref.to(dtype).float(), **tol(dtype, 1e-6, 1e-2))


@pytest.mark.parametrize("n,I", [(64, 64), (136, 200), (8, 8), (2048, 8960), (72, 1000)])
def test_swiglu_from_the_transposed_product(ops, n, I):
    """[2I, n] with gate and up rows in blocks of 8 in, [n, I] out: the same bits as the kernel for the
    product the usual way round."""
    gu = rnd(n, 2 * I, dtype=torch.bfloat16, scale=3.0)                 # 8 gate columns, their 8 up columns, ...
    want = ops.swiglu(gu, interleave=8)
    got = ops.swiglu_t(gu.t().contiguous())
    assert torch.equal(got, want)
    x, w = rnd(n, 96, dtype=torch.bfloat16, seed=1), rnd(2 * I, 96, dtype=torch.bfloat16, scale=0.1, seed=2)
    torch.testing.assert_close(ops.linear_transposed(x, w).float(), ops.linear(x, w).float().t(), atol=2e-2, rtol=2e-2)
    with pytest.raises(ValueError, match="multiples of 8"):
        ops.swiglu_t(torch.zeros(32, 12, dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,H,eps", [(1, 1536, 1e-6), (7, 100, 1e-5), (3, 5120, 1e-6), (2, 33, 0.1)])
def test_rms_norm(ops, dtype, n, H, eps):
    x = rnd(n, H, dtype=dtype, scale=2.0)
    w = (1 + 0.1 * torch.randn(H)).to(dtype).cuda()
    xf = x.float()
    ref = w.float() * xf / torch.sqrt((xf * xf).mean(-1, keepdim=True) + eps)
    out = ops.rms_norm(x, w, eps)
    torch.testing.assert_close(out.float(), ref, **tol(dtype))
    # w = 1 reduces to the library routine
    one = torch.ones(H, dtype=dtype, device="cuda")
    lib = torch.nn.functional.rms_norm(xf, (H,), eps=eps)
    torch.testing.assert_close(ops.rms_norm(x, one, eps).float(), lib, **tol(dtype))
    # (1 + w) form
    out1 = ops.rms_norm(x, w, eps, add_one=True)
    torch.testing.assert_close(out1.float(), ref / w.float() * (w.float() + 1), **tol(dtype, 1e-4, 3e-2))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,H", [(6, 200), (64, 1536), (201, 72), (130, 5120), (77, 3584), (66, 8192), (65, 34)])
def test_add_rms_norm(ops, dtype, n, H):
    """Few rows (a workgroup a row) and many (a wavefront a row), widths of every number of 1 KB runs,
    and one that is no multiple of four (the plain kernel)."""
    eps = 1e-6
    resid = rnd(n, H, seed=3)
    delta = rnd(n, H, dtype=dtype, seed=4)
    w = rnd(H, dtype=dtype, seed=5)
    s = resid + delta.float()
    ref = w.float() * s / torch.sqrt((s * s).mean(-1, keepdim=True) + eps)
    r = resid.clone()
    out = ops.add_rms_norm(r, delta, w, eps)
    assert torch.equal(r, s)
    torch.testing.assert_close(out.float(), ref, **tol(dtype))


def torch_rope(x, pos, theta):
    """python/tests/ops/rope.py:7-30 of the reference."""
    d = x.shape[-1]
    a, b = x[..., : d // 2], x[..., d // 2:]
    i = torch.arange(0, d // 2, dtype=torch.float32, device=x.device)
    freqs = pos.float().unsqueeze(1) / (theta ** (2 * i / d))
    sin, cos = freqs.sin().unsqueeze(1), freqs.cos().unsqueeze(1)
    return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n,nh,d,start,theta", [(5, 3, 16, 0, 10000.0), (33, 12, 128, 1024, 1e6), (4, 7, 80, 300, 5e4)])
def test_rope(ops, dtype, n, nh, d, start, theta):
    x = rnd(n, nh, d, dtype=dtype)
    pos = torch.arange(start, start + n, dtype=torch.int32, device="cuda")
    ref = torch_rope(x.float(), pos, theta)
    out = ops.rope(x, pos, ops.rope_inv_freq(d, theta, "cuda"))
    torch.testing.assert_close(out.float(), ref, **tol(dtype, 5e-4, 2e-2))


def make_paged(k, v, page_size, num_pages, perm_seed=0):
    """Scatter k, v [T, nkv, d] into the key cache [pages, nkv, page_size, d] and the transposed value
    cache [pages, nkv, d, page_size] through a shuffled table."""
    T, nkv, d = k.shape
    need = (T + page_size - 1) // page_size
    g = torch.Generator().manual_seed(perm_seed)
    table = torch.randperm(num_pages, generator=g)[:need].to(torch.int32)
    kc = torch.full((num_pages, nkv, page_size, d), float("nan"), dtype=k.dtype, device="cuda")
    vc = torch.full((num_pages, nkv, d, page_size), float("nan"), dtype=k.dtype, device="cuda")
    for t in range(T):
        p, o = int(table[t // page_size]), t % page_size
        kc[p, :, o] = k[t]
        vc[p, :, :, o] = v[t]
    return kc, vc, table.cuda()


def ref_attention(q, k, v, pos, scale, window):
    """q [n, nh, d] at absolute positions pos over k, v [T, nkv, d]; float32."""
    n, nh, d = q.shape
    nkv = k.shape[1]
    out = torch.empty_like(q)
    j = torch.arange(k.shape[0], device=q.device)
    for h in range(nh):
        g = h // (nh // nkv)
        s = (q[:, h] @ k[:, g].t()) * scale
        vis = j[None, :] <= pos[:, None]
        if window:
            vis &= (pos[:, None] - j[None, :]) < window
        s = s.masked_fill(~vis, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,d,ps,T,window", [
    (4, 2, 16, 16, 49, 0), (12, 2, 128, 16, 300, 0), (3, 1, 32, 8, 100, 0), (6, 2, 48, 8, 90, 20),
    (5, 5, 80, 4, 70, 0), (28, 4, 128, 32, 130, 64), (2, 1, 256, 16, 65, 0)])
def test_attention_generic(ops, dtype, nh, nkv, d, ps, T, window):
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1), rnd(T, nkv, d, dtype=dtype, seed=2)
    kc, vc, table = make_paged(k, v, ps, 64)
    # queries: a prompt portion at the end plus scattered single positions, in two "sequences"
    # that share the same pages through two identical table rows
    pos = torch.tensor(list(range(T - 7, T)) + [0, 1, ps - 1, ps, T // 2], dtype=torch.int32, device="cuda")
    n = pos.numel()
    q = rnd(n, nh, d, dtype=dtype, seed=3)
    seq = torch.tensor([0] * 7 + [1] * (n - 7), dtype=torch.int32, device="cuda")
    bt = torch.stack([table, table]).contiguous()
    scale = 1 / math.sqrt(d)
    out = ops.attention(q.view(n, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, window)
    ref = ref_attention(q.float(), k.float(), v.float(), pos.long(), scale, window)
    torch.testing.assert_close(out.view(n, nh, d).float(), ref, **tol(dtype, 2e-5, 2e-2))


def test_attention_far_key_stands_out(ops):
    """One far key among hundreds is made to dominate: its value must come through."""
    nh, nkv, d, ps, T = 4, 1, 64, 16, 700
    k, v = rnd(T, nkv, d, seed=1) * 0.1, rnd(T, nkv, d, seed=2)
    q = rnd(1, nh, d, seed=3)
    far = 37
    k[far, 0] = q[0, 2] * 50.0 / q[0, 2].norm() ** 2 * math.sqrt(d)   # score 50 for head 2
    kc, vc, table = make_paged(k, v, ps, 64)
    pos = torch.tensor([T - 1], dtype=torch.int32, device="cuda")
    out = ops.attention(q.view(1, nh * d), kc, vc, torch.zeros(1, dtype=torch.int32, device="cuda"), pos,
                        table[None].contiguous(), nh, nkv, d, 1 / math.sqrt(d))
    torch.testing.assert_close(out.view(nh, d)[2], v[far, 0], atol=1e-4, rtol=1e-4)
    # and with a window that ends just after it, it is gone
    out_w = ops.attention(q.view(1, nh * d), kc, vc, torch.zeros(1, dtype=torch.int32, device="cuda"), pos,
                          table[None].contiguous(), nh, nkv, d, 1 / math.sqrt(d), window=T - 1 - far)
    assert (out_w.view(nh, d)[2] - v[far, 0]).abs().max() > 0.1
    out_w2 = ops.attention(q.view(1, nh * d), kc, vc, torch.zeros(1, dtype=torch.int32, device="cuda"), pos,
                           table[None].contiguous(), nh, nkv, d, 1 / math.sqrt(d), window=T - far)
    torch.testing.assert_close(out_w2.view(nh, d)[2], v[far, 0], atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DT)
def test_rope_kv_store(ops, dtype):
    n, nh, nkv, d, ps, pages, theta = 11, 6, 2, 48, 8, 10, 5e4
    qkv = rnd(n, (nh + 2 * nkv) * d, dtype=dtype)
    q, k, v = qkv[:, :nh * d], qkv[:, nh * d:(nh + nkv) * d], qkv[:, (nh + nkv) * d:]
    pos = torch.arange(100, 100 + n, dtype=torch.int32, device="cuda")
    slots = torch.randperm(pages * ps)[:n].to(torch.int32).cuda()
    kc = torch.zeros(pages, nkv, ps, d, dtype=dtype, device="cuda")
    vc = torch.zeros(pages, nkv, d, ps, dtype=dtype, device="cuda")
    q_ref = torch_rope(q.float().reshape(n, nh, d), pos, theta)
    k_ref = torch_rope(k.float().reshape(n, nkv, d), pos, theta)
    v_ref = v.clone().reshape(n, nkv, d)
    ops.rope_kv_store(q, k, v, ops.rope_table(pos, ops.rope_inv_freq(d, theta, "cuda")), slots, kc, vc, nh, nkv, d)
    torch.testing.assert_close(q.float().reshape(n, nh, d), q_ref, **tol(dtype, 5e-4, 2e-2))
    for t in range(n):
        p, o = int(slots[t]) // ps, int(slots[t]) % ps
        torch.testing.assert_close(kc[p, :, o].float(), k_ref[t], **tol(dtype, 5e-4, 2e-2))
        assert torch.equal(vc[p, :, :, o], v_ref[t])
    # untouched slots stay zero
    assert int((kc != 0).any(-1).any(1).sum()) == n


@pytest.mark.parametrize("nh,nkv,d,rot,ps", [(12, 2, 128, 128, 16), (6, 2, 48, 32, 8), (3, 1, 64, 0, 32), (5, 5, 80, 80, 8)])
@pytest.mark.parametrize("layout", ["runs", "shifted", "scattered"])
def test_rope_kv_store_many_tokens(ops, nh, nkv, d, rot, ps, layout):
    """From 1,024 tokens on bfloat16 takes the kernel that moves 16-byte pieces: against the kernel for few
    tokens, eight tokens at a time (the same arithmetic; a product may be fused differently, hence one
    rounding step), with slots in runs from multiples of eight (a value run is one store), runs that start
    elsewhere, slots scattered, a tail of fewer than eight tokens, and slots out of range that are skipped."""
    dtype = torch.bfloat16
    n, pages, theta = 1051, 160, 5e4
    qkv = rnd(n, (nh + 2 * nkv) * d + 8, dtype=dtype)[:, 8:]             # rows that do not start the buffer
    q, k, v = qkv[:, :nh * d], qkv[:, nh * d:(nh + nkv) * d], qkv[:, (nh + nkv) * d:]
    pos = torch.arange(1000, 1000 + n, dtype=torch.int32, device="cuda")
    if layout == "scattered":
        slots = torch.randperm(pages * ps)[:n].to(torch.int32)
    else:
        slots = torch.arange(n, dtype=torch.int32) + (0 if layout == "runs" else 3)
    slots[17] = -1
    slots = slots.cuda()
    table = ops.rope_table(pos, ops.rope_inv_freq(rot, theta, "cuda")) if rot else None      # the step's (cos, sin)

    def run(step):
        qq = qkv.clone()
        kc = torch.full((pages, nkv, ps, d), 3.0, dtype=dtype, device="cuda")
        vc = torch.full((pages, nkv, d, ps), 3.0, dtype=dtype, device="cuda")
        for a in range(0, n, step):
            b = min(n, a + step)
            ops.rope_kv_store(qq[a:b, :nh * d], qq[a:b, nh * d:(nh + nkv) * d], qq[a:b, (nh + nkv) * d:],
                              table[a:b] if rot else None, slots[a:b], kc, vc, nh, nkv, d)
        return qq[:, :nh * d], kc, vc

    q1, kc1, vc1 = run(n)       # one call: the kernel for many tokens
    q2, kc2, vc2 = run(8)       # eight tokens a call: the kernel for few
    torch.testing.assert_close(q1.float(), q2.float(), atol=0.0, rtol=8e-3)
    torch.testing.assert_close(kc1.float(), kc2.float(), atol=0.0, rtol=8e-3)
    assert torch.equal(vc1, vc2)
    assert int((vc1 != 3.0).any(1).any(1).sum()) == n - 1      # every token's slot but the one out of range
    # queries only
    q3 = qkv.clone()
    ops.rope_kv_store(q3[:, :nh * d], None, None, table, None, None, None, nh, nkv, d)
    assert torch.equal(q3[:, :nh * d], q1) and torch.equal(q3[:, nh * d:], qkv[:, nh * d:])


@pytest.mark.parametrize("xdt,wdt,odt", [(torch.float32,) * 3, (torch.bfloat16,) * 3,
                                          (torch.bfloat16, torch.float32, torch.bfloat16),
                                          (torch.bfloat16, torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 100, 64), (5, 1000, 96), (70, 130, 176), (128, 1536, 8960), (3, 151, 33),
                                   (8, 2048, 1536), (1, 1536, 8960), (64, 1000, 176), (17, 17920, 1536), (33, 77, 40)])
def test_linear(ops, xdt, wdt, odt, M, N, K):
    x, w, b = rnd(M, K, dtype=xdt, seed=1), rnd(N, K, dtype=wdt, scale=0.05, seed=2), rnd(N, dtype=wdt, seed=3)
    ref = torch.nn.functional.linear(x.double(), w.double(), b.double()).float()
    out = ops.linear(x, w, b, out_dtype=odt)
    assert out.dtype == odt
    t = tol(odt, 5e-5, 2e-2)
    torch.testing.assert_close(out.float(), ref, **t)
    out_nb = ops.linear(x, w, out_dtype=odt)
    torch.testing.assert_close(out_nb.float(), torch.nn.functional.linear(x.double(), w.double()).float(), **t)
    # into a column slice of a wider buffer
    wide = torch.zeros(M, N + 8, dtype=odt, device="cuda")
    ops.linear(x, w, b, out=wide[:, 4:N + 4])
    torch.testing.assert_close(wide[:, 4:N + 4].float(), ref, **t)
    assert float(wide[:, :4].abs().max()) == 0 and float(wide[:, N + 4:].abs().max()) == 0


@pytest.mark.parametrize("M,N,K", [(65, 136, 72), (200, 2048, 1536), (130, 1536, 8960), (1000, 152, 264)])
def test_linear_by_the_library(ops, M, N, K):
    """The many-rows products that go to the library (straight with and without bias, into rows of a wider
    buffer, with float32 results, transposed) against a float64 product; then with an algorithm chosen by
    timing, and with one fixed by its number."""
    x, w, b = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, scale=0.05, seed=2), \
        rnd(N, dtype=torch.bfloat16, seed=3)
    ref = torch.nn.functional.linear(x.double(), w.double()).float()
    ref_b = ref + b.float()
    calls = []
    real = ops._lib.call
    ops._lib.call = lambda name, *a: (calls.append(name), real(name, *a))[1]
    try:
        t = dict(atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(ops.linear(x, w, b).float(), ref_b, **t)
        torch.testing.assert_close(ops.linear(x, w).float(), ref, **t)
        torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32), ref, atol=1e-3, rtol=1e-3)
        wide = torch.zeros(M, N + 16, dtype=torch.bfloat16, device="cuda")
        ops.linear(x, w, b, out=wide[:, 8:N + 8])
        torch.testing.assert_close(wide[:, 8:N + 8].float(), ref_b, **t)
        assert float(wide[:, :8].abs().max()) == 0 and float(wide[:, N + 8:].abs().max()) == 0
        xw = torch.zeros(M, K + 8, dtype=torch.bfloat16, device="cuda")
        xw[:, :K] = x
        torch.testing.assert_close(ops.linear(xw[:, :K], w, b).float(), ref_b, **t)
        torch.testing.assert_close(ops.linear_transposed(x, w).float(), ref.t(), **t)
        assert calls == ["zi_gemm_lt"] * 6, calls
        # a shape that has been served keeps its algorithm (the library's first proposal); one that has not is timed
        assert ops.linear_tune(x, w, bias=b, candidates=8, rounds=2)[0] == 0
        x2 = rnd(M + 8, K, dtype=torch.bfloat16, seed=5)
        ref2 = torch.nn.functional.linear(x2.double(), w.double()).float()
        for kwargs in (dict(bias=b), dict(transposed=True), dict(out_dtype=torch.float32)):
            chosen, proposed, us = ops.linear_tune(x2, w, candidates=8, rounds=2, **kwargs)
            assert 0 <= chosen < proposed and us > 0
            assert ops.linear_tune(x2, w, candidates=8, rounds=2, **kwargs)[0] == chosen       # a shape is timed once
        torch.testing.assert_close(ops.linear(x2, w, b).float(), ref2 + b.float(), **t)
        torch.testing.assert_close(ops.linear_transposed(x2, w).float(), ref2.t(), **t)
        torch.testing.assert_close(ops.linear(x2, w, out_dtype=torch.float32), ref2, atol=1e-3, rtol=1e-3)
        before = ops.linear(x, w, b)
        ops.linear_choose(x, w, 0, bias=b)
        assert torch.equal(ops.linear(x, w, b), before)
        with pytest.raises(ops.KernelLibraryError, match="proposal"):
            ops.linear_choose(x, w, 10 ** 6, bias=b)
    finally:
        ops._lib.call = real
    assert ops.linear_tune(x[:8], w) is None and ops.linear_tune(x.float(), w.float()) is None


def test_linear_skinny_row_does_not_depend_on_batch(ops):
    """The decode-time product cuts k by the weight's shape alone: a row's result is bit-identical
    whether 1, 8 or 64 rows ride along."""
    x, w = rnd(64, 1536, dtype=torch.bfloat16, seed=1), rnd(2048, 1536, dtype=torch.bfloat16, scale=0.05, seed=2)
    # up to 16 rows run on one kernel, 17 to 64 on another: within each a row does not depend on the others
    full = ops.linear(x, w, out_dtype=torch.float32)
    for m in (17, 40):
        assert torch.equal(full[:m], ops.linear(x[:m].contiguous(), w, out_dtype=torch.float32))
    few = ops.linear(x[:16].contiguous(), w, out_dtype=torch.float32)
    for m in (1, 8):
        assert torch.equal(few[:m], ops.linear(x[:m].contiguous(), w, out_dtype=torch.float32))
    torch.testing.assert_close(few, full[:16], atol=1e-3, rtol=1e-3)
    assert torch.equal(ops.linear(x[:16].contiguous(), w)[:3], ops.linear(x[:3].contiguous(), w))
    assert torch.equal(ops.linear(x, w)[:20], ops.linear(x[:20].contiguous(), w))
    assert torch.equal(ops.linear(x[:3].contiguous(), w), few[:3].to(torch.bfloat16))
    x2, w2 = rnd(64, 8960, dtype=torch.bfloat16, seed=3), rnd(1536, 8960, dtype=torch.bfloat16, scale=0.02, seed=4)
    assert torch.equal(ops.linear(x2[:16].contiguous(), w2, out_dtype=torch.float32)[5:6],
                       ops.linear(x2[5:6].contiguous(), w2, out_dtype=torch.float32))


@pytest.mark.parametrize("N,K", [(1536, 22400), (3584, 18944), (5120, 27648), (1000, 33560), (1192, 28200)])
def test_linear_sums_of_129_to_256_rows(ops, N, K):
    """The product for many rows (32 weight rows a wavefront): partial sums of 129 .. 256 rows against a float32
    product, at the down projections' widths of the larger sizes and at two widths that are multiples of nothing
    much; a row's sums do not depend on how many rows ride along (the cut of k is the weight's alone)."""
    w = rnd(N, K, dtype=torch.bfloat16, scale=0.02, seed=2)
    x = rnd(256, K, dtype=torch.bfloat16, seed=1)
    ref = x.float() @ w.float().t()
    scale = float(ref.abs().max())
    full = None
    for M in (129, 200, 256):
        xm = x[:M].contiguous()
        assert ops.linear_sums_supported(xm, w)
        S = ops.linear_splits(M, N, K)
        assert 1 <= S <= 16 and S == ops.linear_splits(256, N, K)
        sums = ops.linear_sums(xm, w)
        assert tuple(sums.shape) == (S, M, N)
        assert float((sums.sum(0) - ref[:M]).abs().max()) <= 2e-5 * scale
        if M == 256:
            full = sums
    for M in (129, 200):
        assert torch.equal(ops.linear_sums(x[:M].contiguous(), w), full[:, :M])
    # square and small weights stay with the library's product beyond 128 rows
    assert not ops.linear_sums_supported(x[:200, :1536].contiguous(), rnd(1536, 1536, dtype=torch.bfloat16))
    assert ops.linear_sums_supported(x[:128, :1536].contiguous(), rnd(1536, 1536, dtype=torch.bfloat16))


@pytest.mark.parametrize("M", [65, 96, 128, 129, 200, 256])
@pytest.mark.parametrize("I,K", [(8960, 1536), (1000, 200), (18944, 3584)])
def test_linear_swiglu_of_65_to_256_rows(ops, M, I, K, monkeypatch):
    """The same kernel with the SwiGLU epilogue (gate and up rows interleaved in blocks of 8), which the engine
    does not take beyond 64 rows (the library's product and the activation's own launch are faster there): here
    with the limit lifted, against float32."""
    from zedinfer_amd.ops import functional
    from zedinfer_amd.parts.feed_forward import GATE_UP_BLOCK, interleave_rows
    monkeypatch.setattr(functional, "SWIGLU_MAX_ROWS", 256)
    monkeypatch.setattr(functional, "SUMS_MAX_ROWS", 256)
    gate, up = rnd(I, K, dtype=torch.bfloat16, scale=0.05, seed=3), rnd(I, K, dtype=torch.bfloat16, scale=0.05, seed=4)
    x = rnd(M, K, dtype=torch.bfloat16, seed=5)
    w = interleave_rows(gate, up, GATE_UP_BLOCK)
    assert ops.linear_swiglu_supported(x, w)
    g, u = x.float() @ gate.float().t(), x.float() @ up.float().t()
    want = u * (g / (1 + torch.exp(-g)))
    got = ops.linear_swiglu(x, w)
    assert tuple(got.shape) == (M, I)
    assert float((got.float() - want).abs().max()) <= 1e-2 * float(want.abs().max())
    # rows do not depend on each other (from 65 rows on it is this kernel, whose sums run over k in one order)
    if M - 3 > 64:
        assert torch.equal(ops.linear_swiglu(x[:M - 3].contiguous(), w), got[:M - 3])


def test_linear_f32_row_does_not_depend_on_batch(ops):
    """The float32 product sums over k in one fixed order: a row's result is bit-identical whatever M is."""
    x, w = rnd(70, 176, seed=1), rnd(130, 176, seed=2)
    full = ops.linear(x, w)
    one = ops.linear(x[17:18].contiguous(), w)
    assert torch.equal(full[17], one[0])


@pytest.mark.parametrize("dtype", DT)
def test_argmax(ops, dtype):
    x = rnd(5, 1000, dtype=dtype)
    idx, val = ops.argmax(x, return_values=True)
    assert torch.equal(idx.long(), torch.argmax(x.float(), -1))
    torch.testing.assert_close(val, x.float().max(-1).values)
    # ties: the lowest index wins (reference: tests/sampler/test_sampler.cpp:85-122)
    t = torch.zeros(2, 151936, dtype=dtype, device="cuda")
    t[0, 70000] = 3.0
    t[0, 1234] = 3.0
    t[1, -1] = 1.0
    assert ops.argmax(t).tolist() == [1234, 151935]
    assert ops.argmax(torch.zeros(1, 77, device="cuda")).tolist() == [0]
    # long rows are cut over several workgroups; rows may be slices of a wider matrix
    big = rnd(7, 50001, dtype=dtype)[:, 3:40004]
    idx, val = ops.argmax(big, return_values=True)
    assert torch.equal(idx.long(), torch.argmax(big.float(), -1))
    torch.testing.assert_close(val, big.float().max(-1).values)
    z = torch.zeros(3, 20000, dtype=dtype, device="cuda")
    z[1, 8192] = z[1, 19999] = 2.0
    assert ops.argmax(z).tolist() == [0, 8192, 0]


@pytest.mark.parametrize("nh,nkv,d,ps,T,window", [
    (12, 2, 128, 16, 2100, 0), (12, 2, 128, 16, 70, 0), (28, 4, 128, 16, 5000, 0), (3, 1, 64, 8, 200, 0),
    (8, 1, 64, 16, 300, 37), (5, 5, 80, 32, 150, 0), (4, 2, 128, 8, 260, 100), (14, 2, 128, 16, 9, 0),
    (12, 1, 48, 8, 700, 0), (4, 2, 16, 16, 1000, 300), (32, 2, 112, 64, 530, 0), (12, 2, 128, 16, 17000, 0),
    (12, 2, 128, 64, 600, 0), (6, 2, 64, 128, 900, 250), (40, 8, 128, 32, 1300, 0)])      # pages whose value rows are longer than half a line
def test_attention_decode(ops, nh, nkv, d, ps, T, window):
    """The split-keys kernel against the same float32 reference, with a listed subset of the tokens."""
    dtype = torch.bfloat16
    assert ops.attention_decode_supported(dtype, nh, nkv, d, ps)
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1), rnd(T, nkv, d, dtype=dtype, seed=2)
    pages = (T + ps - 1) // ps + 3
    kc, vc, table = make_paged(k, v, ps, pages)
    pos_list = sorted(p for p in {T - 1, T - 2, 0, 1, 7, 8, 63, 64, 65, 127, 128, 255, 256, 257, 511, 512, 16383, 16384, T // 2, T // 3} if p < T)
    pos = torch.tensor(pos_list, dtype=torch.int32, device="cuda")
    n = pos.numel()
    q = rnd(n, nh, d, dtype=dtype, seed=3)
    seq = torch.zeros(n, dtype=torch.int32, device="cuda")
    bt = table[None].contiguous()
    scale = 1 / math.sqrt(d)
    ref = ref_attention(q.float(), k.float(), v.float(), pos.long(), scale, window)
    out = ops.attention_decode(q.view(n, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, T, window)
    torch.testing.assert_close(out.view(n, nh, d).float(), ref, atol=2e-2, rtol=2e-2)
    # a listed subset leaves the other rows alone
    idx = torch.tensor([n - 1, 0, 3], dtype=torch.int32, device="cuda")
    assert n > 4
    out2 = torch.full((n, nh * d), 7.0, dtype=dtype, device="cuda")
    ops.attention_decode(q.view(n, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, T, window, out=out2, tok_index=idx)
    sel = idx.long()
    assert torch.equal(out2[sel], out[sel])
    rest = torch.ones(n, dtype=torch.bool)
    rest[sel.cpu()] = False
    assert bool((out2[rest.cuda()] == 7.0).all())
    # against the plain kernel on the same inputs: both round the same float32 result
    plain_out = ops.attention(q.view(n, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, window)
    torch.testing.assert_close(out.float(), plain_out.float(), atol=1e-2, rtol=1e-2)


def fused_decode_case(ops, nh, nkv, d, ps, lens, S, bias_dtype, rot):
    """Sequences of the given lengths in a shuffled paged cache whose last position (the new token's)
    and unused slots hold NaN, and the partial sums of the new tokens' projections."""
    dtype = torch.bfloat16
    B, width, theta = len(lens), (nh + 2 * nkv) * d, 1e4
    assert ops.attention_decode_fused_supported(dtype, nh, nkv, d, ps, rot, S, width, B)
    pages_per = [(L + ps - 1) // ps for L in lens]
    total_pages = sum(pages_per) + 2
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(total_pages, generator=g).tolist()
    kc = torch.full((total_pages, nkv, ps, d), float("nan"), dtype=dtype, device="cuda")
    vc = torch.full((total_pages, nkv, d, ps), float("nan"), dtype=dtype, device="cuda")
    bt = torch.full((B, max(pages_per)), -1, dtype=torch.int32)
    slots = torch.empty(B, dtype=torch.int32)
    for b, L in enumerate(lens):
        mine = [perm.pop() for _ in range(pages_per[b])]
        bt[b, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        k, v = rnd(L - 1, nkv, d, dtype=dtype, seed=10 + b), rnd(L - 1, nkv, d, dtype=dtype, seed=20 + b)
        for t in range(L - 1):       # the last position is the new token's: its slot stays NaN
            kc[mine[t // ps], :, t % ps] = k[t]
            vc[mine[t // ps], :, :, t % ps] = v[t]
        slots[b] = mine[(L - 1) // ps] * ps + (L - 1) % ps
    bt, slots = bt.cuda(), slots.cuda()
    pos = torch.tensor([L - 1 for L in lens], dtype=torch.int32, device="cuda")
    seq = torch.arange(B, dtype=torch.int32, device="cuda")
    sums = rnd(S, B, width, seed=1)
    bias = rnd(width, seed=2).to(bias_dtype) if bias_dtype is not None else None
    inv_freq = ops.rope_inv_freq(rot, theta, "cuda") if rot else None
    return kc, vc, bt, slots, pos, seq, sums, bias, inv_freq


FUSED_DECODE_CASES = [
    (12, 2, 128, 16, [2100, 1, 64, 65, 257, 300, 1024, 17], 0, 2, torch.bfloat16, 128),
    (3, 1, 64, 8, [200, 5, 9], 0, 1, None, 64),
    (8, 2, 48, 8, [33, 700, 256], 0, 3, torch.float32, 32),
    (4, 2, 128, 16, [500, 120, 99], 100, 5, torch.bfloat16, 128),
    (6, 3, 80, 32, [150, 64], 0, 2, torch.bfloat16, 0),
    (12, 2, 128, 16, [17000, 300], 0, 2, torch.bfloat16, 128),
    (12, 2, 128, 64, [700, 64, 65, 129], 0, 2, torch.bfloat16, 128)]


@pytest.mark.parametrize("nh,nkv,d,ps,lens,window,S,bias_dtype,rot", FUSED_DECODE_CASES)
def test_attention_decode_fused(ops, nh, nkv, d, ps, lens, window, S, bias_dtype, rot):
    """One kernel for rotation, cache store and attention of decoded tokens gives what the rotary kernel
    followed by the decode kernel gives: same output, same new keys and values in the cache.  The slot
    of the new token holds NaN before, and the sequences differ in length (the new key sits in every
    place of a block)."""
    B = len(lens)
    kc, vc, bt, slots, pos, seq, sums, bias, inv_freq = fused_decode_case(ops, nh, nkv, d, ps, lens, S, bias_dtype, rot)
    dtype = torch.bfloat16
    scale, T = 1 / math.sqrt(d), max(lens)
    # the two kernels
    kc1, vc1 = kc.clone(), vc.clone()
    q = torch.empty(B, nh * d, dtype=dtype, device="cuda")
    ops.rope_kv_store_sums(sums, bias, q, ops.rope_table(pos, inv_freq) if inv_freq is not None else None, slots, kc1,
                           vc1, nh, nkv, d)
    ref = ops.attention_decode(q, kc1, vc1, seq, pos, bt, nh, nkv, d, scale, T, window)
    # the one kernel
    kc2, vc2 = kc.clone(), vc.clone()
    table = ops.rope_table(pos, inv_freq) if rot else None
    out = ops.attention_decode_fused(sums, bias, table, slots, kc2, vc2, seq, pos, bt, nh, nkv, d, scale, T, window)
    assert not torch.isnan(out).any()
    torch.testing.assert_close(out.float(), ref.float(), atol=4e-3, rtol=1e-2)
    # token t is of sequence t: the same without the list of sequences
    kc4, vc4 = kc.clone(), vc.clone()
    out4 = ops.attention_decode_fused(sums, bias, table, slots, kc4, vc4, None, pos, bt, nh, nkv, d, scale, T, window)
    assert torch.equal(out4, out)
    assert bool(((kc4 == kc2) | (torch.isnan(kc4) & torch.isnan(kc2))).all())
    assert bool(((vc4 == vc2) | (torch.isnan(vc4) & torch.isnan(vc2))).all())
    for b in range(B):
        pg, o = int(slots[b]) // ps, int(slots[b]) % ps
        torch.testing.assert_close(kc2[pg, :, o].float(), kc1[pg, :, o].float(), atol=1e-3, rtol=8e-3)
        assert torch.equal(vc2[pg, :, :, o], vc1[pg, :, :, o])
    # nothing else in the cache was touched
    same_k = (kc2 == kc1) | (torch.isnan(kc2) & torch.isnan(kc1))
    same_v = (vc2 == vc1) | (torch.isnan(vc2) & torch.isnan(vc1))
    for b in range(B):
        pg, o = int(slots[b]) // ps, int(slots[b]) % ps
        same_k[pg, :, o] = True
    assert bool(same_k.all()) and bool(same_v.all())
    # a layer that reads another layer's cache: queries only, the cache is left alone
    kc3, vc3 = kc1.clone(), vc1.clone()
    out3 = ops.attention_decode_fused(sums, bias, table, None, kc3, vc3, seq, pos, bt, nh, nkv, d, scale, T, window,
                                      write_kv=False)
    torch.testing.assert_close(out3.float(), ref.float(), atol=4e-3, rtol=1e-2)
    assert bool(((kc3 == kc1) | (torch.isnan(kc3) & torch.isnan(kc1))).all())
    assert bool(((vc3 == vc1) | (torch.isnan(vc3) & torch.isnan(vc1))).all())


@pytest.mark.parametrize("nh,nkv,d,ps,lens,window,S,bias_dtype,rot", FUSED_DECODE_CASES + [
    (40, 8, 128, 16, [300, 70, 1], 0, 2, torch.bfloat16, 128),            # groups of three heads a partial sum
    (2, 1, 16, 8, [9, 300, 40, 41, 42, 43, 44, 45, 46, 47, 48, 49, 50, 51, 52, 53], 0, 1, None, 16)])  # 16 tokens
def test_attention_decode_project(ops, nh, nkv, d, ps, lens, window, S, bias_dtype, rot):
    """The output projection read straight from the unmerged chunks against the merged attention times
    the weight: the merge is the merge kernel's (its bfloat16 result is the operand), so only the order
    of the float32 sums differs.  Widths that are no multiple of 64 or of 4."""
    B = len(lens)
    kc, vc, bt, slots, pos, seq, sums, bias, inv_freq = fused_decode_case(ops, nh, nkv, d, ps, lens, S, bias_dtype, rot)
    scale, T = 1 / math.sqrt(d), max(lens)
    table = ops.rope_table(pos, inv_freq) if rot else None
    kc1, vc1 = kc.clone(), vc.clone()
    att = ops.attention_decode_fused(sums, bias, table, slots, kc1, vc1, seq, pos, bt, nh, nkv, d, scale, T, window)
    kc2, vc2 = kc.clone(), vc.clone()
    ws = torch.full((ops.attention_decode_workspace(B, nh, d),), float("nan"), device="cuda")
    got_ws = ops.attention_decode_fused(sums, bias, table, slots, kc2, vc2, seq, pos, bt, nh, nkv, d, scale, T, window,
                                        workspace=ws, leave_chunks=True)
    assert got_ws is ws
    assert bool(((kc2 == kc1) | (torch.isnan(kc2) & torch.isnan(kc1))).all())
    for N in (1536, 200, 70):
        w = (rnd(N, nh * d, seed=7) / math.sqrt(nh * d)).to(torch.bfloat16)
        assert ops.attention_decode_project_supported(w, B, nh, d)
        want = att.float() @ w.float().T
        parts = torch.full((ops.attention_decode_project_splits(nh), B, N), float("nan"), device="cuda")
        out = ops.attention_decode_project(ws, w, pos, nh, d, T, window, out=parts)
        assert out is parts and not torch.isnan(parts).any()
        torch.testing.assert_close(parts.sum(0), want, atol=2e-4 * max(1.0, float(want.abs().max())), rtol=1e-4)
        # a partial sum is the product over its heads alone
        hg = -(-nh // parts.shape[0])
        first = att.float()[:, :hg * d] @ w.float()[:, :hg * d].T
        torch.testing.assert_close(parts[0], first, atol=2e-4 * max(1.0, float(first.abs().max())), rtol=1e-4)


def test_attention_decode_project_shows_a_bound_too_low(ops):
    """Chunks the launch did not cover: the token's whole row is NaN, the other tokens' rows are right."""
    nh, nkv, d, ps, lens = 4, 2, 64, 16, [700, 100]
    kc, vc, bt, slots, pos, seq, sums, bias, inv_freq = fused_decode_case(ops, nh, nkv, d, ps, lens, 2, None, 64)
    scale = 1 / math.sqrt(d)
    table = ops.rope_table(pos, inv_freq)
    w = (rnd(96, nh * d, seed=7) / 16).to(torch.bfloat16)
    att = ops.attention_decode_fused(sums, bias, table, slots, kc.clone(), vc.clone(), seq, pos, bt, nh, nkv, d, scale, 700)
    ws = ops.attention_decode_fused(sums, bias, table, slots, kc.clone(), vc.clone(), seq, pos, bt, nh, nkv, d, scale, 200,
                                    leave_chunks=True)
    parts = ops.attention_decode_project(ws, w, pos, nh, d, 200)
    assert bool(torch.isnan(parts[:, 0]).all())
    torch.testing.assert_close(parts.sum(0)[1], att.float()[1] @ w.float().T, atol=2e-4, rtol=1e-4)


def test_attention_decode_project_refuses_other_shapes(ops):
    w = torch.zeros(64, 12 * 128, dtype=torch.bfloat16, device="cuda")
    assert ops.attention_decode_project_supported(w, 16, 12, 128)
    assert not ops.attention_decode_project_supported(w, 17, 12, 128)            # more tokens than a tile's columns
    assert not ops.attention_decode_project_supported(w.float(), 8, 12, 128)
    assert not ops.attention_decode_project_supported(w, 8, 6, 128)              # not this weight's columns
    assert not ops.attention_decode_project_supported(w[:, :1532], 8, 12, 128)


def test_attention_decode_fused_refuses_other_layouts(ops):
    assert not ops.attention_decode_fused_supported(torch.bfloat16, 12, 2, 128, 16, 24, 2, 2048, 8)    # rot % 16
    assert not ops.attention_decode_fused_supported(torch.bfloat16, 12, 2, 128, 16, 128, 2, 2050, 8)   # stride % 4
    assert not ops.attention_decode_fused_supported(torch.float32, 12, 2, 128, 16, 128, 2, 2048, 8)


@pytest.mark.parametrize("far", [37, 255, 256, 511, 690])
def test_attention_decode_far_key_stands_out(ops, far):
    """One key among hundreds is made to dominate one head (at a chunk's edges too): its value must come
    through the split-keys kernel and the merge of its chunks; a window that ends just after it hides
    it, one key wider shows it again."""
    nh, nkv, d, ps, T = 8, 2, 64, 16, 700
    dtype = torch.bfloat16
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1) * 0.1, rnd(T, nkv, d, dtype=dtype, seed=2)
    q = rnd(1, nh, d, dtype=dtype, seed=3)
    head, g = 5, 5 // (nh // nkv)
    k[far, g] = (q[0, head].float() * 60.0 / q[0, head].float().norm() ** 2 * math.sqrt(d)).to(dtype)
    kc, vc, table = make_paged(k, v, ps, 64)
    pos = torch.tensor([T - 1], dtype=torch.int32, device="cuda")
    seq = torch.zeros(1, dtype=torch.int32, device="cuda")
    bt = table[None].contiguous()
    scale = 1 / math.sqrt(d)
    out = ops.attention_decode(q.view(1, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, T)
    torch.testing.assert_close(out.view(nh, d)[head].float(), v[far, g].float(), atol=2e-2, rtol=2e-2)
    hidden = ops.attention_decode(q.view(1, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, T, T - 1 - far)
    assert float((hidden.view(nh, d)[head].float() - v[far, g].float()).abs().max()) > 0.1
    shown = ops.attention_decode(q.view(1, nh * d), kc, vc, seq, pos, bt, nh, nkv, d, scale, T, T - far)
    torch.testing.assert_close(shown.view(nh, d)[head].float(), v[far, g].float(), atol=2e-2, rtol=2e-2)


def test_attention_decode_ignores_stale_slots(ops):
    """Slots of a page beyond the token's position may hold anything, NaN included."""
    nh, nkv, d, ps, T = 4, 2, 128, 16, 37
    k, v = rnd(T, nkv, d, dtype=torch.bfloat16, seed=1), rnd(T, nkv, d, dtype=torch.bfloat16, seed=2)
    kc, vc, table = make_paged(k, v, ps, 8)        # unused slots are NaN
    pos = torch.tensor([T - 1, 20], dtype=torch.int32, device="cuda")
    q = rnd(2, nh, d, dtype=torch.bfloat16, seed=3)
    out = ops.attention_decode(q.view(2, nh * d), kc, vc, torch.zeros(2, dtype=torch.int32, device="cuda"), pos,
                               table[None].contiguous(), nh, nkv, d, 0.1, T)
    assert not torch.isnan(out).any()
    ref = ref_attention(q.float(), k.float(), v.float(), pos.long(), 0.1, 0)
    torch.testing.assert_close(out.view(2, nh, d).float(), ref, atol=2e-2, rtol=2e-2)


def test_unsupported_shapes_are_refused(ops):
    assert not ops.attention_decode_supported(torch.float32, 12, 2, 128, 16)
    assert not ops.attention_decode_supported(torch.bfloat16, 12, 2, 40, 16)
    assert not ops.attention_decode_supported(torch.bfloat16, 12, 2, 256, 16)
    assert not ops.attention_decode_supported(torch.bfloat16, 34, 2, 128, 16)       # group of 17
    assert not ops.attention_decode_supported(torch.bfloat16, 12, 2, 128, 4)
    q = rnd(1, 12 * 48, dtype=torch.bfloat16)
    kc = torch.zeros(4, 2, 16, 48, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros(4, 2, 48, 16, dtype=torch.bfloat16, device="cuda")
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(ops.KernelLibraryError, match="unsupported shape"):
        ops.attention_decode(rnd(1, 2 * 256, dtype=torch.bfloat16),
                             torch.zeros(4, 2, 16, 256, dtype=torch.bfloat16, device="cuda"),
                             torch.zeros(4, 2, 256, 16, dtype=torch.bfloat16, device="cuda"), z, z,
                             torch.zeros(1, 4, dtype=torch.int32, device="cuda"), 2, 2, 256, 0.1, 1)
    with pytest.raises(ValueError, match="multiple"):
        ops.attention(q, kc, vc, z, z, torch.zeros(1, 4, dtype=torch.int32, device="cuda"), 12, 5, 48, 0.1)
    with pytest.raises(ops.KernelLibraryError, match="larger than"):
        big = torch.zeros(1, 1024, dtype=torch.bfloat16, device="cuda")
        ops.attention(big, torch.zeros(1, 1, 16, 1024, dtype=torch.bfloat16, device="cuda"),
                      torch.zeros(1, 1, 1024, 16, dtype=torch.bfloat16, device="cuda"), z, z,
                      torch.zeros(1, 1, dtype=torch.int32, device="cuda"), 1, 1, 1024, 0.1)


def prefill_tiles(entries, tile=64):
    """entries: [(start, len, past)] -> (tile_entry, tile_off) with the heaviest tile first."""
    tiles = [(past + off + min(tile, n - off), e, off) for e, (s, n, past) in enumerate(entries)
             for off in range(0, n, tile)]
    tiles.sort(key=lambda t: -t[0])
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    return dev([t[1] for t in tiles]), dev([t[2] for t in tiles])


@pytest.mark.parametrize("nh,nkv,d,ps,window,portions", [
    (12, 2, 128, 16, 0, [(0, 300), (300, 77)]),          # a prompt from the start, then a portion on top of it
    (4, 2, 16, 16, 0, [(0, 49), (49, 5), (54, 130)]),
    (3, 1, 32, 8, 0, [(0, 100), (100, 64), (164, 65)]),
    (6, 2, 48, 8, 20, [(0, 90), (90, 40)]),              # head_dim that is no multiple of 32, window
    (5, 5, 80, 32, 0, [(3, 70)]),
    (28, 4, 128, 64, 64, [(0, 130), (130, 200)]),
    (2, 1, 112, 128, 0, [(17, 129)]),
    (14, 2, 64, 16, 150, [(0, 1000)]),
    (4, 2, 128, 16, 0, [(0, 2100), (2100, 130)]),        # tiles that see more than 2,048 keys are cut and merged
    (2, 1, 64, 16, 0, [(4000, 200), (2047, 3), (2040, 70)]),   # cuts at absolute multiples of 2,048, inside a tile too
    (3, 1, 32, 8, 300, [(1900, 400)]),                   # a window across a cut
    (2, 2, 128, 32, 2500, [(3000, 1500)]),               # a window wider than a cut
])
def test_attention_prefill(ops, nh, nkv, d, ps, window, portions):
    """The matrix-core prompt kernel against the float32 reference: portions at several pasts, two
    sequences in one launch that share pages through identical table rows."""
    dtype = torch.bfloat16
    assert ops.attention_prefill_supported(dtype, nh, nkv, d, ps)
    T = max(p + n for p, n in portions)
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1), rnd(T, nkv, d, dtype=dtype, seed=2)
    kc, vc, table = make_paged(k, v, ps, (T + ps - 1) // ps + 3)      # unused slots are NaN
    entries, pos = [], []
    for past, n in portions:
        entries.append((len(pos), n, past))
        pos += list(range(past, past + n))
    n_tok = len(pos)
    pos_t = torch.tensor(pos, dtype=torch.int32, device="cuda")
    q = rnd(n_tok, nh, d, dtype=dtype, seed=3)
    bt = torch.stack([table] * len(entries)).contiguous()
    te, to = prefill_tiles(entries)
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    scale = 1 / math.sqrt(d)
    out = torch.full((n_tok, nh * d), 7.0, dtype=dtype, device="cuda")
    ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te, to, dev([e[0] for e in entries]),
                          dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale, window,
                          out=out)
    assert not torch.isnan(out).any()
    ref = ref_attention(q.float(), k.float(), v.float(), pos_t.long(), scale, window)
    torch.testing.assert_close(out.view(n_tok, nh, d).float(), ref, atol=2e-2, rtol=2e-2)
    # against the plain kernel on the same inputs
    seq = torch.tensor([e for e, (s, n, p) in enumerate(entries) for _ in range(n)], dtype=torch.int32, device="cuda")
    plain_out = ops.attention(q.view(n_tok, nh * d), kc, vc, seq, pos_t, bt, nh, nkv, d, scale, window)
    torch.testing.assert_close(out.float(), plain_out.float(), atol=1.5e-2, rtol=1.5e-2)
    # a tile list that leaves an entry out leaves its rows alone
    if len(entries) > 1:
        out2 = torch.full((n_tok, nh * d), 7.0, dtype=dtype, device="cuda")
        keep = te != 0
        ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te[keep].contiguous(), to[keep].contiguous(),
                              dev([e[0] for e in entries]), dev([e[1] for e in entries]),
                              dev([e[2] for e in entries]), bt, nh, nkv, d, scale, window, out=out2)
        n0 = entries[0][1]
        assert bool((out2[:n0] == 7.0).all()) and torch.equal(out2[n0:], out[n0:])
    # head sizes 64 and 128 take tiles of 128 queries too (a staged block of keys serves twice the queries): the
    # same bits, a query's walk over its keys does not depend on the tile it rides in
    wide = ops.attention_prefill_tile(dtype, d)
    assert wide == (128 if d in (64, 128) else 64)
    if wide == 128:
        te2, to2 = prefill_tiles(entries, tile=128)
        out4 = torch.full((n_tok, nh * d), 7.0, dtype=dtype, device="cuda")
        ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te2, to2, dev([e[0] for e in entries]),
                              dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale,
                              window, out=out4, tile=128)
        assert torch.equal(out4, out)
        # workgroups of four wavefronts that walk blocks of 64 keys (for launches of many tiles): another order of
        # a query's keys, so another rounding, the same for both tile sizes
        alone = {}
        for tile, (ta, tb) in ((64, (te, to)), (128, (te2, to2))):
            alone[tile] = torch.full((n_tok, nh * d), 7.0, dtype=dtype, device="cuda")
            ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, ta, tb, dev([e[0] for e in entries]),
                                  dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale,
                                  window, out=alone[tile], tile=tile, alone=True)
            assert not torch.isnan(alone[tile]).any()
            torch.testing.assert_close(alone[tile].view(n_tok, nh, d).float(), ref, atol=2e-2, rtol=2e-2)
        assert torch.equal(alone[64], alone[128])
    else:
        with pytest.raises(ValueError, match="four wavefronts"):
            ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te, to, dev([e[0] for e in entries]),
                                  dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale,
                                  window, out=out, alone=True)
        with pytest.raises(ValueError, match="tiles of 128"):
            ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te, to, dev([e[0] for e in entries]),
                                  dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale,
                                  window, out=out, tile=128)
    # head sizes 64 and 128 have a second kernel (keys and values straight into LDS): the same bits
    if d in (64, 128):
        before = ops.attention_prefill_variant(0)
        try:
            out3 = torch.full((n_tok, nh * d), 7.0, dtype=dtype, device="cuda")
            ops.attention_prefill(q.view(n_tok, nh * d), kc, vc, te, to, dev([e[0] for e in entries]),
                                  dev([e[1] for e in entries]), dev([e[2] for e in entries]), bt, nh, nkv, d, scale,
                                  window, out=out3)
        finally:
            ops.attention_prefill_variant(before)
        assert before == 1 and torch.equal(out3, out)


def test_attention_prefill_bound_too_low_shows(ops):
    """The host sizes the launch from an upper bound of the keys a query sees; a bound that is too low
    must not write outside the workspace, and leaves NaN where it did not suffice."""
    nh, nkv, d, ps, T = 2, 1, 64, 16, 2300
    dtype = torch.bfloat16
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1), rnd(T, nkv, d, dtype=dtype, seed=2)
    kc, vc, table = make_paged(k, v, ps, T // ps + 2)
    q = rnd(T, nh, d, dtype=dtype, seed=3)
    te, to = prefill_tiles([(0, T, 0)])
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    args = (q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]), table[None].contiguous(), nh, nkv, d, 0.125)
    good = ops.attention_prefill(*args, max_keys=T)
    assert not torch.isnan(good).any()
    low = ops.attention_prefill(*args, max_keys=2048)
    assert not torch.isnan(low[:2048]).any() and torch.equal(low[:2048], good[:2048])
    assert bool(torch.isnan(low[2048:]).all())
    assert ops.attention_prefill_workspace(T, nh, d, 2048) == 0 and ops.attention_prefill_workspace(T, nh, d, 2049) > 0


@pytest.mark.parametrize("nh,nkv,d,T,tile,cuts,window", [(14, 2, 64, 7000, 128, 1, 0), (6, 1, 64, 16500, 128, 2, 0),
                                                         (12, 2, 128, 8200, 64, 1, 0), (6, 2, 64, 17000, 128, 2, 7000)])
def test_attention_prefill_with_the_cut_of_long_prompts(ops, nh, nkv, d, T, tile, cuts, window):
    """A launch of 768 tiles x heads or more whose queries see more than 6,144 keys cuts its tiles every 16,384 keys,
    not every 2,048: one workgroup walks up to 16,384 keys (its block table entries staged in turns), no workspace
    is needed up to there and two cuts are merged beyond.  Rows at the cuts' edges and elsewhere against a float32
    reference; a launch of fewer tiles over the same keys keeps the short cut."""
    dtype, ps = torch.bfloat16, 16
    k, v = rnd(T, nkv, d, dtype=dtype, seed=1), rnd(T, nkv, d, dtype=dtype, seed=2)
    kc, vc, table = make_paged(k, v, ps, T // ps + 2)
    q = rnd(T, nh, d, dtype=dtype, seed=3)
    te, to = prefill_tiles([(0, T, 0)], tile)
    assert te.numel() * nh >= 768
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    scale = 1 / math.sqrt(d)
    need = ops.attention_prefill_workspace(T, nh, d, T, window, te.numel())
    assert (need == 0) == (cuts == 1) and ops.attention_prefill_workspace(T, nh, d, T, window, 10) > need
    out = ops.attention_prefill(q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]), table[None].contiguous(),
                                nh, nkv, d, scale, window, max_keys=T, tile=tile)
    rows = sorted({0, 1, 63, 64, 2047, 2048, 2049, 6143, 6144, 6145, T // 2, T - 129, T - 1, 16383, 16384, 16385} & set(range(T)))
    G = nh // nkv
    for r in rows:
        lo = max(0, r - window + 1) if window else 0                       # a window of w keys: positions r-w+1 .. r
        kk, vv = k[lo:r + 1].float(), v[lo:r + 1].float()                  # [keys, nkv, d]
        for h in range(nh):
            p = torch.softmax((kk[:, h // G] @ q[r, h].float()) * scale, 0)
            ref = p @ vv[:, h // G]
            torch.testing.assert_close(out.view(T, nh, d)[r, h].float(), ref, atol=2e-2, rtol=2e-2)


def test_attention_prefill_far_key_stands_out(ops):
    """One far key among a thousand is made to dominate one query of a late tile."""
    nh, nkv, d, ps, T = 4, 1, 64, 16, 1100
    dtype = torch.bfloat16
    k, v = rnd(T, nkv, d, seed=1) * 0.1, rnd(T, nkv, d, seed=2)
    q = rnd(T, nh, d, seed=3) * 0.1
    far, who = 37, 1003
    q[who, 2] = rnd(d, seed=9)
    k[far, 0] = q[who, 2] * 60.0 / q[who, 2].norm() ** 2 * math.sqrt(d)
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    kc, vc, table = make_paged(k, v, ps, 80)
    te, to = prefill_tiles([(0, T, 0)])
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    out = ops.attention_prefill(q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]), table[None].contiguous(),
                                nh, nkv, d, 1 / math.sqrt(d))
    torch.testing.assert_close(out.view(T, nh, d)[who, 2].float(), v[far, 0].float(), atol=2e-2, rtol=2e-2)
    # with a window that ends just after the far key it is gone; one key wider and it is back
    for window, seen in ((who - far, False), (who - far + 1, True)):
        o = ops.attention_prefill(q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]),
                                  table[None].contiguous(), nh, nkv, d, 1 / math.sqrt(d), window)
        diff = float((o.view(T, nh, d)[who, 2].float() - v[far, 0].float()).abs().max())
        assert (diff < 2e-2) == seen, (window, diff)


def plant_far_key(q, k, who, head, far, d, seed):
    """Make key ``far`` dominate query (who, head): the query is drawn anew at full width, the key points along it
    with a score of 60 after the scale."""
    q[who, head] = rnd(d, seed=seed)
    k[far, 0] = q[who, head] * 60.0 / q[who, head].norm() ** 2 * math.sqrt(d)


@pytest.mark.parametrize("alone", [False, True])
def test_attention_prefill_long_cut_far_keys_stand_out(ops, alone):
    """The cut every 16,384 keys with single keys that dominate: a key of the first cut seen from the second (the
    two cuts are merged), keys just below and just above the cut's edge, and with a window across the edge one key
    inside it and one outside.  With keys and queries of unit width the softmax over thousands of keys is so flat
    that a lost block of 128 keys moves the output by less than the tolerance; a dominating key that is lost, or
    seen where it must not be, moves it by its whole size."""
    nh, nkv, d, ps, T, tile = 6, 1, 64, 16, 17000, 128
    dtype = torch.bfloat16
    k, v = rnd(T, nkv, d, seed=1) * 0.1, rnd(T, nkv, d, seed=2)
    q = rnd(T, nh, d, seed=3) * 0.1
    # (query row, head, far key)
    plants = [(16900, 0, 37), (16700, 1, 16383), (16800, 2, 16384), (16390, 3, 16389), (16500, 4, 2047), (9000, 5, 8191)]
    for i, (who, h, far) in enumerate(plants):
        plant_far_key(q, k, who, h, far, d, seed=20 + i)
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    kc, vc, table = make_paged(k, v, ps, T // ps + 2)
    te, to = prefill_tiles([(0, T, 0)], tile)
    assert te.numel() * nh >= 768 and ops.attention_prefill_workspace(T, nh, d, T, 0, te.numel()) > 0     # two long cuts
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    scale = 1 / math.sqrt(d)
    out = ops.attention_prefill(q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]), table[None].contiguous(),
                                nh, nkv, d, scale, max_keys=T, tile=tile, alone=alone).view(T, nh, d)
    for who, h, far in plants:
        torch.testing.assert_close(out[who, h].float(), v[far, 0].float(), atol=2e-2, rtol=2e-2,
                                   msg=lambda m: f"query {who} head {h} far key {far}: {m}")
    # a window of 600 keys across the 16,384 edge: the key inside it is seen, the one just outside is not
    window = 600
    inside, outside = (16700, 1, 16383), (16900, 0, 16900 - window)
    k2 = k.float()
    plant_far_key(q, k2, outside[0], outside[1], outside[2], d, seed=40)      # q keeps its type: rounded on assignment
    k2 = k2.to(dtype)
    kc2, vc2, table2 = make_paged(k2, v, ps, T // ps + 2)
    o = ops.attention_prefill(q.view(T, nh * d), kc2, vc2, te, to, dev([0]), dev([T]), dev([0]), table2[None].contiguous(),
                              nh, nkv, d, scale, window, max_keys=T, tile=tile, alone=alone).view(T, nh, d)
    torch.testing.assert_close(o[inside[0], inside[1]].float(), v[inside[2], 0].float(), atol=2e-2, rtol=2e-2)
    assert float((o[outside[0], outside[1]].float() - v[outside[2], 0].float()).abs().max()) > 0.5
    o = ops.attention_prefill(q.view(T, nh * d), kc2, vc2, te, to, dev([0]), dev([T]), dev([0]), table2[None].contiguous(),
                              nh, nkv, d, scale, window + 1, max_keys=T, tile=tile, alone=alone).view(T, nh, d)
    torch.testing.assert_close(o[outside[0], outside[1]].float(), v[outside[2], 0].float(), atol=2e-2, rtol=2e-2)


def test_attention_prefill_short_cut_far_keys_stand_out(ops):
    """The cut every 2,048 keys (a launch of few tiles): dominating keys just below and just above the edges at
    2,048 and 4,096, seen from queries of a later cut, with both tile sizes."""
    nh, nkv, d, ps, T = 3, 1, 128, 16, 4500
    dtype = torch.bfloat16
    k, v = rnd(T, nkv, d, seed=1) * 0.1, rnd(T, nkv, d, seed=2)
    q = rnd(T, nh, d, seed=3) * 0.1
    plants = [(4400, 0, 2047), (4300, 1, 2048), (4499, 2, 4095), (4200, 2, 4096), (2100, 1, 5), (2050, 0, 2049)]
    for i, (who, h, far) in enumerate(plants):
        plant_far_key(q, k, who, h, far, d, seed=60 + i)
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    kc, vc, table = make_paged(k, v, ps, T // ps + 2)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    for tile in (64, 128):
        te, to = prefill_tiles([(0, T, 0)], tile)
        assert ops.attention_prefill_workspace(T, nh, d, T, 0, te.numel()) > 0
        out = ops.attention_prefill(q.view(T, nh * d), kc, vc, te, to, dev([0]), dev([T]), dev([0]),
                                    table[None].contiguous(), nh, nkv, d, 1 / math.sqrt(d), max_keys=T, tile=tile).view(T, nh, d)
        for who, h, far in plants:
            torch.testing.assert_close(out[who, h].float(), v[far, 0].float(), atol=2e-2, rtol=2e-2,
                                       msg=lambda m: f"tile {tile} query {who} head {h} far key {far}: {m}")


def test_attention_prefill_refuses_other_shapes(ops):
    assert not ops.attention_prefill_supported(torch.float32, 12, 2, 128, 16)
    assert not ops.attention_prefill_supported(torch.bfloat16, 12, 2, 256, 16)
    assert not ops.attention_prefill_supported(torch.bfloat16, 12, 2, 40, 16)
    assert not ops.attention_prefill_supported(torch.bfloat16, 12, 2, 128, 24)
    assert not ops.attention_prefill_supported(torch.bfloat16, 12, 5, 128, 16)


# ---- the few-rows product's partial sums and the kernels that consume them ------------------------
@pytest.mark.parametrize("M,N,K", [(1, 2048, 1536), (8, 1536, 8960), (16, 17920, 1536), (13, 1536, 1536),
                                   (16, 2048, 1536), (5, 176, 64), (11, 1000, 96), (3, 48, 520), (2, 3584, 18944),
                                   (17, 1536, 1536), (64, 2048, 1536), (33, 1000, 96), (40, 1536, 8960), (64, 17920, 1536),
                                   (20, 100, 72), (65, 1536, 8960), (96, 2048, 1536), (100, 1000, 96), (128, 1536, 1536),
                                   (128, 1536, 8960), (113, 3584, 18944), (80, 48, 520)])
def test_linear_sums(ops, M, N, K):
    bf = torch.bfloat16
    # beyond 128 rows only large weights with twice as many columns as rows (the other test), beyond 256 none
    assert ops.SUMS_MAX_ROWS == 256 and not ops.linear_sums_supported(rnd(257, K, dtype=bf), rnd(N, K, dtype=bf))
    assert ops.linear_sums_supported(rnd(129, K, dtype=bf), rnd(N, K, dtype=bf)) == (K >= 2 * N and N * K >= 1 << 25)
    assert ops.linear_sums_supported(rnd(65, K, dtype=bf), rnd(N, K, dtype=bf))
    assert not ops.linear_sums_supported(rnd(65, K, dtype=bf), rnd(N, K, dtype=bf), ops.FEW_ROWS)
    x, w = rnd(M, K, dtype=bf, seed=1), rnd(N, K, dtype=bf, scale=0.05, seed=2)
    b = rnd(N, dtype=bf, seed=3)
    sums = ops.linear_sums(x, w)
    assert sums.shape == (ops.linear_splits(M, N, K), M, N) and sums.dtype == torch.float32
    ref = x.float() @ w.float().t()
    torch.testing.assert_close(sums.sum(0), ref, atol=2e-3, rtol=2e-3)
    # the consumer-side sum is what linear() itself gives, bit for bit (up to 64 rows: beyond, linear() is the
    # library's product)
    if M <= ops.FEW_ROWS:
        assert torch.equal(ops.reduce_sums(sums, b), ops.linear(x, w, b))
    else:
        torch.testing.assert_close(ops.reduce_sums(sums, b).float(), ops.linear(x, w, b).float(), atol=3e-2, rtol=3e-2)
    # a row's sums do not depend on the rows that ride along (up to 16 rows, and from 17 rows on, whichever of
    # the kernels for up to 64 and up to 128 rows makes them)
    if 1 < M <= 16:
        alone = ops.linear_sums(x[M - 1:M].contiguous(), w)
        assert torch.equal(alone[:, 0], sums[:, M - 1])
    if M > 17:
        fewer = ops.linear_sums(x[:17].contiguous(), w)
        assert torch.equal(fewer[:, 16], sums[:, 16])


@pytest.mark.parametrize("N,K", [(4120, 1024), (5456, 1024), (6168, 1024), (10256, 768), (4096, 1024)])
@pytest.mark.parametrize("M", [17, 33, 50, 64, 65, 81, 100, 128])
def test_linear_sums_with_workgroups_of_every_size(ops, M, N, K):
    """Weights whose cut gives workgroups of five, six, seven, eight and four wavefronts (on 256 compute units), at
    every number of 16-row tiles of x from two to eight: every thread of the workgroup stages its share of the
    block's x slice, and the last round of that passes the slice's end in some of these."""
    bf = torch.bfloat16
    x, w = rnd(M, K, dtype=bf, seed=M), rnd(N, K, dtype=bf, scale=0.05, seed=N)
    sums = ops.linear_sums(x, w)
    assert sums.shape == (ops.linear_splits(M, N, K), M, N)
    ref = x.float() @ w.float().t()
    torch.testing.assert_close(sums.sum(0), ref, atol=2e-3, rtol=2e-3)
    # row 16 as part of 17 rows: the same sums, whichever kernel and however many tiles
    if M > 17:
        assert torch.equal(ops.linear_sums(x[:17].contiguous(), w)[:, 16], sums[:, 16])


@pytest.mark.parametrize("M,I,K", [(1, 8960, 1536), (8, 8960, 1536), (14, 176, 64), (16, 256, 96), (2, 208, 80),
                                   (4, 18944, 3584), (64, 8960, 1536), (24, 176, 64), (50, 18944, 3584)])
def test_linear_swiglu(ops, M, I, K):
    from zedinfer_amd.parts.feed_forward import interleave_rows
    bf = torch.bfloat16
    x = rnd(M, K, dtype=bf, seed=1)
    g, u = rnd(I, K, dtype=bf, scale=0.08, seed=2), rnd(I, K, dtype=bf, scale=0.08, seed=3)
    w = interleave_rows(g, u, 8)
    assert torch.equal(w[:8], g[:8]) and torch.equal(w[8:16], u[:8]) and torch.equal(w[16:24], g[8:16])
    gf, uf = x.float() @ g.float().t(), x.float() @ u.float().t()
    ref = uf * torch.nn.functional.silu(gf)
    if ops.linear_swiglu_supported(x, w):
        out = ops.linear_swiglu(x, w)
        torch.testing.assert_close(out.float(), ref, atol=2e-2, rtol=2e-2)
    else:
        assert ops.linear_splits(M, 2 * I, K) > 1
    # the same through partial sums and the SwiGLU kernel, and through the interleaved 2-D form
    sums = ops.linear_sums(x, w)
    out2 = ops.swiglu(sums, interleave=8, out_dtype=bf)
    torch.testing.assert_close(out2.float(), ref, atol=2e-2, rtol=2e-2)
    gu = ops.linear(x, w)
    out3 = ops.swiglu(gu, interleave=8)
    torch.testing.assert_close(out3.float(), ref, atol=3e-2, rtol=3e-2)


def test_add_rms_norm_from_sums(ops):
    n, H, S = 9, 200, 3
    resid = rnd(n, H, seed=1)
    sums = rnd(S, n, H, seed=2)
    w = (1 + rnd(H, seed=3) * 0.1).to(torch.bfloat16)
    total = resid + sums[0] + sums[1] + sums[2]
    out = ops.add_rms_norm(resid, sums, w, 1e-5, out_dtype=torch.bfloat16)
    torch.testing.assert_close(resid, total, atol=1e-6, rtol=1e-6)
    ref = w.float() * total * torch.rsqrt((total * total).mean(-1, keepdim=True) + 1e-5)
    torch.testing.assert_close(out.float(), ref, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("with_bias", [True, False])
def test_rope_kv_store_sums(ops, dtype, with_bias):
    n, nh, nkv, d, ps, pages, theta, S = 7, 6, 2, 48, 8, 10, 5e4, 3
    width = (nh + 2 * nkv) * d
    sums = rnd(S, n, width, seed=1)
    bias = rnd(width, seed=2).to(dtype) if with_bias else None
    total = sums.sum(0) + (bias.float() if with_bias else 0)
    q, k, v = total[:, :nh * d], total[:, nh * d:(nh + nkv) * d], total[:, (nh + nkv) * d:]
    pos = torch.arange(100, 100 + n, dtype=torch.int32, device="cuda")
    slots = torch.randperm(pages * ps)[:n].to(torch.int32).cuda()
    kc = torch.zeros(pages, nkv, ps, d, dtype=dtype, device="cuda")
    vc = torch.zeros(pages, nkv, d, ps, dtype=dtype, device="cuda")
    q_out = torch.empty(n, nh * d, dtype=dtype, device="cuda")
    table = ops.rope_table(pos, ops.rope_inv_freq(d, theta, "cuda"))
    ops.rope_kv_store_sums(sums, bias, q_out, table, slots, kc, vc, nh, nkv, d)
    q_ref = torch_rope(q.reshape(n, nh, d), pos, theta)
    k_ref = torch_rope(k.reshape(n, nkv, d), pos, theta)
    torch.testing.assert_close(q_out.float().reshape(n, nh, d), q_ref, **tol(dtype, 5e-4, 3e-2))
    for t in range(n):
        p, o = int(slots[t]) // ps, int(slots[t]) % ps
        torch.testing.assert_close(kc[p, :, o].float(), k_ref[t], **tol(dtype, 5e-4, 3e-2))
        torch.testing.assert_close(vc[p, :, :, o].float(), v[t].reshape(nkv, d), **tol(dtype, 1e-6, 2e-2))
    # queries alone (a layer that reads another layer's cache)
    q2 = torch.empty_like(q_out)
    ops.rope_kv_store_sums(sums, bias, q2, table, None, None, None, nh, nkv, d)
    assert torch.equal(q2, q_out)
