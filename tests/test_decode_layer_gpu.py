"""The resident decoder-layer kernel (one launch a layer for up to 16 decoded tokens) alone, against a plain
float32 torch computation of the same layer over the same paged cache (formulas of the reference's layer:
src/frontend/models/transformer_forward.cpp:63-149), at sizes other than the tiny models'."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from zedinfer_amd import ops as o
    o.load()
    return o


def rnd(*shape, scale=1.0, seed=0, dtype=torch.float32):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


def bf(x):
    return x.to(torch.bfloat16).float()


def reference_layer(resid, g1, g2, eps1, eps2, wqkv, bias, wo, wg, wu, wd, pos, theta, rot, nh, nkv, d, scale, window,
                    past_k, past_v):
    """float32, with the activations rounded to bfloat16 where the kernel rounds them.  past_k / past_v: per token
    [p, nkv, d] cached keys and values of its sequence.  Returns (new residual, new keys, new values)."""
    n, H = resid.shape
    Qd, KVd = nh * d, nkv * d

    def norm(x, g, eps):
        return g * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    x1 = bf(norm(resid, g1, eps1))
    qkv = x1 @ wqkv.t() + (bias if bias is not None else 0.0)
    q, k, v = qkv[:, :Qd].view(n, nh, d).clone(), qkv[:, Qd:Qd + KVd].view(n, nkv, d).clone(), qkv[:, Qd + KVd:].view(n, nkv, d)
    if rot:
        half = rot // 2
        inv = theta ** (-torch.arange(0, half, dtype=torch.float32, device=resid.device) * 2.0 / rot)
        ang = pos.float()[:, None] * inv[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        for x in (q, k):
            a, b = x[..., :half].clone(), x[..., half:rot].clone()
            x[..., :half] = a * cos - b * sin
            x[..., half:rot] = b * cos + a * sin
    q, k, v = bf(q), bf(k), bf(v)
    G = nh // nkv
    att = torch.zeros(n, nh, d, device=resid.device)
    for t in range(n):
        p = int(pos[t])
        lo = max(0, p - window + 1) if window else 0
        kk = torch.cat([past_k[t][lo:p], k[t:t + 1]], 0)         # [keys, nkv, d]
        vv = torch.cat([past_v[t][lo:p], v[t:t + 1]], 0)
        for h in range(nh):
            s = (kk[:, h // G] @ q[t, h]) * scale
            att[t, h] = torch.softmax(s, 0) @ vv[:, h // G]
    att = bf(att).view(n, Qd)
    r2 = resid + att @ wo.t()
    x2 = bf(norm(r2, g2, eps2))
    gate, up = x2 @ wg.t(), x2 @ wu.t()
    h = bf(up * (gate / (1.0 + torch.exp(-gate))))
    return r2 + h @ wd.t(), k, v


CASES = [
    # n, H, I, nh, nkv, d, rot, ps, window, bias, positions
    dict(n=8, H=1536, I=8960, nh=12, nkv=2, d=128, rot=128, ps=16, window=0, bias=True, pos=[2100, 2047, 300, 1, 0, 999, 1500, 2200]),
    dict(n=1, H=1536, I=8960, nh=12, nkv=2, d=128, rot=128, ps=16, window=0, bias=True, pos=[700]),
    dict(n=16, H=896, I=4864, nh=14, nkv=2, d=64, rot=64, ps=16, window=0, bias=True, pos=list(range(40, 1000, 60))),
    dict(n=5, H=200, I=344, nh=6, nkv=3, d=48, rot=32, ps=8, window=50, bias=False, pos=[0, 7, 49, 50, 333]),
    dict(n=3, H=96, I=256, nh=3, nkv=1, d=32, rot=0, ps=8, window=0, bias=True, pos=[130, 5, 64]),
    # more attention tasks (12 tokens x 8 kv heads x 3 chunks) than the 256 workgroups, and the first token without
    # cached keys: a workgroup whose first task has nothing to read goes on to one that has
    dict(n=12, H=512, I=1024, nh=16, nkv=8, d=64, rot=64, ps=16, window=0, bias=True, pos=[0] + [2990 + i for i in range(11)]),
    dict(n=11, H=3584, I=18944, nh=28, nkv=4, d=128, rot=128, ps=32, window=0, bias=True, pos=list(range(100, 1200, 100))),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"n{c['n']}_H{c['H']}_d{c['d']}")
def test_decode_layer_against_torch(ops, case):
    from zedinfer_amd.parts.feed_forward import GATE_UP_BLOCK, interleave_rows
    n, H, I, nh, nkv, d, rot, ps, window = (case[k] for k in ("n", "H", "I", "nh", "nkv", "d", "rot", "ps", "window"))
    print(f"decode_layer case {case}", flush=True)
    bt16 = torch.bfloat16
    Qd, KVd = nh * d, nkv * d
    std = 0.8 / math.sqrt(H)
    wqkv = rnd(Qd + 2 * KVd, H, scale=std, seed=1, dtype=bt16)
    bias = rnd(Qd + 2 * KVd, scale=0.3, seed=2, dtype=bt16) if case["bias"] else None
    wo = rnd(H, Qd, scale=0.5 / math.sqrt(Qd), seed=3, dtype=bt16)
    wg, wu = rnd(I, H, scale=std, seed=4, dtype=bt16), rnd(I, H, scale=std, seed=5, dtype=bt16)
    wd = rnd(H, I, scale=0.5 / math.sqrt(I), seed=6, dtype=bt16)
    g1, g2 = (1 + rnd(H, scale=0.1, seed=7)).to(bt16), (1 + rnd(H, scale=0.1, seed=8)).to(bt16)
    eps1, eps2, theta, scale = 1e-6, 3e-6, 10000.0, 1.0 / math.sqrt(d)
    resid = rnd(n, H, seed=9)
    pos = torch.tensor(case["pos"], dtype=torch.int32, device="cuda")
    assert len(case["pos"]) == n
    # every token's sequence has its own pages, dealt out of a shuffled pool
    pages_each = [(p + 1 + ps - 1) // ps for p in case["pos"]]
    num_pages = sum(pages_each) + 3
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(11)).tolist()
    kc = torch.full((num_pages, nkv, ps, d), float("nan"), dtype=bt16, device="cuda")
    vc = torch.full((num_pages, nkv, d, ps), float("nan"), dtype=bt16, device="cuda")
    width = max(pages_each) + 2
    table = torch.full((n, width), -1, dtype=torch.int32)
    past_k, past_v, slots = [], [], []
    for t, p in enumerate(case["pos"]):
        mine = [perm.pop() for _ in range(pages_each[t])]
        table[t, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        k = rnd(max(p, 1), nkv, d, seed=100 + t, dtype=bt16)[:p]
        v = rnd(max(p, 1), nkv, d, seed=200 + t, dtype=bt16)[:p]
        for i in range(p):
            kc[mine[i // ps], :, i % ps] = k[i]
            vc[mine[i // ps], :, :, i % ps] = v[i]
        past_k.append(k.float())
        past_v.append(v.float())
        slots.append(mine[p // ps] * ps + p % ps)
    table = table.cuda()
    slots_t = torch.tensor(slots, dtype=torch.int32, device="cuda")
    max_keys = max(case["pos"]) + 1
    assert ops.decode_layer_supported(bt16, n, H, I, nh, nkv, d, rot, ps, max_keys, window)
    ws = torch.empty(ops.decode_layer_workspace(n, H, I, nh, nkv, d, max_keys, window), dtype=torch.uint8, device="cuda")
    sync = torch.zeros(ops.decode_layer_sync_words(), dtype=torch.int32, device="cuda")
    err = torch.zeros(1, dtype=torch.int32).pin_memory()
    rope = None
    if rot:
        rope = ops.rope_table(pos, ops.rope_inv_freq(rot, theta, torch.device("cuda")))
    want, k_new, v_new = reference_layer(resid, g1.float(), g2.float(), eps1, eps2, wqkv.float(),
                                         bias.float() if bias is not None else None, wo.float(), wg.float(), wu.float(),
                                         wd.float(), pos, theta, rot, nh, nkv, d, scale, window, past_k, past_v)
    wgu = interleave_rows(wg, wu, GATE_UP_BLOCK)
    got = resid.clone()
    for rep in range(2):         # twice: the synchronisation state carries over from launch to launch
        got.copy_(resid)
        ops.decode_layer(got, g1, g2, eps1, eps2, False, wqkv, bias, wo, wgu, wd, rope, slots_t, kc, vc, pos, table,
                         nh, nkv, d, scale, max_keys, window, ws, sync, err)
        torch.cuda.synchronize()
        assert int(err[0]) == 0, "a wait inside the kernel ran out"
        assert not torch.isnan(got).any()
        # against what the layer adds to the residual, not the residual itself (which is as large and exact)
        big = float((want - resid).abs().max())
        worst = float((got - want).abs().max())
        print(f"rep {rep}: worst difference {worst:.3e}, the layer adds up to {big:.3e}", flush=True)
        assert worst <= 0.02 * big
    # the tokens' new keys and values lie in the cache
    for t, p in enumerate(case["pos"]):
        page, off = slots[t] // ps, slots[t] % ps
        torch.testing.assert_close(kc[page, :, off].float(), k_new[t], atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(vc[page, :, :, off].float(), v_new[t], atol=2e-2, rtol=2e-2)


def test_decode_layer_reports_a_wait_that_ran_out(ops):
    """With a spin limit that no barrier can meet, every workgroup gives up its wait and leaves: the kernel ends, the
    host's flag is set, the output is NaN; after the state is zeroed the next call is right again."""
    n, H, I, nh, nkv, d, ps = 4, 256, 512, 4, 2, 64, 16
    bt16 = torch.bfloat16
    Qd, KVd = nh * d, nkv * d
    wqkv, wo = rnd(Qd + 2 * KVd, H, scale=0.05, seed=1, dtype=bt16), rnd(H, Qd, scale=0.05, seed=2, dtype=bt16)
    wgu, wd = rnd(2 * I, H, scale=0.05, seed=3, dtype=bt16), rnd(H, I, scale=0.05, seed=4, dtype=bt16)
    g1, g2 = torch.ones(H, dtype=bt16, device="cuda"), torch.ones(H, dtype=bt16, device="cuda")
    pos = torch.tensor([40, 3, 17, 60], dtype=torch.int32, device="cuda")
    table = torch.arange(n * 4, dtype=torch.int32, device="cuda").view(n, 4)          # 4 pages a token
    slots = (table[torch.arange(n), (pos // ps).long()] * ps + pos % ps).to(torch.int32)
    kc = rnd(n * 4, nkv, ps, d, seed=5, dtype=bt16)
    vc = rnd(n * 4, nkv, d, ps, seed=6, dtype=bt16)
    rope = ops.rope_table(pos, ops.rope_inv_freq(d, 10000.0, torch.device("cuda")))
    ws = torch.empty(ops.decode_layer_workspace(n, H, I, nh, nkv, d, 64, 0), dtype=torch.uint8, device="cuda")
    sync = torch.zeros(ops.decode_layer_sync_words(), dtype=torch.int32, device="cuda")
    err = torch.zeros(1, dtype=torch.int32).pin_memory()
    resid = rnd(n, H, seed=7)

    def run(spin_limit):
        out = resid.clone()
        ops.decode_layer(out, g1, g2, 1e-6, 1e-6, False, wqkv, None, wo, wgu, wd, rope, slots, kc, vc, pos, table,
                         nh, nkv, d, d ** -0.5, 64, 0, ws, sync, err, spin_limit=spin_limit)
        torch.cuda.synchronize()
        return out
    print("decode_layer with a spin limit of 1", flush=True)
    out = run(1)
    assert int(err[0]) == 1
    assert torch.isnan(out).all()
    err.zero_()
    sync.zero_()
    torch.cuda.synchronize()
    good = run(ops.DECODE_LAYER_SPIN_LIMIT)
    assert int(err[0]) == 0 and not torch.isnan(good).any()
    again = run(ops.DECODE_LAYER_SPIN_LIMIT)
    assert torch.equal(good, again)


def test_decode_layer_refuses_what_it_does_not_take(ops):
    bt16 = torch.bfloat16
    assert not ops.decode_layer_supported(bt16, 17, 1536, 8960, 12, 2, 128, 128, 16, 2048)
    assert not ops.decode_layer_supported(torch.float32, 8, 1536, 8960, 12, 2, 128, 128, 16, 2048)
    assert not ops.decode_layer_supported(bt16, 8, 1536, 8960, 12, 2, 256, 256, 16, 2048)
    assert not ops.decode_layer_supported(bt16, 8, 1540, 8960, 12, 2, 128, 128, 16, 2048)
    assert not ops.decode_layer_supported(bt16, 8, 1536, 8960, 12, 2, 128, 128, 12, 2048)
    assert ops.decode_layer_supported(bt16, 8, 1536, 8960, 12, 2, 128, 128, 16, 2048)
