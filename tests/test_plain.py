"""What pins the plain implementation beside the reference's text: special cases that reduce to a
library routine, invariants, and small vectors worked by hand; each chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, a scale before the dot product's
sum, a mask off by one) fails it (CPU)."""
import math

import pytest
import torch
import torch.nn.functional as F

import tiny_configs
from plain import qwen2_plain as plain

torch.manual_seed(0)


def test_rms_norm_reduces_to_the_library_and_keeps_eps_inside_the_root():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, torch.ones(48, dtype=torch.float64), 1e-6),
                               F.rms_norm(x, (48,), eps=1e-6))
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6), F.rms_norm(x, (48,), weight=w, eps=1e-6))
    # a tiny row: eps dominates, y = w x / sqrt(eps); an eps outside the root would give w x / (rms + eps)
    tiny = torch.full((1, 4), 1e-6, dtype=torch.float64)
    y = plain.rms_norm(tiny, torch.ones(4, dtype=torch.float64), 1e-2)
    torch.testing.assert_close(y, tiny / math.sqrt(1e-12 + 1e-2))
    # scale equivariance for eps -> 0, and the weight is plain w, not 1 + w
    torch.testing.assert_close(plain.rms_norm(3 * x, w, 1e-30), plain.rms_norm(x, w, 1e-30))
    assert float(plain.rms_norm(x, torch.zeros(48, dtype=torch.float64), 1e-6).abs().max()) == 0.0


def test_rope_by_hand_pairs_and_signs():
    # d = 4: pairs are (0, 2) and (1, 3); frequencies theta^0 = 1 and theta^(-1/2)
    theta, p = 100.0, 3.0
    pos = torch.tensor([3])
    e0 = torch.tensor([[[1.0, 0, 0, 0]]], dtype=torch.float64)
    e2 = torch.tensor([[[0, 0, 1.0, 0]]], dtype=torch.float64)
    e1 = torch.tensor([[[0, 1.0, 0, 0]]], dtype=torch.float64)
    torch.testing.assert_close(plain.rope_neox(e0, pos, theta)[0, 0],
                               torch.tensor([math.cos(p), 0, math.sin(p), 0], dtype=torch.float64))
    torch.testing.assert_close(plain.rope_neox(e2, pos, theta)[0, 0],
                               torch.tensor([-math.sin(p), 0, math.cos(p), 0], dtype=torch.float64))
    a = p / 10.0
    torch.testing.assert_close(plain.rope_neox(e1, pos, theta)[0, 0],
                               torch.tensor([0, math.cos(a), 0, math.sin(a)], dtype=torch.float64))


def test_rope_invariants():
    x = torch.randn(6, 3, 32, dtype=torch.float64)
    pos = torch.arange(6)
    assert torch.equal(plain.rope_neox(x[:1], torch.tensor([0]), 1e4), x[:1])       # position 0 is the identity
    y = plain.rope_neox(x, pos + 500, 1e6)
    pair = lambda t: t[..., :16] ** 2 + t[..., 16:] ** 2  # noqa: E731
    torch.testing.assert_close(pair(y), pair(x))                                     # each pair keeps its length
    # <R_m q, R_n k> depends on m - n only
    q, k = torch.randn(1, 1, 32, dtype=torch.float64), torch.randn(1, 1, 32, dtype=torch.float64)
    dot = lambda m, n: float((plain.rope_neox(q, torch.tensor([m]), 1e4) * plain.rope_neox(k, torch.tensor([n]), 1e4)).sum())  # noqa: E731
    assert dot(7, 3) == pytest.approx(dot(104, 100), rel=1e-12)
    assert dot(7, 3) != pytest.approx(dot(3, 7), rel=1e-6)
    # the reference's own test formula: python/tests/ops/rope.py:7-30
    i = torch.arange(16, dtype=torch.float64)
    fr = (pos + 500).double()[:, None] / (1e6 ** (2 * i / 32))
    a, b = x[..., :16], x[..., 16:]
    ref = torch.cat([a * fr.cos()[:, None] - b * fr.sin()[:, None], b * fr.cos()[:, None] + a * fr.sin()[:, None]], -1)
    torch.testing.assert_close(y, ref)


def test_attention_reduces_to_the_library():
    T, nh, nkv, d = 9, 6, 2, 16
    q, k, v = (torch.randn(T, n, d, dtype=torch.float64) for n in (nh, nkv, nkv))
    scale = 1 / math.sqrt(d)
    out = plain.causal_gqa_attention(q, k, v, scale)
    kk, vv = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)    # head h uses kv head h // group
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(out, lib.transpose(0, 1))
    # the last row sees everything: plain softmax(q K^T * scale) V without any mask
    last = torch.softmax((q[-1, 0] @ k[:, 0].t()) * scale, -1) @ v[:, 0]
    torch.testing.assert_close(out[-1, 0], last)
    # the first row sees only itself
    torch.testing.assert_close(out[0], vv[0])
    # one head, one kv head
    o1 = plain.causal_gqa_attention(q[:, :1], k[:, :1], v[:, :1], scale)
    torch.testing.assert_close(o1, F.scaled_dot_product_attention(q[:, :1].transpose(0, 1), k[:, :1].transpose(0, 1),
                                                                  v[:, :1].transpose(0, 1), is_causal=True).transpose(0, 1))
    # uniform values come back unchanged
    u = torch.ones(T, nkv, d, dtype=torch.float64) * 0.37
    torch.testing.assert_close(plain.causal_gqa_attention(q, k, u, scale), torch.full_like(q, 0.37))
    # the reference's own mask: python/tests/ops/self_attention.py:7-26, tril(diagonal = S - L)
    mask = torch.ones(T, T, dtype=torch.bool).tril(diagonal=0)
    s = (q[:, 3] @ kk[:, 3].t()) * scale
    torch.testing.assert_close(out[:, 3], torch.softmax(s.masked_fill(~mask, float("-inf")), -1) @ vv[:, 3])


def test_attention_window():
    T, d = 12, 8
    q, k, v = (torch.randn(T, 1, d, dtype=torch.float64) for _ in range(3))
    full = plain.causal_gqa_attention(q, k, v, 0.3)
    torch.testing.assert_close(plain.causal_gqa_attention(q, k, v, 0.3, window=T), full)
    torch.testing.assert_close(plain.causal_gqa_attention(q, k, v, 0.3, window=1), v)   # only itself
    w3 = plain.causal_gqa_attention(q, k, v, 0.3, window=3)
    i = 7
    torch.testing.assert_close(w3[i, 0], torch.softmax((q[i, 0] @ k[5:8, 0].t()) * 0.3, -1) @ v[5:8, 0])
    torch.testing.assert_close(w3[:3], full[:3])


def test_swiglu_embedding_linear_argmax():
    g, u = torch.randn(4, 10, dtype=torch.float64) * 3, torch.randn(4, 10, dtype=torch.float64)
    torch.testing.assert_close(plain.swiglu(g, u), F.silu(g) * u)
    E = torch.randn(20, 6)
    assert torch.equal(plain.embedding(torch.tensor([3, 19, 3]), E), F.embedding(torch.tensor([3, 19, 3]), E))
    x, w, b = torch.randn(3, 6), torch.randn(5, 6), torch.randn(5)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))
    assert plain.argmax_lowest_index(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1      # first among equals


def tiny_weights(name, seed=0):
    import torch
    from zedinfer_amd.config import Qwen2Config
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import random_weights
    cfg = Qwen2Config.from_dict(tiny_configs.CONFIGS[name])
    w = random_weights(expected_weights(qwen2_forward_config(cfg)), seed, torch.float64, noisy_norms=True, std=0.1)
    if cfg.tie_word_embeddings:
        del w["lm_head.weight"]
    return dict(tiny_configs.CONFIGS[name]), w


def test_attention_block_depends_on_distances_only():
    """A shift of all positions changes nothing in the attention block: only distances count."""
    cfg, w = tiny_weights("B")
    cfg = plain.normalized_config(cfg)
    x = torch.randn(10, 96, dtype=torch.float64)
    a0 = plain.attention_block(x, w, "model.layers.0.", cfg, torch.arange(10), None)
    a1 = plain.attention_block(x, w, "model.layers.0.", cfg, torch.arange(10) + 777, None)
    torch.testing.assert_close(a0, a1, atol=1e-9, rtol=1e-9)
    # while a change of distances does
    a2 = plain.attention_block(x, w, "model.layers.0.", cfg, torch.arange(10) * 2, None)
    assert float((a0 - a2).abs().max()) > 1e-4


def test_optional_norm_of_query_and_key_heads():
    """With q_norm / k_norm gains among the weights every query and key head is normed over head_dim before the
    rotation: the size of the projections then does not matter (a norm after the biases, before anything else),
    the gains do, one per dim (which a norm placed after the rotation would pair differently), and gains of one
    with unit-RMS heads change nothing."""
    cfg, w = tiny_weights("B")
    cfg = plain.normalized_config(dict(cfg, rms_norm_eps=1e-30))
    p, d = "model.layers.0.", cfg["head_dim"]
    x = torch.randn(9, 96, dtype=torch.float64)
    w = dict(w)
    w[p + "self_attn.q_norm.weight"] = 1 + 0.3 * torch.randn(d, dtype=torch.float64)
    w[p + "self_attn.k_norm.weight"] = 1 + 0.3 * torch.randn(d, dtype=torch.float64)
    a0 = plain.attention_block(x, w, p, cfg, torch.arange(9), None)
    bigger = dict(w)
    for name in ("q_proj.weight", "q_proj.bias", "k_proj.weight", "k_proj.bias"):
        bigger[p + "self_attn." + name] = 5.0 * w[p + "self_attn." + name]
    torch.testing.assert_close(plain.attention_block(x, bigger, p, cfg, torch.arange(9), None), a0, atol=1e-9, rtol=1e-9)
    other = dict(w)
    other[p + "self_attn.k_norm.weight"] = w[p + "self_attn.k_norm.weight"].flip(0)
    assert float((plain.attention_block(x, other, p, cfg, torch.arange(9), None) - a0).abs().max()) > 1e-4
    # the gain of dim k multiplies dim k of the normed head before the rotation mixes dims k and k + d/2: with the
    # two halves' gains exchanged and the head's halves exchanged by hand the result differs, so the order matters
    nh = cfg["num_attention_heads"]
    q = plain.linear(x, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).view(9, nh, d)
    normed_then_rotated = plain.rope_neox(plain.rms_norm(q, w[p + "self_attn.q_norm.weight"], 1e-30), torch.arange(9), cfg["rope_theta"])
    rotated_then_normed = plain.rms_norm(plain.rope_neox(q, torch.arange(9), cfg["rope_theta"]), w[p + "self_attn.q_norm.weight"], 1e-30)
    assert float((normed_then_rotated - rotated_then_normed).abs().max()) > 1e-3
    # without the gains among the weights nothing is normed
    plainly = {k: v for k, v in w.items() if "_norm.weight" not in k or "layernorm" in k}
    assert float((plain.attention_block(x, plainly, p, cfg, torch.arange(9), None) - a0).abs().max()) > 1e-4


def test_model_norm_and_residual_placement():
    cfg, w = tiny_weights("A")
    ids = [5, 17, 3, 300, 5]
    E = w["model.embed_tokens.weight"]
    eps = cfg["rms_norm_eps"]
    # (1) with the output projections silenced the blocks add nothing: logits = E . norm(E[ids])
    z = {k: (torch.zeros_like(v) if ("o_proj" in k or "down_proj" in k) else v) for k, v in w.items()}
    h = F.rms_norm(E[ids], (64,), weight=w["model.norm.weight"], eps=eps)
    torch.testing.assert_close(plain.forward(cfg, z, ids, torch.float64), h @ E.t())
    # (2) values made uniform (v weights 0, a constant bias): attention returns the bias for every token,
    #     so layer 0 adds o_proj(bias) to the raw embedding, not to its norm, and the feed-forward
    #     reads the norm of that sum
    one = {k: v.clone() for k, v in z.items()}
    bias = torch.randn(32, dtype=torch.float64)
    one["model.layers.0.self_attn.v_proj.weight"].zero_()
    one["model.layers.0.self_attn.v_proj.bias"] = bias
    one["model.layers.0.self_attn.o_proj.weight"] = w["model.layers.0.self_attn.o_proj.weight"]
    one["model.layers.0.mlp.down_proj.weight"] = w["model.layers.0.mlp.down_proj.weight"]
    att = bias.view(2, 16).repeat_interleave(2, 0).reshape(64)         # kv head of head h is h // 2
    h1 = E[ids] + F.linear(att, one["model.layers.0.self_attn.o_proj.weight"])
    y = F.rms_norm(h1, (64,), weight=w["model.layers.0.post_attention_layernorm.weight"], eps=eps)
    mlp = F.linear(F.silu(F.linear(y, w["model.layers.0.mlp.gate_proj.weight"])) *
                   F.linear(y, w["model.layers.0.mlp.up_proj.weight"]), w["model.layers.0.mlp.down_proj.weight"])
    h2 = h1 + mlp
    want = F.rms_norm(h2, (64,), weight=w["model.norm.weight"], eps=eps) @ E.t()
    torch.testing.assert_close(plain.forward(cfg, one, ids, torch.float64), want)


def test_model_is_causal_and_untied_head_is_used():
    cfg, w = tiny_weights("B")
    ids = [1, 50, 999, 7, 7, 123]
    full = plain.forward(cfg, w, ids, torch.float64)
    torch.testing.assert_close(plain.forward(cfg, w, ids[:4], torch.float64), full[:4])   # later tokens do not reach back
    w2 = dict(w)
    w2["lm_head.weight"] = w["lm_head.weight"] * 2
    torch.testing.assert_close(plain.forward(cfg, w2, ids, torch.float64), full * 2)


def test_window_layers_follow_the_config():
    cfg, w = tiny_weights("C")
    assert [plain.layer_window(cfg, L) for L in range(3)] == [None, 20, 20]
    ids = list(range(3, 43))
    full = plain.forward(dict(cfg, use_sliding_window=False), w, ids, torch.float64)
    win = plain.forward(cfg, w, ids, torch.float64)
    torch.testing.assert_close(win[:20], full[:20])                  # inside the window nothing differs
    assert float((win[25:] - full[25:]).abs().max()) > 1e-6
    torch.testing.assert_close(plain.forward(dict(cfg, sliding_window=40), w, ids, torch.float64), full)


def test_sampling_distribution():
    # reference: tests/sampler/test_sampler.cpp:157-202
    logits = torch.tensor([1.0, 3.0, 2.0, -1.0, 2.5])
    p, idx = plain.truncated_distribution(logits, 0.01, 0, 1.0)
    assert idx[0].item() == 1 and p[0].item() > 0.999                # T -> 0 is argmax
    p, idx = plain.truncated_distribution(logits, 1.0, 2, 1.0)
    assert idx.tolist() == [1, 4] and p.sum().item() == pytest.approx(1.0)
    p, idx = plain.truncated_distribution(torch.tensor([10.0, 0.0, 0.0, 0.0]), 1.0, 0, 0.5)
    assert idx.tolist() == [0]                                       # a dominant token fills top_p alone
    sm = torch.softmax(logits, 0)
    p, idx = plain.truncated_distribution(logits, 1.0, 0, float(sm[1] + sm[4]) - 1e-4)
    assert idx.tolist() == [1, 4]                                    # smallest prefix that reaches top_p
    p, idx = plain.truncated_distribution(logits, 1.0, 0, 1.0, repetition_penalty=2.0, recent=[1, 3, 1])
    l2 = logits.clone()
    l2[1] = 3.0 / 4.0                                                # penalised once per occurrence
    l2[3] = -2.0
    torch.testing.assert_close(p[idx.argsort()], torch.softmax(l2, 0))
