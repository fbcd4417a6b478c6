"""A plain, slow Qwen2 forward pass: whole sequences, no cache, no paging, one
function per part, float32 (or float64) torch on the CPU.

It is written from the reference's formulas (each function cites file:line,
paths relative to the reference checkout) and shares no code with the engine:
it reads the model folder with the ``safetensors`` package and ``json``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """out[i,:] = table[ids[i],:], no scaling
    (src/backend/ops/embedding/cpu/embedding_cpu.cpp:10-23; src/frontend/models/transformer_forward.cpp:54-60)."""
    return table[ids.long()]


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = w * x / sqrt(mean(x^2) + eps), eps inside the root, plain w
    (src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:17-29; python/tests/ops/rms_norm.py:7-9)."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return w * (x / torch.sqrt(ms + eps))


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M,N] = x[M,K] . w[N,K]^T + b[N]
    (src/backend/ops/linear/op.cpp:57-58; src/backend/ops/linear/cpu/linear_cpu.cpp:26-85)."""
    y = x @ w.t()
    return y + b if b is not None else y


def rope_neox(x: torch.Tensor, pos: torch.Tensor, theta: float) -> torch.Tensor:
    """Split-half rotation of x [T, heads, d] by absolute positions pos [T]:
    angle_k = pos / theta^(2k/d); out[k] = a cos - b sin; out[k+d/2] = b cos + a sin
    with a = x[k], b = x[k+d/2]
    (src/backend/ops/rope/cpu/rope_cpu.cpp:33,47-52,62-65; python/tests/ops/rope.py:7-30)."""
    d = x.shape[-1]
    half = d // 2
    k = torch.arange(half, dtype=x.dtype)
    inv = 1.0 / torch.pow(torch.tensor(theta, dtype=x.dtype), 2.0 * k / d)
    ang = pos.to(x.dtype)[:, None] * inv[None, :]          # [T, d/2]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         window: Optional[int] = None) -> torch.Tensor:
    """q [T, nh, d], k and v [T, nkv, d], all of one sequence starting at position 0.
    Query row i, head h (kv head h // (nh/nkv)) sees keys j in [0, i]: s_j = (q.k_j) * scale
    (scale after the dot product), softmax with the maximum subtracted, o = sum_j P_j v_j
    (src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:106-162; the grouping at :111,
    the scale at :135, the causal bound at :116).  With ``window`` = W, only keys with
    i - j < W are seen; the reference parses the window keys but never uses them
    (src/frontend/models/base.cpp:807-813), so the windowed case is not pinned by it."""
    T, nh, d = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    out = torch.empty_like(q)
    for h in range(nh):
        g = h // group
        s = (q[:, h, :] @ k[:, g, :].t()) * scale            # [T, T]
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        visible = j <= i
        if window is not None:
            visible &= (i - j) < window
        s = s.masked_fill(~visible, float("-inf"))
        s = s - s.max(dim=-1, keepdim=True).values
        p = torch.exp(s)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """out = up * gate / (1 + exp(-gate))
    (src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23)."""
    return up * (gate / (1.0 + torch.exp(-gate)))


def argmax_lowest_index(logits: torch.Tensor) -> int:
    """Highest logit; the lowest index among equals
    (src/backend/ops/argmax/cpu/argmax_cpu.cpp:11-55, ties at :17-19)."""
    best, best_i = None, -1
    for i, v in enumerate(logits.tolist()):
        if best is None or v > best:
            best, best_i = v, i
    return best_i


# --------------------------------------------------------------------------
# blocks and the whole model
# --------------------------------------------------------------------------
def attention_block(x, w: Dict[str, torch.Tensor], p: str, cfg: dict, pos, window):
    """q/k/v projections with biases, rotation of q and k, attention, output projection
    without bias (src/frontend/models/transformer_forward.cpp:71-78, :99-112).  When the weights hold
    ``self_attn.q_norm.weight`` and ``self_attn.k_norm.weight`` [head_dim], every query and key head is RMS-normed
    over head_dim before the rotation (:80-96; Qwen2 checkpoints hold none)."""
    T = x.shape[0]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = linear(x, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
    k = linear(x, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
    v = linear(x, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
    if p + "self_attn.q_norm.weight" in w:
        eps = cfg.get("rms_norm_eps", 1e-6)
        q = rms_norm(q.view(T, nh, d), w[p + "self_attn.q_norm.weight"], eps).reshape(T, nh * d)
        k = rms_norm(k.view(T, nkv, d), w[p + "self_attn.k_norm.weight"], eps).reshape(T, nkv * d)
    q = rope_neox(q.view(T, nh, d), pos, cfg["rope_theta"])
    k = rope_neox(k.view(T, nkv, d), pos, cfg["rope_theta"])
    a = causal_gqa_attention(q, k, v.view(T, nkv, d), 1.0 / math.sqrt(d), window)
    return linear(a.reshape(T, nh * d), w[p + "self_attn.o_proj.weight"])


def mlp_block(x, w: Dict[str, torch.Tensor], p: str):
    """down(swiglu(gate(x), up(x))), no biases (transformer_forward.cpp:128-137)."""
    g = linear(x, w[p + "mlp.gate_proj.weight"])
    u = linear(x, w[p + "mlp.up_proj.weight"])
    return linear(swiglu(g, u), w[p + "mlp.down_proj.weight"])


def layer_window(cfg: dict, layer: int) -> Optional[int]:
    """Qwen2's config keys: with use_sliding_window, layers from max_window_layers on use a
    window of sliding_window keys; the others see all keys.  (Keys parsed at
    src/frontend/models/base.cpp:807-813 and unused by the reference.)"""
    if cfg.get("use_sliding_window", False) and layer >= cfg.get("max_window_layers", 21):
        return int(cfg.get("sliding_window", 4096))
    return None


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: Sequence[int],
            dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.  Pre-norm residual blocks: h += attn(norm(h));
    h += mlp(norm(h)); final norm; LM head, tied to the embedding table when the file has no
    lm_head.weight (transformer_forward.cpp:63-156; tie at src/frontend/models/base.cpp:410-416)."""
    cfg = normalized_config(cfg)
    w = {k: v.to(dtype) for k, v in w.items()}
    ids_t = torch.tensor(list(ids), dtype=torch.long)
    pos = torch.arange(len(ids), dtype=torch.long)
    eps = cfg["rms_norm_eps"]
    h = embedding(ids_t, w["model.embed_tokens.weight"])
    for L in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{L}."
        x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        h = h + attention_block(x, w, p, cfg, pos, layer_window(cfg, L))
        x = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + mlp_block(x, w, p)
    h = rms_norm(h, w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(h, head)


def normalized_config(cfg: dict) -> dict:
    """Defaults of the optional keys (src/frontend/models/base.cpp:683-720)."""
    c = dict(cfg)
    c.setdefault("num_key_value_heads", c["num_attention_heads"])
    if not c.get("head_dim"):
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    c.setdefault("rms_norm_eps", 1e-6)
    c.setdefault("rope_theta", 10000.0)
    c.setdefault("tie_word_embeddings", False)
    return c


def load_folder(folder: str):
    """(config dict, {tensor name: tensor}) of a model folder, read with the safetensors package."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, w


def greedy_generate(cfg: dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], n: int,
                    dtype: torch.dtype = torch.float32) -> List[int]:
    """n greedy tokens, recomputing the whole sequence each time."""
    ids = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(cfg, w, ids, dtype)
        t = int(torch.argmax(logits[-1]).item())
        out.append(t)
        ids.append(t)
    return out


# --------------------------------------------------------------------------
# sampling (src/frontend/sampler/sampler.cpp:195-265, :410-490)
# --------------------------------------------------------------------------
def truncated_distribution(logits: torch.Tensor, temperature: float, top_k: int, top_p: float,
                           repetition_penalty: float = 1.0, recent: Sequence[int] = ()):
    """(probabilities, token ids), sorted by falling probability, after repetition penalty on
    raw logits (l > 0 ? l / p : l * p, applied once per listed token occurrence), temperature,
    softmax, top-k, top-p (smallest prefix whose sum reaches top_p) and renormalisation."""
    l = logits.to(torch.float32).clone()
    if repetition_penalty != 1.0:
        for t in recent:
            if 0 <= t < l.numel():
                l[t] = l[t] / repetition_penalty if l[t] > 0 else l[t] * repetition_penalty
    if temperature != 1.0:
        l = l / temperature
    p = torch.exp(l - l.max())
    p = p / p.sum()
    order = torch.sort(p, descending=True, stable=True)
    probs, idx = order.values, order.indices
    if 0 < top_k < probs.numel():
        probs, idx = probs[:top_k], idx[:top_k]
    if top_p < 1.0:
        c = torch.cumsum(probs, 0)
        cut = int((c >= top_p).nonzero()[0].item()) + 1 if bool((c >= top_p).any()) else probs.numel()
        probs, idx = probs[:cut], idx[:cut]
    probs = probs / probs.sum()
    return probs, idx
