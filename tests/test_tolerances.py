"""Can the bfloat16 tolerance of the GPU tests fail?  The plain implementation is run with one
plausible mistake at a time (no rotation, a rotation with the wrong sign or pairing, no 1/sqrt(d), a
causal bound off by one, a page of keys taken from the wrong place, a missing bias) on the
configurations and requests the GPU tests use, and the shift of the logits is held against the
tolerance the GPU tests apply.  With the narrow N(0, 0.02) weights of the tiny configurations attention
is nearly uniform and several of these pass unseen, which is why the GPU tests run "sharp" variants as
well; with those every mistake exceeds the tolerance several times over, while a forward pass that
rounds every op's result to bfloat16 stays at a third of it or less."""
import contextlib

import pytest
import torch

import tiny_configs
import traces
from plain import qwen2_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, bf16_within, sharp_std


def model(name, std, dtype=torch.bfloat16):
    from zedinfer_amd.config import Qwen2Config
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import random_weights
    cfgd = tiny_configs.CONFIGS[name] if isinstance(name, str) else name
    cfg = Qwen2Config.from_dict(cfgd)
    seed = tiny_configs.SEEDS.get(name, 7) if isinstance(name, str) else 7
    w = random_weights(expected_weights(qwen2_forward_config(cfg)), seed, dtype, noisy_norms=True, std=std)
    if cfg.tie_word_embeddings:
        del w["lm_head.weight"]
    return dict(cfgd), {k: v.float() for k, v in w.items()}


@contextlib.contextmanager
def patched(**fns):
    old = {n: getattr(plain, n) for n in fns}
    for n, f in fns.items():
        setattr(plain, n, f)
    try:
        yield old
    finally:
        for n, f in old.items():
            setattr(plain, n, f)


REAL = dict(plain.__dict__)      # the unpatched functions


def rope_interleaved(x, pos, theta):
    """The pairing (2k, 2k+1) instead of (k, k + d/2)."""
    d = x.shape[-1]
    k = torch.arange(d // 2, dtype=x.dtype)
    ang = pos.to(x.dtype)[:, None] / torch.pow(torch.tensor(theta, dtype=x.dtype), 2.0 * k / d)[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2], out[..., 1::2] = a * cos - b * sin, b * cos + a * sin
    return out


def attention_missing_own_key(q, k, v, scale, window=None):
    """Query i sees keys [0, i - 1]: the bound one too low (the first query keeps its own key)."""
    out = REAL["causal_gqa_attention"](q, k, v, scale, window).clone()
    T, nh, d = q.shape
    group = nh // k.shape[1]
    for h in range(nh):
        g = h // group
        s = (q[:, h] @ k[:, g].t()) * scale
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        vis = (j < i) | ((i == 0) & (j == 0))
        if window is not None:
            vis &= (i - j) < window
        p = torch.softmax(s.masked_fill(~vis, float("-inf")), -1)
        out[:, h] = p @ v[:, g]
    return out


def attention_wrong_page(page):
    """Keys and values of positions [page, 2 page) are those of [0, page): a block table entry that names
    the wrong page."""
    def f(q, k, v, scale, window=None):
        k, v = k.clone(), v.clone()
        n = min(page, k.shape[0] - page)
        if n > 0:
            k[page:page + n], v[page:page + n] = k[:n].clone(), v[:n].clone()
        return REAL["causal_gqa_attention"](q, k, v, scale, window)
    return f


def linear_without_bias_of(width):
    def f(x, w, b=None):
        return REAL["linear"](x, w, None if (b is not None and b.numel() == width) else b)
    return f


def mistakes(cfg):
    c = plain.normalized_config(cfg)
    qd = c["num_attention_heads"] * c["head_dim"]
    ps = 8 if c["hidden_size"] in (96, 80) else 16
    return {
        "no rotation": dict(rope_neox=lambda x, pos, theta: x),
        "rotation with the wrong sign": dict(rope_neox=lambda x, pos, theta: REAL["rope_neox"](x, -pos, theta)),
        "rotation of neighbouring pairs": dict(rope_neox=rope_interleaved),
        "no 1/sqrt(d)": dict(causal_gqa_attention=lambda q, k, v, s, window=None:
                             REAL["causal_gqa_attention"](q, k, v, 1.0, window)),
        "causal bound one too low": dict(causal_gqa_attention=attention_missing_own_key),
        "a wrong page": dict(causal_gqa_attention=attention_wrong_page(ps)),
        "no query bias": dict(linear=linear_without_bias_of(qd)),
    }


def shift(cfg, w, reqs, ref, **fns):
    """(worst, mean) difference of the patched forward pass from ``ref``, relative to the largest |logit|."""
    worst = total = 0.0
    scale = max(float(r.abs().max()) for r in ref.values())
    with patched(**fns):
        for rid, toks in reqs.items():
            d = (plain.forward(cfg, w, toks) - ref[rid]).abs()
            worst, total = max(worst, float(d.max())), total + float(d.mean(dim=-1).sum())
    return worst / scale, total / sum(len(t) for t in reqs.values()) / scale


def rounded(fn):
    return lambda *a, **k: fn(*a, **k).to(torch.bfloat16).float()


ROUNDING = {n: rounded(REAL[n]) for n in ("linear", "rms_norm", "rope_neox", "swiglu", "causal_gqa_attention")}


def requests_of(name, cfg, count=4):
    from test_engine_gpu import LENGTHS
    lens = sorted(LENGTHS[name], reverse=True)[:count]
    return {f"r{i}": traces.random_tokens(cfg["vocab_size"], n, seed=100 + i) for i, n in enumerate(lens)}


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_mistake_exceeds_the_tolerance_with_sharp_weights(name):
    cfg, w = model(name, tiny_configs.SHARP_STD)
    reqs = requests_of(name, cfg)
    ref = {rid: plain.forward(cfg, w, toks) for rid, toks in reqs.items()}
    for what, fns in mistakes(cfg).items():
        worst, mean = shift(cfg, w, reqs, ref, **fns)
        print(f"{name} sharp, {what}: worst {worst:.3f} mean {mean:.4f} of the largest logit")
        # twice the tolerance in one measure at least (either fails a GPU test): a loosened tolerance fails
        # here before it hides a mistake
        assert worst > 2 * BF16_REL_WORST or mean > 2 * BF16_REL_MEAN, what
        assert not bf16_within(worst, mean, 1.0)
    worst, mean = shift(cfg, w, reqs, ref, **ROUNDING)
    print(f"{name} sharp, every op rounded to bfloat16: worst {worst:.4f} mean {mean:.5f}")
    assert worst < BF16_REL_WORST / 3 and mean < BF16_REL_MEAN / 3


def test_narrow_weights_hide_the_rotation():
    """Why the sharp variants exist: with N(0, 0.02) weights a forward pass without rotation stays inside
    the tolerance."""
    for name in "AB":
        cfg, w = model(name, 0.02)
        reqs = requests_of(name, cfg, 2)
        ref = {rid: plain.forward(cfg, w, toks) for rid, toks in reqs.items()}
        ms = mistakes(cfg)
        for what in ("no rotation", "rotation with the wrong sign"):
            worst, mean = shift(cfg, w, reqs, ref, **ms[what])
            assert bf16_within(worst, mean, 1.0), (name, what, worst, mean)


def test_real_layer_shapes_are_sharp_as_they_are():
    """Two layers of the 1.5B sizes with N(0, 0.02) weights (tests/test_real_shapes_gpu.py): queries and
    keys are 1,536 terms wide there, and every mistake already shows."""
    from test_real_shapes_gpu import SHAPES
    cfgd = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=4099, max_position_embeddings=4096,
                num_hidden_layers=2, rope_theta=1000000.0, rms_norm_eps=1e-6, use_sliding_window=False,
                torch_dtype="float32", eos_token_id=4098, **SHAPES["1.5B"])
    assert abs(sharp_std(cfgd["hidden_size"]) - 0.02) < 0.001
    cfg, w = model(cfgd, 0.02)
    reqs = {"p": traces.random_tokens(4099, 72, seed=1)}
    ref = {"p": plain.forward(cfg, w, reqs["p"])}
    ms = mistakes(cfg)
    for what in ("no rotation", "no 1/sqrt(d)", "causal bound one too low", "a wrong page"):
        worst, mean = shift(cfg, w, reqs, ref, **ms[what])
        print(f"1.5B sizes, {what}: worst {worst:.3f} mean {mean:.4f}")
        assert worst > 2 * BF16_REL_WORST or mean > 2 * BF16_REL_MEAN, what


@pytest.mark.parametrize("seed", [0, 5, 102])
def test_sweep_configurations_are_sharp(seed):
    """The seeded configurations of tests/test_config_sweep_gpu.py with their bfloat16 checkpoint's width."""
    from test_config_sweep_gpu import configuration
    c, _ = configuration(seed)
    cfg, w = model(c, sharp_std(c["hidden_size"]))
    reqs = {"r": traces.random_tokens(c["vocab_size"], 100, seed=seed)}
    ref = {"r": plain.forward(cfg, w, reqs["r"])}
    ms = mistakes(cfg)
    for what in ("no rotation", "no 1/sqrt(d)"):
        worst, mean = shift(cfg, w, reqs, ref, **ms[what])
        print(f"sweep seed {seed}, {what}: worst {worst:.3f} mean {mean:.4f}")
        assert worst > 2 * BF16_REL_WORST or mean > 2 * BF16_REL_MEAN, what
    worst, mean = shift(cfg, w, reqs, ref, **ROUNDING)
    assert worst < BF16_REL_WORST / 2 and mean < BF16_REL_MEAN / 2, (worst, mean)
