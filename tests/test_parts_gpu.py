"""Each part alone against the plain functions, and two toy architectures defined here, registered, built
and stepped through the engine without a change to the framework's files: one with a mixer that keeps a
state of its own per request; one with a feed-forward that routes tokens to experts, a position encoding
of its own, and a run order that names a layer twice and lets a layer read another layer's cache."""
import json
import math
import os

import pytest
import torch

import traces
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]


def tol(dtype, f32=2e-5, bf16=3e-2):
    return dict(atol=f32, rtol=f32) if dtype == torch.float32 else dict(atol=bf16, rtol=bf16)


def assert_close_to_scale(got, ref, dtype, f32=2e-5, bf16=0.02):
    """Largest difference against the largest |reference| (bfloat16 rounds every intermediate to 8 bits
    of mantissa, so an element near zero carries the rounding of the large terms it is the sum of)."""
    scale = float(ref.abs().max())
    worst = float((got - ref).abs().max())
    assert worst <= (f32 if dtype == torch.float32 else bf16) * max(scale, 1e-6), (worst, scale)


def as_rows(t):
    """A part may return its addition as a stack [S, n, H] of float32 partial sums."""
    return t.float().sum(0) if t.dim() == 3 else t.float()


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + 7 * len(shape) + sum(shape))
    return torch.randn(*shape, generator=g) * scale


def runtime(dtype):
    from zedinfer_amd.parts import Runtime
    return Runtime(torch.device("cuda", torch.cuda.current_device()), dtype)


def spec(kind, params=None, weights=None):
    from zedinfer_amd.config.forward_config import PartSpec
    return PartSpec(kind, params or {}, weights or {})


def one_sequence_batch(cache, seq, tokens_or_n, vocab=1 << 30, planners=()):
    """The device batch of one entry that brings n tokens to ``seq``."""
    from zedinfer_amd.engine.batch import StepEntry, build_device_batch
    toks = list(tokens_or_n) if not isinstance(tokens_or_n, int) else [0] * tokens_or_n
    cache.ensure(seq, seq.length + len(toks))
    return build_device_batch([StepEntry(seq, toks, [])], cache, vocab, cache.device, planners=planners)


# ---- norm -------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("add_one", [False, True])
def test_rmsnorm_part(dtype, add_one):
    from zedinfer_amd.parts import NORMS
    n, H, eps = 9, 200, 3e-4
    w = 1 + rnd(H, seed=1, scale=0.3)
    x = rnd(n, H, seed=2, scale=2.0)
    part = NORMS.get("rmsnorm")(spec("rmsnorm", {"dim": H, "eps": eps, "add_one": add_one}),
                                {"weight": w.to(dtype).cuda()}, runtime(dtype))
    wp = w.to(dtype).float() + (1.0 if add_one else 0.0)
    got = part.forward(x.to(dtype).cuda()).float().cpu()
    torch.testing.assert_close(got, plain.rms_norm(x.to(dtype).float(), wp, eps), **tol(dtype))
    # the fused form: the float32 residual takes the addition, the output is the norm of the sum
    resid = x.clone().cuda()
    delta = rnd(n, H, seed=3).to(dtype).cuda()
    got = part.add_forward(resid, delta).float().cpu()
    total = x + delta.float().cpu()
    torch.testing.assert_close(resid.cpu(), total, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(got, plain.rms_norm(total, wp, eps), **tol(dtype))


# ---- feed-forward -----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n", [1, 7, 130])
def test_swiglu_part(dtype, n):
    from zedinfer_amd.parts import FEED_FORWARDS
    H, I = 72, 200
    w = {"gate": rnd(I, H, seed=1, scale=0.2), "up": rnd(I, H, seed=2, scale=0.2), "down": rnd(H, I, seed=3, scale=0.2)}
    x = rnd(n, H, seed=4)
    part = FEED_FORWARDS.get("swiglu")(spec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                                       {k: v.to(dtype).cuda() for k, v in w.items()}, runtime(dtype))
    got = as_rows(part.forward(x.to(dtype).cuda())).cpu()
    wf = {k: v.to(dtype).float() for k, v in w.items()}
    xf = x.to(dtype).float()
    ref = plain.linear(plain.swiglu(plain.linear(xf, wf["gate"]), plain.linear(xf, wf["up"])), wf["down"])
    assert_close_to_scale(got, ref, dtype)


@pytest.mark.parametrize("n,H,I", [(256, 72, 200), (136, 96, 72), (1024, 128, 344)])
def test_swiglu_part_both_orientations_of_the_product(n, H, I, monkeypatch):
    """Many rows in bfloat16: the library may make the gate/up product faster transposed.  Both ways,
    chosen here through the runtime's recorded choices, give the plain result (and nearly each other's);
    without a choice the forward pass takes the straight one and measures nothing; ``tune`` measures
    outside of a step, records its decision, and the forward pass then follows it.  (The library keeps its
    first algorithm for every product here, so that bits can be compared before and after ``tune``.)"""
    from zedinfer_amd.parts import FEED_FORWARDS
    monkeypatch.setenv("ZEDINFER_TUNE_LIBRARY", "0")
    dtype = torch.bfloat16
    w = {"gate": rnd(I, H, seed=1, scale=0.2), "up": rnd(I, H, seed=2, scale=0.2), "down": rnd(H, I, seed=3, scale=0.2)}
    x = rnd(n, H, seed=4)
    rt = runtime(dtype)
    part = FEED_FORWARDS.get("swiglu")(spec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                                       {k: v.to(dtype).cuda() for k, v in w.items()}, rt)
    wf = {k: v.to(dtype).float() for k, v in w.items()}
    xf = x.to(dtype).float()
    ref = plain.linear(plain.swiglu(plain.linear(xf, wf["gate"]), plain.linear(xf, wf["up"])), wf["down"])
    key = ("gate_up_transposed", n, 2 * I, H)
    got = {}
    assert not rt.choices
    default = as_rows(part.forward(x.to(dtype).cuda())).cpu()
    assert not rt.choices                                   # a step decides and measures nothing
    for wins in (False, True):
        rt.choices[key] = wins
        got[wins] = as_rows(part.forward(x.to(dtype).cuda())).cpu()
        assert_close_to_scale(got[wins], ref, dtype)
    assert torch.equal(default, got[False])
    del rt.choices[key]
    part.tune(n)
    assert isinstance(rt.choices.get(key), bool)
    part.tune(n)                                            # decided once
    measured = as_rows(part.forward(x.to(dtype).cuda())).cpu()
    assert torch.equal(measured, got[rt.choices[key]])
    torch.testing.assert_close(got[True], got[False], atol=2e-2 * float(ref.abs().max()), rtol=0)


def test_library_algorithms_are_chosen_at_warm_up_and_can_be_repeated(tmp_path, monkeypatch):
    """``Engine.warm_up`` lets the parts time the library's proposals for their many-rows products and records
    what was taken; a second engine given those choices puts them in force without timing; with
    ZEDINFER_TUNE_LIBRARY=0 nothing is timed or recorded.  Steps of that many rows agree with the plain
    implementation whatever was chosen."""
    import tiny_configs
    import traces
    from plain import qwen2_plain as plain_model
    from tolerances import bf16_within
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.ops import _lib
    folder = tiny_configs.write_tiny(str(tmp_path / "m"), "B", dtype=torch.bfloat16, std=tiny_configs.SHARP_STD)
    cfg, w = plain_model.load_folder(folder)
    ps = tiny_configs.PAGE_SIZES["B"]
    sched = SchedulerConfig(num_kv_blocks=64, kv_block_size=ps, max_batch_requests=4)
    calls = []
    real = _lib.call
    monkeypatch.setattr(_lib, "call", lambda name, *a: (calls.append(name), real(name, *a))[1])
    first = Engine.from_folder(folder, "bfloat16", sched)
    choices = first.warm_up([192])
    products = {k: v for k, v in choices.items() if k[0] == "library_product"}
    assert len(products) >= 4 and all(k[1] == 192 and isinstance(v, int) for k, v in products.items()), choices
    assert calls.count("zi_gemm_lt_tune") == len(products)      # a shape is timed once; later layers take the record
    calls.clear()
    second = Engine.from_folder(folder, "bfloat16", sched)
    assert second.warm_up([192], choices=choices) == choices
    assert calls.count("zi_gemm_lt_choose") >= len(products) and "zi_gemm_lt_tune" not in calls
    toks = traces.random_tokens(cfg["vocab_size"], 192, seed=3)
    ref = plain_model.forward(cfg, w, toks)
    for e in (first, second):
        seq = e.open("r")
        got = e.step([StepEntry(seq, toks, list(range(192)))]).cpu()
        d = (got - ref).abs()
        assert bf16_within(float(d.max()), float(d.mean()), float(ref.abs().max()))
        e.close(seq)
    monkeypatch.setenv("ZEDINFER_TUNE_LIBRARY", "0")
    calls.clear()
    third = Engine.from_folder(folder, "bfloat16", sched)
    assert not [k for k in third.warm_up([320]) if k[0] == "library_product"]
    assert "zi_gemm_lt_tune" not in calls


# ---- embedding and head -----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
def test_embedding_and_head_parts(dtype):
    from zedinfer_amd.parts import EMBEDDINGS, HEADS
    V, H = 333, 56
    table = rnd(V, H, seed=1).to(dtype)
    rt = runtime(dtype)
    emb = EMBEDDINGS.get("token")(spec("token", {"vocab_size": V, "hidden_size": H}), {"weight": table.cuda()}, rt)
    ids = torch.tensor([0, 332, 17, 17], dtype=torch.int32, device="cuda")
    out = emb.forward(ids)
    assert out.dtype == torch.float32 and torch.equal(out.cpu(), plain.embedding(ids.long().cpu(), table.float()))
    head = HEADS.get("linear")(spec("linear", {"vocab_size": V, "hidden_size": H, "tied_to": None}),
                               {"weight": table.cuda()}, rt)
    x = rnd(5, H, seed=2).to(dtype)
    logits = head.forward(x.cuda())
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), plain.linear(x.float(), table.float()), **tol(dtype, 2e-5, 1e-3))


# ---- position encoding ------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rotary_dim", [48, 16])
def test_rope_part_encodes_and_hands_over_the_table_the_store_kernel_takes(dtype, rotary_dim):
    """The encoding alone: ``encode`` turns q and k in place; ``step_table`` gives the step's (cos, sin), with which
    the store kernel (the attention's fast path) turns q in place and puts the turned k and the raw v into a cache."""
    from types import SimpleNamespace
    from zedinfer_amd import ops
    from zedinfer_amd.parts import POSITION_ENCODINGS
    n, nh, nkv, d, ps, pages, theta = 6, 4, 2, 48, 8, 5, 3e4
    part = POSITION_ENCODINGS.get("rope_neox")(spec("rope_neox", {"head_dim": d, "theta": theta,
                                                                   "rotary_dim": rotary_dim}), {}, runtime(dtype))
    qkv = rnd(n, (nh + 2 * nkv) * d, seed=1).to(dtype).cuda()
    qkv2 = qkv.clone()
    q, k, v = qkv[:, :nh * d], qkv[:, nh * d:(nh + nkv) * d], qkv[:, (nh + nkv) * d:]
    q0, k0, v0 = q.float().cpu().clone(), k.float().cpu().clone(), v.clone()
    pos = torch.arange(20, 20 + n, dtype=torch.int32, device="cuda")
    slots = torch.tensor([3, 9, 17, 39, 0, 8], dtype=torch.int32, device="cuda")

    def ref(x, heads):
        x = x.view(n, heads, d).clone()
        x[..., :rotary_dim] = plain.rope_neox(x[..., :rotary_dim].contiguous(), pos.long().cpu(), theta)
        return x
    part.encode(q, k, pos, nh, nkv, d)
    torch.testing.assert_close(q.float().cpu().view(n, nh, d), ref(q0, nh), **tol(dtype, 5e-4, 2e-2))
    torch.testing.assert_close(k.float().cpu().view(n, nkv, d), ref(k0, nkv), **tol(dtype, 5e-4, 2e-2))
    assert torch.equal(v, v0)
    # the table, and the kernel that turns and stores by it
    batch = SimpleNamespace(shared={}, num_tokens=n, positions=pos)
    table = part.step_table(batch)
    assert tuple(table.shape) == (n, rotary_dim // 2, 2) and part.step_table(batch) is table      # once a step
    q2, k2, v2 = qkv2[:, :nh * d], qkv2[:, nh * d:(nh + nkv) * d], qkv2[:, (nh + nkv) * d:]
    kc = torch.zeros(pages, nkv, ps, d, dtype=dtype, device="cuda")
    vc = torch.zeros(pages, nkv, d, ps, dtype=dtype, device="cuda")
    ops.rope_kv_store(q2, k2, v2, table, slots, kc, vc, nh, nkv, d)
    assert torch.equal(q2, q)                        # the same turn, bit for bit
    assert torch.equal(k2.float().cpu(), k0.to(dtype).float())      # k itself is left as it was
    for t in range(n):
        p, o = int(slots[t]) // ps, int(slots[t]) % ps
        torch.testing.assert_close(kc[p, :, o].float(), k[t].view(nkv, d).float(), **tol(dtype, 1e-6, 1e-2))
        assert torch.equal(vc[p, :, :, o], v0[t].view(nkv, d))
    # keys and values that are encoded already are stored as they are
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.kv_store(k, v, slots, kc2, vc2, nkv, d)
    assert torch.equal(vc2, vc)
    for t in range(n):
        p, o = int(slots[t]) // ps, int(slots[t]) % ps
        assert torch.equal(kc2[p, :, o], k[t].view(nkv, d))


# ---- mixer ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,d,window,bias,qk_norm", [(6, 2, 32, 0, True, False), (5, 1, 48, 11, False, False),
                                                          (4, 4, 64, 0, True, False), (6, 2, 32, 0, True, True),
                                                          (5, 1, 48, 11, False, True)])
def test_attention_part_in_portions(dtype, nh, nkv, d, window, bias, qk_norm):
    """The attention mixer alone, fed a sequence in portions (a long one, then short ones and single
    tokens), against the plain attention block over the whole sequence; also with every query and key head
    normed before the rotation (an option of the part that the architecture built here does not use)."""
    from zedinfer_amd.cache.manager import CacheManager
    from zedinfer_amd.parts import MIXERS
    H, T, ps, theta = 88, 61, 8, 7e3
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "qb", "k_bias": "kb", "v_bias": "vb"}
    w = {"q": rnd(nh * d, H, seed=1, scale=0.15), "k": rnd(nkv * d, H, seed=2, scale=0.15),
         "v": rnd(nkv * d, H, seed=3, scale=0.15), "o": rnd(H, nh * d, seed=4, scale=0.15),
         "q_bias": rnd(nh * d, seed=5, scale=0.5), "k_bias": rnd(nkv * d, seed=6, scale=0.5),
         "v_bias": rnd(nkv * d, seed=7, scale=0.5)}
    if not bias:
        w = {k: v for k, v in w.items() if not k.endswith("bias")}
    eps = 3e-4
    if qk_norm:
        names.update({"q_norm": "qn", "k_norm": "kn"})
        w.update({"q_norm": 1 + rnd(d, seed=11, scale=0.3), "k_norm": 1 + rnd(d, seed=12, scale=0.3)})
    w = {k: v.to(dtype) for k, v in w.items()}
    rt = runtime(dtype)
    sp = spec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "qkv_bias": bias,
                            "window": window, "qk_norm": qk_norm, "qk_norm_eps": eps,
                            "position": spec("rope_neox", {"head_dim": d, "theta": theta, "rotary_dim": d})}, names)
    mixer = MIXERS.get("attention")(sp, {k: v.cuda() for k, v in w.items()}, rt)
    cache = CacheManager({0: mixer.cache_request()}, {}, 16, ps, 2, dtype, rt.device, max_step_tokens=64)
    from zedinfer_amd.config.forward_config import ScheduleStep
    mem = cache.memories([ScheduleStep(0, 0)])[0]
    x = rnd(T, H, seed=8).to(dtype)
    seq = cache.open("s")
    got, i = [], 0
    for n in [23, 2, 1, 9, 1, 1, 3, 20, 1]:
        batch = one_sequence_batch(cache, seq, n, planners=[mixer.planner()])
        got.append(as_rows(mixer.forward(x[i:i + n].cuda(), batch, mem)).cpu())
        cache.commit(seq, seq.length + n)
        i += n
    assert i == T
    cfg = {"num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d, "rope_theta": theta, "rms_norm_eps": eps}
    wf = {"L.self_attn.q_proj.weight": w["q"], "L.self_attn.k_proj.weight": w["k"], "L.self_attn.v_proj.weight": w["v"],
          "L.self_attn.o_proj.weight": w["o"]}
    if qk_norm:
        wf.update({"L.self_attn.q_norm.weight": w["q_norm"], "L.self_attn.k_norm.weight": w["k_norm"]})
    if bias:
        wf.update({"L.self_attn.q_proj.bias": w["q_bias"], "L.self_attn.k_proj.bias": w["k_bias"],
                   "L.self_attn.v_proj.bias": w["v_bias"]})
    ref = plain.attention_block(x.float(), {k: v.float() for k, v in wf.items()}, "L.", cfg,
                                torch.arange(T), window or None)
    assert_close_to_scale(torch.cat(got), ref, dtype, 3e-5, 0.02)
    cache.close(seq)
    cache.check()


# ---- a toy architecture with a stateful mixer ---------------------------------------------------
def _define_toy():
    """A mixer with a fixed-size state per request, y_t = s_t . Wout with s_t = decay * s_{t-1} + x_t . Win,
    and an architecture that alternates it with attention.  Everything is registered from here."""
    from dataclasses import dataclass
    from typing import Dict, Optional

    from zedinfer_amd.config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, default_schedule
    from zedinfer_amd.config.model_config import ModelConfig
    from zedinfer_amd.config.registry import register_architecture, registered_architectures
    from zedinfer_amd.parts import MIXERS, Mixer, StateRequest, register_mixer
    from zedinfer_amd.weights.loader import WeightSpec

    if "ToyStateForCausalLM" in registered_architectures():
        return

    @register_mixer("toy_decayed_sum")
    class DecayedSum(Mixer):
        @staticmethod
        def weight_specs(spec) -> Dict[str, WeightSpec]:
            H, S = int(spec.params["hidden_size"]), int(spec.params["state_size"])
            return {"win": WeightSpec((S, H)), "wout": WeightSpec((H, S))}

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.S = int(spec.params["state_size"])
            self.decay = float(spec.params["decay"])
            self.win, self.wout = weights["win"].float(), weights["wout"].float()

        def state_request(self) -> Optional[StateRequest]:
            return StateRequest((self.S,), torch.float32)

        def forward(self, x, batch, memory):
            u = x.float() @ self.win.t()
            out = torch.empty_like(u)
            for start, n, slot in zip(batch.host_start, batch.host_len, batch.host_slot):
                s = memory.state[int(slot)]
                for t in range(int(start), int(start) + int(n)):
                    s = self.decay * s + u[t]
                    out[t] = s
                memory.state[int(slot)] = s
            return (out @ self.wout.t()).to(x.dtype)

    @register_mixer("toy_decayed_sum_on_device")
    class DecayedSumOnDevice(DecayedSum):
        """The same mixer with nothing but launches over device arrays, so that its steps can be captured
        as graphs.  It keeps state per request, so padding would advance it: ``padding_safe`` stays False
        (the default) and the engine must not pad its steps."""

        graph_safe = True

        def forward(self, x, batch, memory):
            u = x.float() @ self.win.t()                                        # [n, S]
            t = torch.arange(batch.num_tokens, device=x.device)
            entry = batch.tok_seq.long()
            j = (batch.positions - batch.entry_past[entry]).float()             # place of the token in its entry
            same = (entry[:, None] == entry[None, :]) & (t[None, :] <= t[:, None])
            m = torch.where(same, self.decay ** (t[:, None] - t[None, :]).clamp(min=0).float(), 0.0)
            s0 = memory.state[batch.entry_slot.long()][entry]                   # every token's starting state
            s = m @ u + (self.decay ** (j + 1.0))[:, None] * s0
            last = (batch.entry_start + batch.entry_len - 1).long()
            memory.state.index_copy_(0, batch.entry_slot.long(), s[last])
            return (s @ self.wout.t()).to(x.dtype)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        toy_state_size: int = 8
        toy_decay: float = 0.5

        @classmethod
        def from_dict(cls, d):
            kw = cls._base_kwargs(d)
            kw["toy_state_size"] = int(d["toy_state_size"])
            kw["toy_decay"] = float(d["toy_decay"])
            cfg = cls(**kw)
            cfg.validate()
            return cfg

    def toy_forward_config(cfg: ToyConfig, kind: str = "toy_decayed_sum") -> ModelForwardConfig:
        H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        layers = []
        for L in range(cfg.num_hidden_layers):
            p = f"model.layers.{L}."
            if L % 2 == 0:
                mixer = PartSpec(kind, {"hidden_size": H, "state_size": cfg.toy_state_size,
                                                     "decay": cfg.toy_decay},
                                 {"win": p + "toy.win.weight", "wout": p + "toy.wout.weight"})
            else:
                mixer = PartSpec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                               "qkv_bias": False, "window": 0,
                                               "position": PartSpec("rope_neox", {"head_dim": d, "theta": cfg.rope_theta})},
                                 {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                                  "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"})
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size},
                           {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                            "down": p + "mlp.down_proj.weight"})
            norms = {"input": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": p + "input_layernorm.weight"}),
                     "post_mixer": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps},
                                            {"weight": p + "post_attention_layernorm.weight"})}
            layers.append(LayerSpec("prenorm", mixer, ffn, norms))
        return ModelForwardConfig(
            architecture="ToyStateForCausalLM", hidden_size=H, vocab_size=cfg.vocab_size,
            embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "model.embed_tokens.weight"}),
            layers=tuple(layers), schedule=default_schedule(cfg.num_hidden_layers),
            final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
            lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None},
                             {"weight": "lm_head.weight"}))

    register_architecture("ToyStateForCausalLM", ToyConfig, toy_forward_config)
    register_architecture("ToyStateOnDeviceForCausalLM", ToyConfig,
                          lambda cfg: toy_forward_config(cfg, "toy_decayed_sum_on_device"))


TOY = dict(architectures=["ToyStateForCausalLM"], model_type="toy_state", hidden_size=48, intermediate_size=80,
           vocab_size=301, max_position_embeddings=256, num_hidden_layers=3, num_attention_heads=3,
           num_key_value_heads=1, head_dim=16, rope_theta=5000.0, rms_norm_eps=2e-6, toy_state_size=10, toy_decay=0.75)


def toy_plain_forward(cfg, w, ids):
    T = len(ids)
    pos = torch.arange(T)
    eps = cfg["rms_norm_eps"]
    h = plain.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for L in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{L}."
        x = plain.rms_norm(h, w[p + "input_layernorm.weight"], eps)
        if L % 2 == 0:
            u = x @ w[p + "toy.win.weight"].t()
            s = torch.zeros(cfg["toy_state_size"])
            ys = []
            for t in range(T):
                s = cfg["toy_decay"] * s + u[t]
                ys.append(s)
            h = h + torch.stack(ys) @ w[p + "toy.wout.weight"].t()
        else:
            h = h + plain.attention_block(x, w, p, cfg, pos, None)
        x = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + plain.mlp_block(x, w, p)
    return plain.linear(plain.rms_norm(h, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_stateful_mixer(tmp_path, dtype):
    _define_toy()
    from zedinfer_amd.config import SchedulerConfig, load_config
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.weights import write_model_folder
    folder = str(tmp_path / "toy")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY, f)
    arch, cfg = load_config(folder)
    assert arch.name == "ToyStateForCausalLM"
    write_model_folder(folder, cfg, expected_weights(arch.forward_config(cfg)), seed=5, dtype=torch.float32,
                       std=0.08, noisy_norms=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY, f)
    pcfg, w = plain.load_folder(folder)
    requests = {f"t{i}": traces.random_tokens(TOY["vocab_size"], n, seed=40 + i) for i, n in enumerate([37, 64, 9, 50, 23])}
    ref = {rid: toy_plain_forward(pcfg, w, toks) for rid, toks in requests.items()}
    engine = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=24, kv_block_size=8, max_batch_requests=4))
    assert len(engine.cache.state) == 2 and len(engine.cache.tensors) == 1     # two stateful layers, one with a cache
    for make in (traces.whole, traces.portions, traces.mixed):
        steps = make(requests)
        out = traces.run_in_process(engine, steps)
        worst, mean, scale, rows, where = traces.compare(steps, out, ref, requests)
        assert rows == sum(len(t) for t in requests.values())
        if dtype == "float32":
            assert worst <= 2e-4 * max(1.0, scale), where
        else:
            assert worst <= 0.08 * scale and mean <= 0.015 * scale, where
    # slots were reused by later requests and started from a zero state each time
    assert engine.cache.slots.takes > engine.cache.slots.total


def test_steps_of_a_stateful_mixer_are_not_padded(tmp_path, monkeypatch):
    """A mixer with state per request that can be captured as a graph: decode steps replay as graphs, but
    prompt portions, whose graphs need padding, run as they are, because the mixer does not say that
    padding is harmless to it.  With the flag forced the padding tokens advance the state and the logits
    are wrong, which is what the flag is for."""
    _define_toy()
    from zedinfer_amd.config import SchedulerConfig, load_config
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.parts import MIXERS
    from zedinfer_amd.weights import write_model_folder
    toy = dict(TOY, architectures=["ToyStateOnDeviceForCausalLM"], model_type="toy_state_on_device")
    folder = str(tmp_path / "toy")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(toy, f)
    arch, cfg = load_config(folder)
    write_model_folder(folder, cfg, expected_weights(arch.forward_config(cfg)), seed=5, dtype=torch.float32,
                       std=0.08, noisy_norms=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(toy, f)
    pcfg, w = plain.load_folder(folder)
    toks = {r: traces.random_tokens(toy["vocab_size"], 150, seed=60 + i) for i, r in enumerate("abc")}
    ref = {r: toy_plain_forward(pcfg, w, t) for r, t in toks.items()}

    def run(engine):
        """Portions of 35 tokens (a shape that recurs: it would be padded to 64 and recorded), then single
        tokens; the worst difference from the plain implementation."""
        seqs = {r: engine.open(r) for r in toks}
        fed = {r: 0 for r in toks}
        worst = 0.0
        plan = [[(r, 35)] for _ in range(3) for r in "abc"] + [[("a", 1), ("b", 1), ("c", 1)]] * 20
        for step in plan:
            out = engine.step([StepEntry(seqs[r], toks[r][fed[r]:fed[r] + n], [n - 1]) for r, n in step])
            for i, (r, n) in enumerate(step):
                fed[r] += n
                worst = max(worst, float((out[i].cpu() - ref[r][fed[r] - 1]).abs().max()))
        for s in seqs.values():
            engine.close(s)
        return worst

    sched = SchedulerConfig(num_kv_blocks=80, kv_block_size=8, max_batch_requests=4)
    engine = Engine.from_folder(folder, "float32", sched)
    assert engine.use_graphs and not engine.padding_safe
    assert run(engine) <= 2e-4
    assert engine.prompt_graph_replays == 0 and engine.graph_replays >= 10
    # the same with the mixer claiming that padding is harmless: the portions are padded, recorded and replayed,
    # the padding tokens advance the state, and the logits that follow are wrong
    monkeypatch.setattr(MIXERS.get("toy_decayed_sum_on_device"), "padding_safe", True)
    padded = Engine.from_folder(folder, "float32", sched)
    assert padded.padding_safe
    assert run(padded) > 1e-2
    assert padded.prompt_graph_replays > 0


# ---- a second toy architecture: routed feed-forward, another position encoding, a run order that is data ----
def _define_toy_routed():
    """A feed-forward that routes each token to one of its experts, a position encoding that rotates
    neighbouring pairs (2i, 2i+1), and an architecture whose run order names a layer twice and lets a
    layer read another layer's cache.  Everything is registered from here."""
    from dataclasses import dataclass
    from typing import Dict

    from zedinfer_amd import ops
    from zedinfer_amd.config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, ScheduleStep
    from zedinfer_amd.config.model_config import ModelConfig
    from zedinfer_amd.config.registry import register_architecture, registered_architectures
    from zedinfer_amd.parts import FeedForward, PositionEncoding, register_feed_forward, register_position_encoding
    from zedinfer_amd.weights.loader import WeightSpec

    if "ToyRoutedForCausalLM" in registered_architectures():
        return

    @register_feed_forward("toy_top1_experts")
    class Top1Experts(FeedForward):
        """y = p_e * expert_e(x) with e the most probable expert of softmax(x . Wr^T) (float32)."""

        @staticmethod
        def weight_specs(spec) -> Dict[str, WeightSpec]:
            H, I, E = (int(spec.params[k]) for k in ("hidden_size", "intermediate_size", "experts"))
            w = {"router": WeightSpec((E, H))}
            for e in range(E):
                w.update({f"gate{e}": WeightSpec((I, H)), f"up{e}": WeightSpec((I, H)), f"down{e}": WeightSpec((H, I))})
            return w

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.E = int(spec.params["experts"])
            self.w = weights

        def forward(self, x):
            logits = x.float() @ self.w["router"].float().t()
            prob = torch.softmax(logits, dim=-1)
            choice = prob.argmax(-1)
            out = torch.zeros(x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
            for e in range(self.E):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                xe = x[rows].contiguous()
                g, u = ops.linear(xe, self.w[f"gate{e}"]), ops.linear(xe, self.w[f"up{e}"])
                ye = ops.linear(ops.swiglu(g, u), self.w[f"down{e}"])
                out[rows] = ye.float() * prob[rows, e][:, None]
            return out.to(x.dtype)

    @register_position_encoding("toy_rope_pairs")
    class RopePairs(PositionEncoding):
        """Neighbouring pairs (2i, 2i+1) of every head turn by pos * theta^(-2i/d)."""

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            d = int(spec.params["head_dim"])
            i = torch.arange(d // 2, dtype=torch.float32, device=rt.device)
            self.inv = 1.0 / torch.pow(torch.tensor(float(spec.params["theta"]), device=rt.device), 2.0 * i / d)

        def turn(self, x, positions, heads, d):
            t = x.float().view(x.shape[0], heads, d // 2, 2)
            ang = positions.float()[:, None] * self.inv[None, :]
            c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
            a, b = t[..., 0], t[..., 1]
            return torch.stack([a * c - b * s, b * c + a * s], dim=-1).view(x.shape[0], heads * d).to(x.dtype)

        def encode(self, q, k, positions, nh, nkv, d):
            q.copy_(self.turn(q, positions, nh, d))
            k.copy_(self.turn(k, positions, nkv, d))

    @dataclass(frozen=True)
    class ToyRoutedConfig(ModelConfig):
        toy_experts: int = 3

        @classmethod
        def from_dict(cls, d):
            kw = cls._base_kwargs(d)
            kw["toy_experts"] = int(d["toy_experts"])
            cfg = cls(**kw)
            cfg.validate()
            return cfg

    def forward_config(cfg) -> ModelForwardConfig:
        H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        layers = []
        for L in range(cfg.num_hidden_layers):
            p = f"model.layers.{L}."
            mixer = PartSpec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "qkv_bias": L == 1, "window": 0,
                                           "position": PartSpec("toy_rope_pairs", {"head_dim": d, "theta": cfg.rope_theta})},
                             dict({"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                                   "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"},
                                  **({"q_bias": p + "self_attn.q_proj.bias", "k_bias": p + "self_attn.k_proj.bias",
                                      "v_bias": p + "self_attn.v_proj.bias"} if L == 1 else {})))
            if L == 0:
                ffn = PartSpec("toy_top1_experts", {"hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                                    "experts": cfg.toy_experts},
                               dict({"router": p + "moe.router.weight"},
                                    **{f"{n}{e}": p + f"moe.experts.{e}.{n}_proj.weight"
                                       for e in range(cfg.toy_experts) for n in ("gate", "up", "down")}))
            else:
                ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size},
                               {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                                "down": p + "mlp.down_proj.weight"})
            norms = {"input": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": p + "input_layernorm.weight"}),
                     "post_mixer": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps},
                                            {"weight": p + "post_attention_layernorm.weight"})}
            layers.append(LayerSpec("prenorm", mixer, ffn, norms))
        # layer 0 runs twice (the same weights, a cache each time); layer 2 attends over the keys and
        # values that layer 1 stored and stores none of its own
        schedule = (ScheduleStep(0, 0), ScheduleStep(1, 1), ScheduleStep(0, 2), ScheduleStep(2, 1, writes_cache=False))
        return ModelForwardConfig(
            architecture="ToyRoutedForCausalLM", hidden_size=H, vocab_size=cfg.vocab_size,
            embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "model.embed_tokens.weight"}),
            layers=tuple(layers), schedule=schedule,
            final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
            lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None},
                             {"weight": "lm_head.weight"}))

    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig, forward_config)


TOY_ROUTED = dict(architectures=["ToyRoutedForCausalLM"], model_type="toy_routed", hidden_size=64, intermediate_size=48,
                  vocab_size=257, max_position_embeddings=256, num_hidden_layers=3, num_attention_heads=4,
                  num_key_value_heads=2, head_dim=16, rope_theta=3000.0, rms_norm_eps=3e-6, toy_experts=3)


def toy_routed_plain_forward(cfg, w, ids):
    w = {k: v.float() for k, v in w.items()}
    T = len(ids)
    pos = torch.arange(T)
    eps, nh, nkv, d = cfg["rms_norm_eps"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]

    def pairs(x, heads):
        t = x.view(T, heads, d // 2, 2)
        inv = 1.0 / torch.pow(torch.tensor(cfg["rope_theta"]), 2.0 * torch.arange(d // 2, dtype=torch.float32) / d)
        ang = pos.float()[:, None] * inv[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = t[..., 0], t[..., 1]
        return torch.stack([a * c - b * s, b * c + a * s], dim=-1).view(T, heads, d)

    h = plain.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    stored = {}
    for layer, cache, writes in ((0, 0, True), (1, 1, True), (0, 2, True), (2, 1, False)):
        p = f"model.layers.{layer}."
        x = plain.rms_norm(h, w[p + "input_layernorm.weight"], eps)
        q = pairs(plain.linear(x, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias")), nh)
        if writes:
            k = pairs(plain.linear(x, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias")), nkv)
            v = plain.linear(x, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias")).view(T, nkv, d)
            stored[cache] = (k, v)
        k, v = stored[cache]
        a = plain.causal_gqa_attention(q, k, v, 1.0 / math.sqrt(d))
        h = h + plain.linear(a.reshape(T, nh * d), w[p + "self_attn.o_proj.weight"])
        x = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        if layer == 0:
            prob = torch.softmax(x @ w[p + "moe.router.weight"].t(), dim=-1)
            choice = prob.argmax(-1)
            y = torch.zeros_like(x)
            for t in range(T):
                e = int(choice[t])
                g = plain.linear(x[t:t + 1], w[p + f"moe.experts.{e}.gate_proj.weight"])
                u = plain.linear(x[t:t + 1], w[p + f"moe.experts.{e}.up_proj.weight"])
                y[t] = prob[t, e] * plain.linear(plain.swiglu(g, u), w[p + f"moe.experts.{e}.down_proj.weight"])[0]
            h = h + y
        else:
            h = h + plain.mlp_block(x, w, p)
    return plain.linear(plain.rms_norm(h, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16w"])
def test_toy_architecture_with_routing_pairs_rotation_and_a_shared_cache(tmp_path, dtype):
    """float32, and bfloat16 with a bfloat16 checkpoint: there the attention takes the few-rows products and
    their partial sums, the position encoding (which offers no table of angles) gets q and k once the attention
    has added the sums up, and the layer that reads another layer's cache stores nothing."""
    _define_toy_routed()
    from zedinfer_amd.config import SchedulerConfig, load_config
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.weights import write_model_folder
    folder = str(tmp_path / "toy_routed")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY_ROUTED, f)
    arch, cfg = load_config(folder)
    assert arch.name == "ToyRoutedForCausalLM"
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    write_model_folder(folder, cfg, expected_weights(arch.forward_config(cfg)), seed=11, dtype=stored, std=0.1,
                       noisy_norms=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY_ROUTED, f)
    pcfg, w = plain.load_folder(folder)
    requests = {f"t{i}": traces.random_tokens(TOY_ROUTED["vocab_size"], n, seed=70 + i) for i, n in enumerate([41, 64, 7, 55, 30])}
    ref = {rid: toy_routed_plain_forward(pcfg, w, toks) for rid, toks in requests.items()}
    engine = Engine.from_folder(folder, "float32" if dtype == "float32" else "bfloat16",
                                SchedulerConfig(num_kv_blocks=32, kv_block_size=8, max_batch_requests=4))
    assert len(engine.cache.tensors) == 3          # four runs of layers, three caches
    for make in (traces.whole, traces.last_decoded, traces.mixed):
        steps = make(requests)
        out = traces.run_in_process(engine, steps)
        worst, mean, scale, rows, where = traces.compare(steps, out, ref, requests)
        assert rows == sum(len(t) for t in requests.values())
        if dtype == "float32":
            assert worst <= 3e-4 * max(1.0, scale), where
        else:
            # a token whose two best experts are nearly as probable may go to the other one in bfloat16:
            # the mean stays small, single rows may not
            assert mean <= 0.02 * scale, (mean, scale, where)


# ---- a third toy architecture: a position encoding with two axes ----------------------------------
def _define_toy_two_axes():
    """A position encoding that reads two positions per token (as an encoding of image patches reads a
    row and a column): the first half of every head's pairs turns by the position on axis 0, the second
    half by the position on axis 1.  Registered from here; the step's entries may bring positions of
    their own."""
    from zedinfer_amd import ops
    from zedinfer_amd.config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, default_schedule
    from zedinfer_amd.config.model_config import ModelConfig
    from zedinfer_amd.config.registry import register_architecture, registered_architectures
    from zedinfer_amd.parts import PositionEncoding, register_position_encoding

    if "ToyTwoAxesForCausalLM" in registered_architectures():
        return

    @register_position_encoding("toy_rope_two_axes")
    class RopeTwoAxes(PositionEncoding):
        position_axes = 2
        graph_safe = True       # launches over device arrays only

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            d = int(spec.params["head_dim"])
            k = torch.arange(d // 2, dtype=torch.float32, device=rt.device)
            self.inv = 1.0 / torch.pow(torch.tensor(float(spec.params["theta"]), device=rt.device), 2.0 * k / d)

        def turn(self, x, positions, heads, d):
            assert positions.shape == (x.shape[0], 2)
            half = d // 2
            axis = (torch.arange(half, device=x.device) >= half // 2).long()          # pair -> axis
            ang = positions.float()[:, axis] * self.inv[None, :]                       # [n, d/2]
            c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
            t = x.float().view(x.shape[0], heads, d)
            a, b = t[..., :half], t[..., half:]
            return torch.cat([a * c - b * s, b * c + a * s], dim=-1).view(x.shape[0], heads * d).to(x.dtype)

        def encode(self, q, k, positions, nh, nkv, d):
            q.copy_(self.turn(q, positions, nh, d))
            k.copy_(self.turn(k, positions, nkv, d))

    def forward_config(cfg) -> ModelForwardConfig:
        H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        layers = []
        for L in range(cfg.num_hidden_layers):
            p = f"model.layers.{L}."
            mixer = PartSpec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "qkv_bias": False, "window": 0,
                                           "position": PartSpec("toy_rope_two_axes", {"head_dim": d, "theta": cfg.rope_theta})},
                             {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                              "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"})
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size},
                           {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                            "down": p + "mlp.down_proj.weight"})
            norms = {"input": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": p + "input_layernorm.weight"}),
                     "post_mixer": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps},
                                            {"weight": p + "post_attention_layernorm.weight"})}
            layers.append(LayerSpec("prenorm", mixer, ffn, norms))
        return ModelForwardConfig(
            architecture="ToyTwoAxesForCausalLM", hidden_size=H, vocab_size=cfg.vocab_size,
            embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "model.embed_tokens.weight"}),
            layers=tuple(layers), schedule=default_schedule(cfg.num_hidden_layers),
            final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
            lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None},
                             {"weight": "lm_head.weight"}))

    register_architecture("ToyTwoAxesForCausalLM", ModelConfig, forward_config)


TOY_TWO_AXES = dict(architectures=["ToyTwoAxesForCausalLM"], model_type="toy_two_axes", hidden_size=40, intermediate_size=56,
                    vocab_size=211, max_position_embeddings=256, num_hidden_layers=2, num_attention_heads=2,
                    num_key_value_heads=1, head_dim=24, rope_theta=100.0, rms_norm_eps=1e-6)


def toy_two_axes_plain_forward(cfg, w, ids, pos2):
    """``pos2`` [T, 2]: the position of every token on both axes."""
    w = {k: v.float() for k, v in w.items()}
    T = len(ids)
    eps, nh, nkv, d = cfg["rms_norm_eps"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    half = d // 2
    inv = 1.0 / torch.pow(torch.tensor(cfg["rope_theta"]), 2.0 * torch.arange(half, dtype=torch.float32) / d)
    ang = torch.cat([pos2[:, :1].float().expand(T, half // 2), pos2[:, 1:].float().expand(T, half - half // 2)], 1) * inv

    def turn(x, heads):
        t = x.view(T, heads, d)
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = t[..., :half], t[..., half:]
        return torch.cat([a * c - b * s, b * c + a * s], dim=-1)

    h = plain.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for L in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{L}."
        x = plain.rms_norm(h, w[p + "input_layernorm.weight"], eps)
        q = turn(plain.linear(x, w[p + "self_attn.q_proj.weight"]), nh)
        k = turn(plain.linear(x, w[p + "self_attn.k_proj.weight"]), nkv)
        v = plain.linear(x, w[p + "self_attn.v_proj.weight"]).view(T, nkv, d)
        a = plain.causal_gqa_attention(q, k, v, 1.0 / math.sqrt(d))
        h = h + plain.linear(a.reshape(T, nh * d), w[p + "self_attn.o_proj.weight"])
        x = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + plain.mlp_block(x, w, p)
    return plain.linear(plain.rms_norm(h, w["model.norm.weight"], eps), w["lm_head.weight"])


def test_toy_architecture_with_positions_on_two_axes(tmp_path):
    """The step carries positions on as many axes as the model's position encodings read.  Entries that
    bring none get their tokens' indices on every axis; entries may bring their own (here: a grid whose
    rows are 7 wide, so that axis 1 runs 0..6 again and again while the cache index goes on counting).
    Prompt portions, single tokens (replayed as graphs when they bring no positions) and both mixed."""
    _define_toy_two_axes()
    from zedinfer_amd.config import SchedulerConfig, load_config
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.weights import write_model_folder
    folder = str(tmp_path / "toy_two_axes")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY_TWO_AXES, f)
    arch, cfg = load_config(folder)
    write_model_folder(folder, cfg, expected_weights(arch.forward_config(cfg)), seed=3, dtype=torch.float32, std=0.15,
                       noisy_norms=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY_TWO_AXES, f)
    pcfg, w = plain.load_folder(folder)
    T = 90
    toks = {r: traces.random_tokens(TOY_TWO_AXES["vocab_size"], T, seed=20 + i) for i, r in enumerate("gs")}
    idx = torch.arange(T)
    grid = torch.stack([idx // 7, idx % 7], dim=1)                  # request "g": rows and columns of a grid
    seqn = torch.stack([idx, idx], dim=1)                           # request "s": brings no positions
    ref = {"g": toy_two_axes_plain_forward(pcfg, w, toks["g"], grid),
           "s": toy_two_axes_plain_forward(pcfg, w, toks["s"], seqn)}
    assert float((ref["g"] - toy_two_axes_plain_forward(pcfg, w, toks["g"], seqn)).abs().max()) > 0.05   # the axes matter
    engine = Engine.from_folder(folder, "float32", SchedulerConfig(num_kv_blocks=40, kv_block_size=8, max_batch_requests=4))
    assert engine.position_axes == 2
    seqs = {r: engine.open(r) for r in toks}
    fed = {r: 0 for r in toks}
    worst = 0.0
    plan = [[("g", 20)], [("s", 33), ("g", 9)], [("g", 1), ("s", 1)], [("g", 17), ("s", 1)]] + [[("s", 1), ("g", 1)]] * 8 \
        + [[("s", 1)]] * 12 + [[("g", 30)], [("s", 20), ("g", 5)]]
    for step in plan:
        entries = []
        for r, n in step:
            pos = grid[fed[r]:fed[r] + n].tolist() if r == "g" else None
            entries.append(StepEntry(seqs[r], toks[r][fed[r]:fed[r] + n], list(range(n)), positions=pos))
        out = engine.step(entries).cpu()
        row = 0
        for r, n in step:
            worst = max(worst, float((out[row:row + n] - ref[r][fed[r]:fed[r] + n]).abs().max()))
            fed[r], row = fed[r] + n, row + n
    assert worst <= 2e-4, worst
    with pytest.raises(ValueError, match="positions"):
        engine.step([StepEntry(seqs["g"], [5, 6], [0], positions=[[0, 0]])])
