"""A toy mixer that keeps ONE tensor of its own making in every page of the cache (a short latent per token,
float32, no keys and no values), defined, registered, built and stepped from here: the cache manager allocates
what the mixer's request names and hands it over by name, the engine grows and frees the pages as for any other
layer, and nothing under the framework's folders knows what the pages hold.  The architecture alternates it with
attention, whose pages (keys, values) live beside the latents under the same page ids."""
import json
import math
import os

import pytest
import torch

import traces
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


def _define():
    from typing import Dict, Optional

    from zedinfer_amd.config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, default_schedule
    from zedinfer_amd.config.model_config import ModelConfig
    from zedinfer_amd.config.registry import register_architecture, registered_architectures
    from zedinfer_amd.parts import PAGE, KVCacheRequest, Mixer, PageTensor, register_mixer
    from zedinfer_amd.weights.loader import WeightSpec

    if "ToyLatentForCausalLM" in registered_architectures():
        return

    @register_mixer("toy_latent_attention")
    class LatentAttention(Mixer):
        """c_t = Wc x_t (r values, kept in the cache); y_t = Wo sum_s softmax_s(q_t . c_s / sqrt(r)) c_s over
        s <= t, with q_t = Wq x_t."""

        @staticmethod
        def weight_specs(spec) -> Dict[str, WeightSpec]:
            H, r = int(spec.params["hidden_size"]), int(spec.params["latent_size"])
            return {"wc": WeightSpec((r, H)), "wq": WeightSpec((r, H)), "wo": WeightSpec((H, r))}

        def __init__(self, spec, weights, rt):
            super().__init__(spec, weights, rt)
            self.r = int(spec.params["latent_size"])
            self.wc, self.wq, self.wo = (weights[k].float() for k in ("wc", "wq", "wo"))

        def cache_request(self) -> Optional[KVCacheRequest]:
            return KVCacheRequest("full", 0, (("latent", PageTensor((PAGE, self.r), torch.float32)),))

        def forward(self, x, batch, memory):
            view = batch.groups[memory.group]
            pages = memory.tensors["latent"]                     # [pages, page size, r]
            ps = pages.shape[1]
            c, q = x.float() @ self.wc.t(), x.float() @ self.wq.t()
            pages.view(-1, self.r)[view.slots.long()] = c        # the step's own latents, where the engine says
            out = torch.empty_like(c)
            for e, (start, n, past) in enumerate(zip(batch.host_start, batch.host_len, batch.host_past)):
                start, n, past = int(start), int(n), int(past)
                table = view.block_tables[e, :-(-(past + n) // ps)].long()
                seen = pages[table].reshape(-1, self.r)[:past + n]                      # [past + n, r]
                s = q[start:start + n] @ seen.t() / math.sqrt(self.r)
                later = torch.arange(past + n, device=x.device)[None, :] > (past + torch.arange(n, device=x.device))[:, None]
                out[start:start + n] = torch.softmax(s.masked_fill(later, float("-inf")), dim=-1) @ seen
            return (out @ self.wo.t()).to(x.dtype)

    def forward_config(cfg) -> ModelForwardConfig:
        H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        layers = []
        for L in range(cfg.num_hidden_layers):
            p = f"model.layers.{L}."
            if L % 2 == 0:
                mixer = PartSpec("toy_latent_attention", {"hidden_size": H, "latent_size": LATENT},
                                 {"wc": p + "toy.wc.weight", "wq": p + "toy.wq.weight", "wo": p + "toy.wo.weight"})
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
            architecture="ToyLatentForCausalLM", hidden_size=H, vocab_size=cfg.vocab_size,
            embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "model.embed_tokens.weight"}),
            layers=tuple(layers), schedule=default_schedule(cfg.num_hidden_layers),
            final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
            lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None},
                             {"weight": "lm_head.weight"}))

    register_architecture("ToyLatentForCausalLM", ModelConfig, forward_config)


LATENT = 12
TOY = dict(architectures=["ToyLatentForCausalLM"], model_type="toy_latent", hidden_size=40, intermediate_size=72,
           vocab_size=257, max_position_embeddings=256, num_hidden_layers=3, num_attention_heads=2,
           num_key_value_heads=1, head_dim=16, rope_theta=7000.0, rms_norm_eps=3e-6)


def plain_forward(cfg, w, ids):
    """Whole sequence, no cache."""
    T = len(ids)
    pos = torch.arange(T)
    eps = cfg["rms_norm_eps"]
    h = plain.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for L in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{L}."
        x = plain.rms_norm(h, w[p + "input_layernorm.weight"], eps)
        if L % 2 == 0:
            c, q = x @ w[p + "toy.wc.weight"].t(), x @ w[p + "toy.wq.weight"].t()
            s = (q @ c.t() / math.sqrt(LATENT)).masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
            h = h + (torch.softmax(s, dim=-1) @ c) @ w[p + "toy.wo.weight"].t()
        else:
            h = h + plain.attention_block(x, w, p, cfg, pos, None)
        x = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + plain.mlp_block(x, w, p)
    return plain.linear(plain.rms_norm(h, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_a_page_tensor_of_its_own(tmp_path, dtype):
    _define()
    from zedinfer_amd.config import SchedulerConfig, load_config
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.weights import write_model_folder
    folder = str(tmp_path / "toy_latent")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY, f)
    arch, cfg = load_config(folder)
    assert arch.name == "ToyLatentForCausalLM"
    write_model_folder(folder, cfg, expected_weights(arch.forward_config(cfg)), seed=9, dtype=torch.float32, std=0.1,
                       noisy_norms=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TOY, f)
    pcfg, w = plain.load_folder(folder)
    requests = {f"t{i}": traces.random_tokens(TOY["vocab_size"], n, seed=90 + i) for i, n in enumerate([37, 64, 9, 50, 23])}
    ref = {rid: plain_forward(pcfg, w, toks) for rid, toks in requests.items()}
    ps, pages = 8, 26            # so few pages that the mixed trace uses them again
    engine = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=pages, kv_block_size=ps, max_batch_requests=4))
    # what the manager allocated: for the latent layers one float32 tensor [pages, page, r] each, whatever the engine's
    # type; for the attention layer its keys and values; all under one group's page ids
    assert len(engine.cache.groups) == 1 and sorted(engine.cache.groups[0].caches) == [0, 1, 2]
    shapes = {cid: {name: (tuple(t.shape), t.dtype) for name, t in ts.items()} for cid, ts in engine.cache.tensors.items()}
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    assert shapes[0] == shapes[2] == {"latent": ((pages, ps, LATENT), torch.float32)}
    assert shapes[1] == {"k": ((pages, 1, ps, 16), act), "v": ((pages, 1, 16, ps), act)}
    assert engine.cache.bytes_per_page(engine.model.cache_requests(), ps, act) == \
        2 * ps * LATENT * 4 + 2 * ps * 16 * (4 if dtype == "float32" else 2)
    for make in (traces.whole, traces.portions, traces.mixed):
        steps = make(requests)
        out = traces.run_in_process(engine, steps)
        worst, mean, scale, rows, where = traces.compare(steps, out, ref, requests)
        assert rows == sum(len(t) for t in requests.values())
        if dtype == "float32":
            assert worst <= 2e-4 * max(1.0, scale), where
        else:
            assert worst <= 0.08 * scale and mean <= 0.015 * scale, where
    engine.cache.check()
    assert not engine.cache.live and engine.cache.groups[0].pool.takes > pages       # pages were used again
