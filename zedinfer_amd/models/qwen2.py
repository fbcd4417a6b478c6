"""Qwen2 dense (``Qwen2ForCausalLM``): the description of the model in parts.

Pre-norm decoder blocks of grouped-query attention with q/k/v biases and
split-half rotary encoding, a SwiGLU feed-forward, RMSNorm, an untied or tied
output head (reference: include/frontend/models/qwen2.hpp:17-42 sets
has_qkv_bias=true, has_qk_norm=false; the forward is
src/frontend/models/transformer_forward.cpp:18-160; tensor names from
src/frontend/models/forward_config.hpp:176-192 with the ``model.`` prefix the
checkpoint carries, src/frontend/models/base.cpp:1386-1410).

Sliding window.  The reference parses ``use_sliding_window``, ``sliding_window``
and ``max_window_layers`` and never reads them (reference: base.cpp:807-813):
it attends over all keys in every layer whatever they say.  Here they select
the mixer per layer, by the meaning the keys have in the Qwen2 configuration
format ("max_window_layers: the first that many layers use full attention, the
layers after them the sliding window"): with ``use_sliding_window`` the layers
from ``max_window_layers`` on see only the last ``sliding_window`` keys.  So for
a configuration with ``use_sliding_window: true`` this engine's logits differ
from the reference's as soon as a sequence is longer than the window; no file of
the reference pins the windowed case.  ``ZEDINFER_IGNORE_SLIDING_WINDOW=1`` in
the environment makes every layer attend over all keys, as the reference does.
All configurations of the benchmarks say ``use_sliding_window: false``.
"""
from __future__ import annotations

import os

from ..config.forward_config import (LayerSpec, ModelForwardConfig, PartSpec, default_schedule)
from ..config.model_config import Qwen2Config
from ..config.registry import register_architecture


def layer_window(cfg: Qwen2Config, layer: int) -> int:
    """Keys layer ``layer`` sees (0: all of them)."""
    if os.environ.get("ZEDINFER_IGNORE_SLIDING_WINDOW", "0") not in ("", "0"):
        return 0        # the reference's behaviour: the window keys are parsed and not used
    if cfg.use_sliding_window and layer >= cfg.max_window_layers:
        return cfg.sliding_window
    return 0


def qwen2_forward_config(cfg: Qwen2Config) -> ModelForwardConfig:
    H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layers = []
    for L in range(cfg.num_hidden_layers):
        p = f"model.layers.{L}."
        position = PartSpec("rope_neox", {"head_dim": d, "theta": cfg.rope_theta, "rotary_dim": d})
        mixer = PartSpec(
            "attention",
            {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "qkv_bias": True,
             "window": layer_window(cfg, L), "position": position},
            {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
             "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight",
             "q_bias": p + "self_attn.q_proj.bias", "k_bias": p + "self_attn.k_proj.bias",
             "v_bias": p + "self_attn.v_proj.bias"})
        ffn = PartSpec(
            "swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size},
            {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
             "down": p + "mlp.down_proj.weight"})
        norms = {
            "input": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps},
                              {"weight": p + "input_layernorm.weight"}),
            "post_mixer": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps},
                                   {"weight": p + "post_attention_layernorm.weight"}),
        }
        layers.append(LayerSpec("prenorm", mixer, ffn, norms))
    fc = ModelForwardConfig(
        architecture="Qwen2ForCausalLM",
        hidden_size=H,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H},
                           {"weight": "model.embed_tokens.weight"}),
        layers=tuple(layers),
        schedule=default_schedule(cfg.num_hidden_layers),
        final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
        lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H,
                                    "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None},
                         {"weight": "lm_head.weight"}),
        tie_word_embeddings=cfg.tie_word_embeddings,
        eos_token_ids=cfg.eos_token_ids,
        max_position_embeddings=cfg.max_position_embeddings,
        family={"qkv_bias": True, "qk_norm": False, "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
                "use_sliding_window": cfg.use_sliding_window, "sliding_window": cfg.sliding_window,
                "max_window_layers": cfg.max_window_layers},
    )
    fc.validate()
    return fc


register_architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_forward_config, aliases=("qwen2",))
