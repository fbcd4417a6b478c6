"""Typed configuration and the architecture registry (CPU)."""
import json

import pytest

import tiny_configs
from zedinfer_amd.config import (ConfigError, Qwen2Config, ScheduleStep, SchedulerConfig, find_architecture,
                                 load_config, registered_architectures)
from zedinfer_amd.models import expected_weights
from zedinfer_amd.models.qwen2 import qwen2_forward_config


def test_defaults_follow_the_reference():
    # reference: src/frontend/models/base.cpp:683-720 and :807-813
    cfg = Qwen2Config.from_dict(dict(hidden_size=64, intermediate_size=128, vocab_size=100,
                                     max_position_embeddings=32, num_hidden_layers=1, num_attention_heads=4))
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 10000.0 and cfg.tie_word_embeddings is False
    assert cfg.eos_token_ids == (151643,) and cfg.bos_token_id == 151643 and cfg.torch_dtype == "bfloat16"
    assert (cfg.sliding_window, cfg.max_window_layers, cfg.use_sliding_window) == (4096, 21, False)


def test_eos_array_and_explicit_head_dim():
    # reference: tests/models/test_model_config.cpp:153-227 (eos_token_id as an array)
    cfg = Qwen2Config.from_dict(tiny_configs.TINY_B)
    assert cfg.eos_token_ids == (998, 999) and cfg.eos_token_id == 998
    assert cfg.head_dim == 32
    c = Qwen2Config.from_dict(tiny_configs.TINY_C)
    assert c.head_dim == 48 and c.head_dim != c.hidden_size // c.num_attention_heads


def test_missing_and_bad_keys():
    d = dict(tiny_configs.TINY_A)
    del d["vocab_size"], d["hidden_size"]
    with pytest.raises(ConfigError, match="hidden_size, vocab_size"):
        Qwen2Config.from_dict(d)
    with pytest.raises(ConfigError, match="multiple"):
        Qwen2Config.from_dict(dict(tiny_configs.TINY_A, num_key_value_heads=3))
    with pytest.raises(ConfigError, match="rms_norm_eps"):
        Qwen2Config.from_dict(dict(tiny_configs.TINY_A, rms_norm_eps=0.0))


def test_another_activation_is_refused_and_rope_scaling_is_said(capsys):
    # the reference reads hidden_act and computes SiLU whatever it says (base.cpp:686,
    # transformer_forward.cpp:128-137); rope_scaling is not among the keys it parses (base.cpp:683-720)
    with pytest.raises(ConfigError, match="hidden_act 'gelu'"):
        Qwen2Config.from_dict(dict(tiny_configs.TINY_A, hidden_act="gelu"))
    assert Qwen2Config.from_dict(dict(tiny_configs.TINY_A, hidden_act="silu")).hidden_act == "silu"
    capsys.readouterr()
    Qwen2Config.from_dict(dict(tiny_configs.TINY_A))
    assert "rope_scaling" not in capsys.readouterr().err
    cfg = Qwen2Config.from_dict(dict(tiny_configs.TINY_A, rope_scaling={"type": "yarn", "factor": 4.0}))
    said = capsys.readouterr().err
    assert "rope_scaling" in said and "ignored" in said
    assert cfg.rope_theta == Qwen2Config.from_dict(dict(tiny_configs.TINY_A)).rope_theta


def test_registry(tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    assert find_architecture({"architectures": ["Qwen2ForCausalLM"]}).name == "Qwen2ForCausalLM"
    assert find_architecture({"model_type": "qwen2"}).name == "Qwen2ForCausalLM"
    with pytest.raises(ConfigError, match="registered: .*Qwen2ForCausalLM"):
        find_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    (tmp_path / "config.json").write_text(json.dumps(tiny_configs.TINY_A))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "Qwen2ForCausalLM" and isinstance(cfg, Qwen2Config) and cfg.intermediate_size == 176


def test_forward_config_is_built_from_config_alone():
    for name, d in tiny_configs.CONFIGS.items():
        cfg = Qwen2Config.from_dict(d)
        fc = qwen2_forward_config(cfg)
        assert len(fc.layers) == cfg.num_hidden_layers and len(fc.schedule) == cfg.num_hidden_layers
        m = fc.layers[0].mixer.params
        assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == \
            (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim)
        assert m["position"].params["theta"] == cfg.rope_theta
        assert fc.layers[0].norms["input"].params["eps"] == cfg.rms_norm_eps
        exp = expected_weights(fc)
        assert exp["model.layers.0.self_attn.q_proj.weight"].shape == (cfg.num_attention_heads * cfg.head_dim,
                                                                       cfg.hidden_size)
        assert exp["model.layers.0.mlp.down_proj.weight"].shape == (cfg.hidden_size, cfg.intermediate_size)
        assert (exp["lm_head.weight"].fallback is not None) == cfg.tie_word_embeddings
    # the window is chosen layer by layer
    fc = qwen2_forward_config(Qwen2Config.from_dict(tiny_configs.TINY_C))
    assert [l.mixer.params["window"] for l in fc.layers] == [0, 20, 20]


def test_window_keys_can_be_ignored_as_the_reference_does(monkeypatch):
    """The reference parses the window keys and never uses them (src/frontend/models/base.cpp:807-813)."""
    monkeypatch.setenv("ZEDINFER_IGNORE_SLIDING_WINDOW", "1")
    fc = qwen2_forward_config(Qwen2Config.from_dict(tiny_configs.TINY_C))
    assert [l.mixer.params["window"] for l in fc.layers] == [0, 0, 0]


def test_schedule_validation():
    import dataclasses
    fc = qwen2_forward_config(Qwen2Config.from_dict(tiny_configs.TINY_A))
    ok = dataclasses.replace(fc, schedule=(ScheduleStep(0, 0), ScheduleStep(1, 1), ScheduleStep(0, 2),
                                           ScheduleStep(1, 1, writes_cache=False)))
    ok.validate()
    with pytest.raises(ValueError, match="both write"):
        dataclasses.replace(fc, schedule=(ScheduleStep(0, 0), ScheduleStep(1, 0))).validate()
    with pytest.raises(ValueError, match="no earlier step writes"):
        dataclasses.replace(fc, schedule=(ScheduleStep(0, 1, writes_cache=False), ScheduleStep(1, 1))).validate()
    with pytest.raises(ValueError, match="names layer"):
        dataclasses.replace(fc, schedule=(ScheduleStep(5, 0),)).validate()


def test_scheduler_config_defaults():
    # reference: include/zedinfer/scheduler.hpp:42-60
    s = SchedulerConfig()
    assert (s.max_batch_tokens, s.max_batch_requests, s.max_prefill_tokens, s.max_queue_size, s.kv_block_size) == \
        (2048, 64, 512, 256, 16)
    assert s.gpu_memory_utilization == pytest.approx(0.9)
    with pytest.raises(ValueError):
        SchedulerConfig(kv_block_size=0).validate()


def test_workspaces_that_are_outgrown_stay_alive():
    """A graph captured with a workspace goes on using it after a larger step has outgrown it: the old
    allocation must keep its address and its contents, and views of a shape come back as they were."""
    import torch
    from zedinfer_amd.parts import Runtime
    rt = Runtime("cpu", torch.float32)
    small = rt.buffer("x", (4,))
    small.fill_(3.0)
    assert rt.buffer("x", (4,)) is small and rt.outgrown_bytes() == 0
    ptr = small.data_ptr()
    large = rt.buffer("x", (400,))
    large.fill_(7.0)
    other = [torch.full((4,), 9.0) for _ in range(64)]      # allocations that could take freed memory
    assert small.data_ptr() == ptr and bool((small == 3.0).all()) and rt.outgrown_bytes() == 16
    assert rt.buffer("x", (4,)).data_ptr() == large.data_ptr()    # new steps use the new allocation
    grown = rt.buffer("x", (401,))
    assert grown.data_ptr() != large.data_ptr() and rt._buffers[("x", torch.float32)].numel() >= 600
    del other
