"""The safetensors reader/writer, weight binding and its single error, random weights (CPU)."""
import json
import os
import struct

import pytest
import torch

import tiny_configs
from zedinfer_amd.config import Qwen2Config
from zedinfer_amd.models import expected_weights
from zedinfer_amd.models.qwen2 import qwen2_forward_config
from zedinfer_amd.weights import (SafetensorsError, SafetensorsFolder, WeightError, load_weights, random_weights,
                                  storage_dtype, write_model_folder, write_safetensors)


def expected(name):
    return expected_weights(qwen2_forward_config(Qwen2Config.from_dict(tiny_configs.CONFIGS[name])))


def test_round_trip_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
         "d": torch.randn(2, 2).to(torch.float16)}
    write_safetensors(str(tmp_path / "x.safetensors"), t)
    back = load_file(str(tmp_path / "x.safetensors"))
    assert set(back) == set(t) and all(torch.equal(back[k], t[k]) for k in t)
    save_file(t, str(tmp_path / "y.safetensors"))
    f = SafetensorsFolder(str(tmp_path))
    assert all(torch.equal(f.tensor(k), t[k]) for k in t)
    f.close()


def test_container_errors(tmp_path):
    with pytest.raises(SafetensorsError, match="does not exist"):
        SafetensorsFolder(str(tmp_path / "nope"))
    with pytest.raises(SafetensorsError, match="no .safetensors"):
        SafetensorsFolder(str(tmp_path))
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    (tmp_path / "short.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="past the data section"):
        SafetensorsFolder(str(tmp_path))
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    (tmp_path / "short.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 16)
    with pytest.raises(SafetensorsError, match="needs 16"):
        SafetensorsFolder(str(tmp_path))
    hdr = json.dumps({"w": {"dtype": "Q4", "shape": [4], "data_offsets": [0, 2]}}).encode()
    (tmp_path / "short.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 2)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFolder(str(tmp_path))


def test_later_shard_wins(tmp_path):
    write_safetensors(str(tmp_path / "model-00001.safetensors"), {"w": torch.zeros(2), "x": torch.ones(1)})
    write_safetensors(str(tmp_path / "model-00002.safetensors"), {"w": torch.full((2,), 5.0)})
    f = SafetensorsFolder(str(tmp_path))
    assert f.tensor("w").tolist() == [5.0, 5.0] and f.tensor("x").tolist() == [1.0]
    f.close()


def test_one_error_lists_everything(tmp_path):
    exp = expected("B")
    w = random_weights(exp, 0, torch.float32)
    del w["model.layers.1.mlp.up_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(7)
    w["model.layers.2.mlp.down_proj.weight"] = torch.zeros(256, 96)
    w["model.layers.9.extra.weight"] = torch.zeros(1)
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    with pytest.raises(WeightError) as ei:
        load_weights(str(tmp_path), exp, torch.float32, "cpu")
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["layers.9.extra.weight"]
    assert len(e.wrong_shape) == 2 and "k_proj.bias: expected [32], file has [7]" in e.wrong_shape[0]
    msg = str(e)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "up_proj", "extra", "[256, 96]"):
        assert piece in msg


def test_tied_head(tmp_path):
    exp = expected("A")                       # tie_word_embeddings=true
    folder = tiny_configs.write_tiny(str(tmp_path / "a"), "A")
    names = SafetensorsFolder(folder).names()
    assert "lm_head.weight" not in names      # a tied head is not written
    w = load_weights(folder, exp, torch.float32, "cpu")
    assert w["lm_head.weight"].data_ptr() == w["model.embed_tokens.weight"].data_ptr()
    # a file that does hold lm_head.weight wins over the tie (reference: base.cpp:410-416)
    full = dict(w)
    full["lm_head.weight"] = torch.randn(512, 64)
    os.makedirs(tmp_path / "b")
    write_safetensors(str(tmp_path / "b" / "model.safetensors"), full)
    w2 = load_weights(str(tmp_path / "b"), exp, torch.float32, "cpu")
    assert torch.equal(w2["lm_head.weight"], full["lm_head.weight"])
    # untied and absent: missing
    expB = expected("B")
    wb = random_weights(expB, 0, torch.float32)
    del wb["lm_head.weight"]
    os.makedirs(tmp_path / "c")
    write_safetensors(str(tmp_path / "c" / "model.safetensors"), wb)
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(str(tmp_path / "c"), expB, torch.float32, "cpu")


def test_storage_types(tmp_path):
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert storage_dtype(bf, "float", bf) == bf and storage_dtype(f16, "float", bf) == bf
    assert storage_dtype(f32, "float", bf) == f32          # a tensor stored in 32-bit stays so
    assert storage_dtype(bf, "float", f32) == f32 and storage_dtype(f16, "float", f32) == f32
    assert storage_dtype(torch.int64, "int", bf) == torch.int32
    exp = expected("A")
    w = random_weights(exp, 3, bf)
    w = {k: v for k, v in w.items() if k != "lm_head.weight"}
    w["model.norm.weight"] = w["model.norm.weight"].float()
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    got = load_weights(str(tmp_path), exp, bf, "cpu")
    assert got["model.norm.weight"].dtype == f32 and got["model.embed_tokens.weight"].dtype == bf
    got32 = load_weights(str(tmp_path), exp, f32, "cpu")
    assert all(t.dtype == f32 for t in got32.values())
    assert torch.equal(got32["model.embed_tokens.weight"], w["model.embed_tokens.weight"].float())


def test_names_without_the_model_prefix(tmp_path):
    exp = expected("A")
    w = {k[len("model."):] if k.startswith("model.") else k: v
         for k, v in random_weights(exp, 0, torch.float32).items() if k != "lm_head.weight"}
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    got = load_weights(str(tmp_path), exp, torch.float32, "cpu")
    assert set(got) == set(exp)


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    exp = expected("B")
    a = random_weights(exp, 7, torch.float32)
    b = random_weights(dict(reversed(list(exp.items()))), 7, torch.float32)
    assert all(torch.equal(a[k], b[k]) for k in exp)
    c = random_weights(exp, 8, torch.float32)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    assert torch.equal(a["model.norm.weight"], torch.ones(96))
    n = random_weights(exp, 7, torch.float32, noisy_norms=True)["model.norm.weight"]
    assert 0.0 < float((n - 1).abs().mean()) < 0.05
    assert abs(float(a["model.layers.0.mlp.up_proj.weight"].std()) - 0.02) < 0.002
    cfg = Qwen2Config.from_dict(tiny_configs.TINY_B)
    folder = write_model_folder(str(tmp_path / "m"), cfg, exp, 7)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    again = load_weights(folder, exp, torch.float32, "cpu")
    assert torch.equal(again["model.layers.2.self_attn.v_proj.bias"],
                       a["model.layers.2.self_attn.v_proj.bias"].to(torch.bfloat16).float())
    assert json.load(open(os.path.join(folder, "config.json")))["intermediate_size"] == 256
