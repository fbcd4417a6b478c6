"""Seeded random tiny configurations through the engine against the plain implementation: the sizes and
options that the three fixed configurations do not hold (head sizes 16..256, groups of 1..32 query heads,
widths and vocabularies that are multiples of nothing, windows shorter than a page, one to four layers),
with float32 and bfloat16 checkpoints (the latter with weights wide enough that attention is peaked and a
wrong rotation or scale shows in bfloat16 too: tests/test_tolerances.py), in both engine precisions, whole / decoded / in portions / mixed
with pages used again.  Whatever a kernel does not take must go to one that does: never a wrong result."""
import json
import os
import random

import pytest
import torch

import traces
from plain import qwen2_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL, sharp_std

pytestmark = pytest.mark.gpu


def usual(rng):
    d = rng.choice([16, 16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 1, 2, 2, 3, 4])
    G = rng.choice([1, 1, 2, 3, 4, 5, 6, 7, 8, 16])
    if nkv * G * d > 1024:
        G = max(1, 1024 // (nkv * d))
    hidden = rng.choice([32, 40, 48, 56, 72, 88, 96, 104, 136, 200, 264])
    L = rng.choice([1, 2, 2, 3, 4])
    c = dict(hidden_size=hidden, intermediate_size=rng.choice([24, 40, 88, 104, 176, 200, 344]),
             vocab_size=rng.choice([50, 257, 512, 1000, 1031, 2049]), num_hidden_layers=L,
             num_attention_heads=nkv * G, num_key_value_heads=nkv, head_dim=d,
             rope_theta=rng.choice([1e4, 5e4, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]))
    if rng.random() < 0.5:
        c.update(use_sliding_window=True, sliding_window=rng.choice([4, 9, 16, 20, 33, 64, 100]),
                 max_window_layers=rng.randrange(0, L + 1))
    return c


def unusual(rng):
    d = rng.choice([16, 48, 144, 160, 256])
    nkv = rng.choice([1, 2, 3])
    G = rng.choice([1, 3, 17, 20, 32]) if d <= 48 else rng.choice([1, 2, 3])
    c = dict(hidden_size=rng.choice([33, 36, 44, 90, 97, 100, 202]), intermediate_size=rng.choice([50, 77, 99, 130]),
             vocab_size=rng.choice([33, 101, 1025]), num_hidden_layers=rng.choice([1, 2]),
             num_attention_heads=nkv * G, num_key_value_heads=nkv, head_dim=d, rope_theta=1e4, rms_norm_eps=1e-6)
    if rng.random() < 0.4:
        c.update(use_sliding_window=True, sliding_window=rng.choice([3, 17, 50]), max_window_layers=0)
    return c


def odd_heads(rng):
    """Head sizes that are multiples of 2 only: no matrix-core kernel takes them, the plain ones must."""
    d = rng.choice([6, 10, 22, 30])
    nkv = rng.choice([1, 2])
    G = rng.choice([1, 2, 5])
    c = dict(hidden_size=rng.choice([40, 64, 72]), intermediate_size=rng.choice([48, 88]),
             vocab_size=rng.choice([101, 260]), num_hidden_layers=2, num_attention_heads=nkv * G,
             num_key_value_heads=nkv, head_dim=d, rope_theta=1e4, rms_norm_eps=1e-6)
    if rng.random() < 0.5:
        c.update(use_sliding_window=True, sliding_window=rng.choice([5, 24]), max_window_layers=1)
    return c


def configuration(seed):
    rng = random.Random(seed)
    c = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", max_position_embeddings=1024,
             torch_dtype="float32", bos_token_id=0, use_sliding_window=False)
    c.update(odd_heads(rng) if seed >= 200 else unusual(rng) if seed >= 100 else usual(rng))
    c.update(tie_word_embeddings=rng.random() < 0.5, eos_token_id=c["vocab_size"] - 1)
    return c, rng


@pytest.mark.parametrize("seed", [0, 3, 5, 6, 100, 102, 105, 106, 200, 201])
def test_random_configuration(seed, tmp_path):
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    c, rng = configuration(seed)
    print(f"seed {seed}: {c}")
    cfgo = Qwen2Config.from_dict(c)
    lens = [1, 2, 17, 33, 64, 100, 129, 47][: rng.choice([5, 6, 8])]
    rng.shuffle(lens)
    for ck, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        folder = str(tmp_path / ck)
        os.makedirs(folder)
        write_model_folder(folder, cfgo, expected_weights(qwen2_forward_config(cfgo)), seed=seed, dtype=dt,
                           noisy_norms=True, std=0.02 if ck == "f32" else sharp_std(c["hidden_size"]))
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(c, f)
        cfg, w = plain.load_folder(folder)
        reqs = {f"r{i}": traces.random_tokens(cfg["vocab_size"], n, seed=seed * 100 + i) for i, n in enumerate(lens)}
        ref = {rid: plain.forward(cfg, w, toks) for rid, toks in reqs.items()}
        for dtype in ("float32", "bfloat16"):
            for shape in (traces.whole, traces.last_decoded, traces.portions, traces.mixed):
                steps = shape(reqs)
                pages = traces.max_live_tokens(steps) // 16
                eng = Engine.from_folder(folder, dtype, SchedulerConfig(
                    num_kv_blocks=pages, kv_block_size=16, max_batch_requests=8, max_batch_tokens=pages * 16,
                    max_seq_len=pages * 16))
                out = traces.run_in_process(eng, steps)
                worst, mean, scale, rows, where = traces.compare(steps, out, ref, reqs)
                what = f"checkpoint {ck}, engine {dtype}, {shape.__name__}: worst {worst:.2e} at {where}, scale {scale:.2e}"
                assert rows > 0
                if dtype == "float32":
                    assert worst <= F32_TOL * max(1.0, scale), what
                else:
                    assert worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale, what
