"""The tiny Qwen2 configurations the tests use.  A and B differ in every size and option; C adds
an explicit head_dim that is not hidden/heads and a sliding window on the later layers."""
import json
import os

TINY_A = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=64, intermediate_size=176,
    vocab_size=512, max_position_embeddings=256, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
    use_sliding_window=False, sliding_window=4096, max_window_layers=21, torch_dtype="float32",
    eos_token_id=511, bos_token_id=0)

TINY_B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=96, intermediate_size=256,
    vocab_size=1000, max_position_embeddings=512, num_hidden_layers=3, num_attention_heads=3,
    num_key_value_heads=1, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    use_sliding_window=False, torch_dtype="float32", eos_token_id=[998, 999], bos_token_id=1)

TINY_C = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=80, intermediate_size=208,
    vocab_size=777, max_position_embeddings=512, num_hidden_layers=3, num_attention_heads=6,
    num_key_value_heads=2, head_dim=48, rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False,
    use_sliding_window=True, sliding_window=20, max_window_layers=1, torch_dtype="float32",
    eos_token_id=776, bos_token_id=1)

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
PAGE_SIZES = {"A": 16, "B": 8, "C": 8}
SEEDS = {"A": 0, "B": 1, "C": 2}
NOISY_NORMS = {"A": False, "B": True, "C": True}


SHARP_STD = 0.1     # weights this wide make attention peaked: a wrong rotation or scale moves the logits by their whole size


def write_tiny(folder, name, dtype=None, std=0.02):
    """Write config.json and model.safetensors of a tiny configuration with the engine's
    random-weights mode; returns the folder.  ``std`` is the width of the matrices and biases
    (SHARP_STD for the "sharp" variants of the tests)."""
    import torch
    from zedinfer_amd.config import Qwen2Config
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    cfg = Qwen2Config.from_dict(CONFIGS[name])
    fc = qwen2_forward_config(cfg)
    write_model_folder(folder, cfg, expected_weights(fc), seed=SEEDS[name], dtype=dtype or torch.float32,
                       noisy_norms=NOISY_NORMS[name], std=std)
    # keep the keys of the test's dict exactly (eos list and so on)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(CONFIGS[name], f, indent=1)
    return folder
