"""A context of 20,000 tokens: the bfloat16 serving kernels (prompt attention over many blocks, decode
attention past 16,384 keys, where its chunks grow, replayed as graphs) against the float32 path of the same
model, which runs the plain kernels.  The plain implementation on the CPU would take minutes at this
length; the float32 path is checked against it at short lengths by the other tests."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_long_context_serving_kernels_agree_with_the_float32_path(tmp_path):
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    cfg = Qwen2Config.from_dict(dict(
        architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=2003, max_position_embeddings=32768,
        num_hidden_layers=2, rope_theta=1000000.0, rms_norm_eps=1e-6, use_sliding_window=False,
        torch_dtype="bfloat16", eos_token_id=2002, hidden_size=512, intermediate_size=1408, num_attention_heads=8,
        num_key_value_heads=2, head_dim=128, tie_word_embeddings=True))
    folder = str(tmp_path / "long")
    write_model_folder(folder, cfg, expected_weights(qwen2_forward_config(cfg)), seed=3, dtype=torch.bfloat16,
                       noisy_norms=True)
    T, decoded = 20000, 40
    toks = torch.randint(0, 2002, (T + decoded,), generator=torch.Generator().manual_seed(0)).tolist()
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=(T + decoded) // 16 + 8, kv_block_size=16,
                                                                 max_batch_requests=4, max_batch_tokens=4096))
        eng.graph_after = 2
        seq = eng.open("long")
        rows = []
        for a in range(0, T, 2048):
            b = min(T, a + 2048)
            rows.append(eng.step([StepEntry(seq, toks[a:b], [b - a - 1])]).cpu())
        for i in range(T, T + decoded):
            rows.append(eng.step([StepEntry(seq, [toks[i]], [0])]).cpu())
        assert eng.graph_replays >= decoded - 2
        eng.close(seq)
        outs[dtype] = torch.cat(rows)
    diff = (outs["float32"] - outs["bfloat16"]).abs()
    scale = float(outs["float32"].abs().max())
    print(f"rows={diff.shape[0]} worst={float(diff.max()):.3e} mean={float(diff.mean()):.3e} scale={scale:.3e}")
    assert float(diff.max()) <= 0.06 * scale and float(diff.mean()) <= 0.012 * scale


def test_a_long_prompt_in_one_step_agrees_with_the_float32_path(tmp_path):
    """13,000 tokens of one prompt in one step: tiles x heads enough for the prompt attention's long cut along the
    keys (one workgroup walks all of a tile's keys, nothing is merged), against the 32-bit engine at rows from the
    first to the last; then a second portion on top of it, which has few tiles and takes the short cut."""
    from zedinfer_amd import ops
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine, StepEntry
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    cfg = Qwen2Config.from_dict(dict(
        architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=2003, max_position_embeddings=32768,
        num_hidden_layers=2, rope_theta=1000000.0, rms_norm_eps=1e-6, use_sliding_window=False,
        torch_dtype="bfloat16", eos_token_id=2002, hidden_size=512, intermediate_size=1408, num_attention_heads=8,
        num_key_value_heads=2, head_dim=128, tie_word_embeddings=True))
    folder = str(tmp_path / "long")
    write_model_folder(folder, cfg, expected_weights(qwen2_forward_config(cfg)), seed=4, dtype=torch.bfloat16,
                       noisy_norms=True)
    T, more = 13000, 700
    toks = torch.randint(0, 2002, (T + more,), generator=torch.Generator().manual_seed(1)).tolist()
    want = [0, 1, 2047, 2048, 6143, 6144, 9999, T - 1]
    cuts = []
    real = ops.attention_prefill_workspace

    def seen(rows, nh, d, max_keys, window=0, num_tiles=0):
        cuts.append((num_tiles * nh, real(rows, nh, d, max_keys, window, num_tiles)))
        return cuts[-1][1]
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=(T + more) // 16 + 8, kv_block_size=16,
                                                                 max_batch_requests=2, max_batch_tokens=T + 64,
                                                                 max_seq_len=16384))
        seq = eng.open("long")
        ops.attention_prefill_workspace = seen
        try:
            first = eng.step([StepEntry(seq, toks[:T], want)]).cpu()
            second = eng.step([StepEntry(seq, toks[T:], [0, more - 1])]).cpu()
        finally:
            ops.attention_prefill_workspace = real
        eng.close(seq)
        outs[dtype] = torch.cat([first, second])
    # the serving engine's first step had tiles enough for the long cut (no workspace), its second had not
    assert [(g >= 768, need == 0) for g, need in cuts] == [(True, True)] * 2 + [(False, False)] * 2, cuts
    diff = (outs["float32"] - outs["bfloat16"]).abs()
    scale = float(outs["float32"].abs().max())
    print(f"rows={diff.shape[0]} worst={float(diff.max()):.3e} mean={float(diff.mean()):.3e} scale={scale:.3e}")
    assert float(diff.max()) <= 0.06 * scale and float(diff.mean()) <= 0.012 * scale
