"""A context of 20,000 tokens: the bfloat16 serving kernels (prompt attention over many blocks, decode
attention past 16,384 keys, where its chunks grow, replayed as graphs) against the float32 path of the same
model, which runs the plain kernels.  The plain implementation on the CPU would take minutes at this
length; the float32 path is checked against it at short lengths by the other tests."""
import pytest
import torch

from tolerances import sharp_std

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
    # sharp weights: attention is peaked, so a lost or doubled run of keys moves the logits beyond the tolerance
    write_model_folder(folder, cfg, expected_weights(qwen2_forward_config(cfg)), seed=3, dtype=torch.bfloat16,
                       noisy_norms=True, std=sharp_std(cfg.hidden_size))
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
                       noisy_norms=True, std=sharp_std(cfg.hidden_size))
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


LONG_PLAIN = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=2003, max_position_embeddings=8192,
    num_hidden_layers=2, rope_theta=1000000.0, rms_norm_eps=1e-6, use_sliding_window=False, torch_dtype="bfloat16",
    eos_token_id=2002, hidden_size=256, intermediate_size=400, num_attention_heads=4, num_key_value_heads=2,
    head_dim=128, tie_word_embeddings=False)


def long_plain_steps(a, b):
    """Request "a" (4,640 tokens): 2,100 in one step, portions of 700, 64, 2 and 1,734, then 40 tokens one by one;
    request "b" (300 tokens) starts late, in portions beside a's, and decodes beside a's decoded tokens.  Wanted
    rows lie around the prompt attention's 2,048-key cut, at the ends of the portions, and at every decoded token."""
    steps = []

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})
    add([{"id": "a", "tokens": a[:2100], "want": [0, 1, 2046, 2047, 2048, 2049, 2099]}])
    add([{"id": "a", "tokens": a[2100:2800], "want": [0, 1, 350, 699]}])
    add([{"id": "a", "tokens": a[2800:2864], "want": [0, 63]}, {"id": "b", "tokens": b[:130], "want": [0, 129]}])
    add([{"id": "b", "tokens": b[130:260], "want": [0, 129]}, {"id": "a", "tokens": a[2864:2866], "want": [0, 1]}])
    add([{"id": "a", "tokens": a[2866:4600], "want": [0, 1229, 1230, 1231, 1733]}])       # crosses 4,096 keys
    fb = 260
    for i in range(4600, 4640):
        entries = [{"id": "a", "tokens": a[i:i + 1], "want": [0]}]
        if fb < len(b):
            entries.append({"id": "b", "tokens": b[fb:fb + 1], "want": [0]})
            fb += 1
        end = (["a"] if i == 4639 else []) + (["b"] if fb == len(b) and len(entries) == 2 else [])
        add(entries, end)
    assert fb == len(b)
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_against_the_plain_implementation(tmp_path, dtype):
    """The engine at 4,640 tokens against the plain implementation on the CPU (whole sequence, no cache), so that what
    the two engine paths share (the batch builder, the attention planner, the bound of the keys that sizes the
    decode launches, block tables wider than 128 columns, the host image of a decode step) is held against
    something that shares none of it.  The trace crosses the prompt attention's cut at 2,048 keys with its merge,
    the bound's steps of 512 (4,608 while decoding: the graph is keyed anew), decode attention over 18 chunks, and
    290 pages a request.  Weights are sharp, so that a lost or doubled run of keys moves the logits
    (reference formulas: src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:106-162)."""
    import traces
    from plain import qwen2_plain as plain
    from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL, sharp_std
    from zedinfer_amd.config import Qwen2Config, SchedulerConfig
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.models import expected_weights
    from zedinfer_amd.models.qwen2 import qwen2_forward_config
    from zedinfer_amd.weights import write_model_folder
    cfg = Qwen2Config.from_dict(LONG_PLAIN)
    folder = str(tmp_path / "long_plain")
    write_model_folder(folder, cfg, expected_weights(qwen2_forward_config(cfg)), seed=5,
                       dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32, noisy_norms=True,
                       std=sharp_std(cfg.hidden_size))
    requests = {"a": traces.random_tokens(2002, 4640, seed=11), "b": traces.random_tokens(2002, 300, seed=12)}
    pcfg, w = plain.load_folder(folder)
    reference = {rid: plain.forward(pcfg, w, toks) for rid, toks in requests.items()}
    steps = long_plain_steps(requests["a"], requests["b"])
    eng = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=(4640 + 300) // 16 + 8, kv_block_size=16,
                                                             max_batch_requests=4, max_batch_tokens=4096, max_seq_len=8192))
    eng.graph_after = 2
    out = traces.run_in_process(eng, steps)
    assert any(len(key[2]) and max(key[2]) > 128 for key in eng._graphs), "block tables wider than 128 columns were to be crossed"
    assert eng.graph_replays >= 20          # the decoded tokens ran as graphs, before and after the bound moved
    worst, mean, scale, rows, where = traces.compare(steps, out, reference, requests)
    print(f"[long {dtype}] rows={rows} worst={worst:.3e} mean={mean:.3e} scale={scale:.3e} at {where}")
    assert rows == 7 + 4 + 4 + 4 + 5 + 40 + 40
    if dtype == "float32":
        assert worst <= F32_TOL * max(1.0, scale), f"worst difference at (step, request, position) {where}"
    else:
        assert worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale, f"worst difference at {where}"
