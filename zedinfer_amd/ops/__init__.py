"""The operators: thin, checked Python entries over the HIP kernels.

Each function checks devices, storage types, shapes and strides on the host,
then launches on torch's current stream.  The op-level names follow the
reference's Python module (reference: python/bindings/zedinfer_ops.cpp:257-291:
add, argmax, embedding, linear, rms_norm, rope, swiglu).
"""
from .functional import (add, add_rms_norm, argmax, attention, attention_decode, attention_decode_chunks,
                         attention_decode_fused,
                         attention_decode_fused_supported, attention_decode_project,
                         attention_decode_project_splits, attention_decode_project_supported,
                         attention_decode_supported, attention_decode_workspace, attention_prefill,
                         attention_prefill_supported, attention_prefill_tile, attention_prefill_tile_min, attention_prefill_variant,
                         attention_prefill_workspace, compute_units, decode_layer, decode_layer_stamps, decode_layer_supported, decode_layer_sync_words,
                         decode_layer_workspace, device_synchronize, embedding, gather_rows, kv_store,
                         has_cuda, has_gpu, linear, linear_choose, linear_splits, linear_sums,
                         linear_sums_supported, linear_swiglu, linear_swiglu_supported,
                         linear_transposed, linear_tune, reduce_sums, rms_norm, rope, rope_inv_freq,
                         rope_kv_store, rope_kv_store_sums, rope_table, sample, swiglu, swiglu_t,
                         DECODE_LAYER_SPIN_LIMIT, FEW_ROWS, SUMS_MAX_ROWS)
from ._lib import KernelLibraryError, library_path, load

__all__ = [
    "DECODE_LAYER_SPIN_LIMIT",
    "add", "add_rms_norm", "argmax", "attention", "attention_decode", "attention_decode_chunks", "attention_decode_fused",
    "attention_decode_fused_supported", "attention_decode_project", "attention_decode_project_splits",
    "attention_decode_project_supported", "attention_decode_supported", "attention_decode_workspace",
    "attention_prefill", "attention_prefill_supported", "attention_prefill_tile", "attention_prefill_tile_min", "attention_prefill_variant",
    "attention_prefill_workspace", "compute_units", "decode_layer", "decode_layer_stamps", "decode_layer_supported", "decode_layer_sync_words",
    "decode_layer_workspace", "device_synchronize", "embedding", "gather_rows", "has_cuda", "kv_store", "has_gpu",
    "linear", "linear_choose", "linear_splits", "linear_sums", "linear_sums_supported", "linear_swiglu",
    "linear_swiglu_supported", "linear_transposed", "linear_tune", "reduce_sums", "rms_norm", "rope",
    "rope_inv_freq", "rope_kv_store", "rope_kv_store_sums", "rope_table", "sample", "swiglu", "swiglu_t",
    "KernelLibraryError", "library_path", "load", "FEW_ROWS", "SUMS_MAX_ROWS",
]
