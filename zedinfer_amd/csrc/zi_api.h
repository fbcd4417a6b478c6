// The entry points of the kernel library that launch work on a stream: one declaration each, seen by the
// file that defines it (so the two cannot drift apart) and by the step tape (tape.hip), which calls them
// by name with recorded arguments.  Every one returns 0, or non-zero with a message for zi_last_error().
// Pointers are device memory unless a comment at the definition says otherwise.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

// attention_decode.hip
int zi_attention_decode(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_chunks, float* workspace, int64_t workspace_floats, hipStream_t stream);
// attention_decode.hip
int zi_attention_decode_fused(void* out, int dt, int n_idx, int64_t ldo, const float* sums, int splits, int64_t
    split_stride, int64_t ldp, const void* bias, int bias_dt, const float* table, int rot, const int32_t* slots,
    int64_t cache_slots, int write_kv, void* kcache, void* vcache, const int32_t* tok_index, const int32_t* tok_seq,
    const int32_t* tok_pos, const int32_t* block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int
    page_size, int window, float scale, int max_chunks, float* workspace, int64_t workspace_floats, hipStream_t
    stream);
// attention_decode.hip
int zi_attention_decode_project(float* sums, const float* workspace, int64_t workspace_floats, int n, const int32_t*
    tok_pos, int window, int max_chunks, const void* w, int dt, int64_t ldw, int N, int nh, int d, hipStream_t
    stream);
// attention_generic.hip
int zi_attention_generic(void* out, const void* q, int dt, int n, int64_t ldq, int64_t ldo, const void* kcache, const
    void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale,
    hipStream_t stream);
// attention_prefill.hip
int zi_attention_prefill(void* out, const void* q, int dt, int num_tiles, int64_t ldq, int64_t ldo, const void*
    kcache, const void* vcache, const int32_t* tile_entry, const int32_t* tile_off, const int32_t* entry_start, const
    int32_t* entry_len, const int32_t* entry_past, const int32_t* block_tables, int max_pages, int num_pages, int nh,
    int nkv, int d, int page_size, int window, float scale, int rows, int max_chunks, float* workspace, int64_t
    workspace_floats, int tile, int alone, int chunk_keys, hipStream_t stream);
// decode_layer.hip
int zi_decode_layer(float* resid, int n, int H, int I, const void* norm1, const void* norm2, int norm_dt, float eps1,
    float eps2, int add_one, const void* wqkv, int64_t ld_qkv, const void* bias, int bias_dt, const void* wo, int64_t
    ld_o, const void* wgu, int64_t ld_gu, const void* wd, int64_t ld_d, int dt, const float* table, int rot, const
    int32_t* slots, int64_t cache_slots, void* kcache, void* vcache, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_keys, void* workspace, int64_t workspace_bytes, uint32_t* sync, int* err, int spin_limit, hipStream_t stream);
// elementwise.hip
int zi_embedding(void* out, int out_dt, const void* table, int table_dt, const int32_t* ids, int n, int hidden, int
    vocab, hipStream_t stream);
// elementwise.hip
int zi_gather_rows(void* out, const void* in, int dt, const int32_t* idx, int n_out, int n_in, int hidden, hipStream_t
    stream);
// elementwise.hip
int zi_add(void* c, int c_dt, const void* a, int a_dt, const void* b, int b_dt, int64_t n, hipStream_t stream);
// elementwise.hip
int zi_swiglu_t(void* out, const void* gut, int dt, int n, int inter, int64_t ldt, hipStream_t stream);
// elementwise.hip
int zi_swiglu(void* out, int out_dt, const void* gate, const void* up, int dt, int n, int inter, int64_t ld_gate,
    int64_t ld_up, int interleave, int splits, int64_t split_stride, hipStream_t stream);
// gemm_generic.hip
int zi_gemm_generic(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt, const void* bias, int
    bias_dt, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, hipStream_t stream);
// gemm_lt.hip
int zi_gemm_lt(void* out, int out_dt, const void* x, const void* weight, const void* bias, int transposed, int64_t M,
    int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* workspace, int64_t workspace_bytes, hipStream_t
    stream);
// gemm_skinny.hip
int zi_gemm_skinny(void* out, int out_dt, int mode, const void* x, const void* w, const void* bias, int M, int N, int
    K, int64_t ldx, int64_t ldw, int64_t ldo, float* workspace, int64_t workspace_floats, hipStream_t stream);
// gemm_skinny.hip
int zi_reduce_splits(void* out, int out_dt, const float* sums, const void* bias, int M, int N, int64_t ldo, int
    splits, hipStream_t stream);
// norm.hip
int zi_rmsnorm(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt, int n, int hidden, int64_t
    ldx, int64_t ldo, float eps, int add_one, hipStream_t stream);
// norm.hip
int zi_add_rmsnorm(void* out, int out_dt, float* resid, const void* delta, int delta_dt, int splits, int64_t
    split_stride, const void* w, int w_dt, int n, int hidden, float eps, int add_one, hipStream_t stream);
// rope_kv.hip
int zi_rope_kv_store(void* q, const void* k, const void* v, int dt, int n, int64_t ldq, int64_t ldk, int64_t ldv,
    const int32_t* slots, const float* table, void* kcache, void* vcache, int64_t cache_slots, int nh, int nkv, int d,
    int rot, int page_size, int write_kv, hipStream_t stream);
// rope_kv.hip
int zi_rope_kv_store_split(void* q_out, int dt, int64_t ldq, const float* part, int splits, int64_t split_stride,
    int64_t ldp, const void* bias, int bias_dt, int n, const int32_t* slots, const float* table, void* kcache, void*
    vcache, int64_t cache_slots, int nh, int nkv, int d, int rot, int page_size, int write_kv, hipStream_t stream);
// rope_kv.hip
int zi_rope(void* out, const void* in, int dt, int n, int64_t ld_in, int64_t ld_out, const int32_t* pos, const float*
    inv_freq, int nh, int d, int rot, hipStream_t stream);
// rope_kv.hip
int zi_rope_table(float* out, const int32_t* pos, const float* inv_freq, int n, int half, hipStream_t stream);
// sampling.hip
int zi_argmax(int32_t* out_idx, float* out_val, const void* logits, int dt, int rows, int vocab, int64_t ld, float*
    workspace, int64_t workspace_floats, hipStream_t stream);
// sampling.hip
int zi_sample(int32_t* out, const float* logits, int64_t ld, float* work, int rows, int vocab, const float*
    temperature, const int32_t* top_k, const float* top_p, const float* penalty, const float* uniform, const int32_t*
    recent, const int32_t* recent_len, int max_recent, hipStream_t stream);
}

// Every entry point above, for code that wants them all (X is applied to each name).
#define ZI_STREAM_ENTRY_POINTS(X) \
    X(zi_attention_decode) \
    X(zi_attention_decode_fused) \
    X(zi_attention_decode_project) \
    X(zi_attention_generic) \
    X(zi_attention_prefill) \
    X(zi_decode_layer) \
    X(zi_embedding) \
    X(zi_gather_rows) \
    X(zi_add) \
    X(zi_swiglu_t) \
    X(zi_swiglu) \
    X(zi_gemm_generic) \
    X(zi_gemm_lt) \
    X(zi_gemm_skinny) \
    X(zi_reduce_splits) \
    X(zi_rmsnorm) \
    X(zi_add_rmsnorm) \
    X(zi_rope_kv_store) \
    X(zi_rope_kv_store_split) \
    X(zi_rope) \
    X(zi_rope_table) \
    X(zi_argmax) \
    X(zi_sample)
