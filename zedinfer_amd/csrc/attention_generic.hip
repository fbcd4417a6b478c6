// Causal grouped-query attention over the paged cache: the plain kernel.
//
// One wavefront per (token, query head); with a token list only the listed tokens are done
// (n counts the list then).  The token at absolute position p of
// its sequence sees the keys at positions [lo, p], lo = 0, or p - window + 1
// for a windowed layer; keys and values are found through the sequence's block
// table.  s_j = (q . k_j) * scale, softmax with the running maximum subtracted,
// o = sum_j P_j v_j, all in float32 (reference:
// src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:106-162; the scale
// after the dot product at :135, the causal bound at :116).
//
// It takes every head size up to 512, any number of heads and groups, any page
// size, both storage types, prompts and decoded tokens alike, and its result
// for a token depends only on that token's position and keys, not on the
// batch.  The faster kernels cover the common shapes; this one covers the rest
// and the float32 path.
#include "zi_common.h"
#include "zi_api.h"

#define ATTN_MAX_D 512
#define ATTN_ACC (ATTN_MAX_D / ZI_WAVE)

template <typename T>
__global__ void __launch_bounds__(ZI_WAVE)
attention_generic_kernel(T* __restrict__ out, const T* __restrict__ q, int64_t ldq, int64_t ldo,
                         const T* __restrict__ kcache, const T* __restrict__ vcache,
                         const int32_t* __restrict__ tok_index, const int32_t* __restrict__ tok_seq,
                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_tables,
                         int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window,
                         float scale) {
    __shared__ float qs[ATTN_MAX_D];
    __shared__ float ps[ZI_WAVE];
    __shared__ int64_t vbase[ZI_WAVE];
    const int t = tok_index ? tok_index[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (nh / nkv);
    const int p = tok_pos[t];
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;

    const T* qr = q + (int64_t)t * ldq + (int64_t)h * d;
    for (int j = lane; j < d; j += ZI_WAVE) qs[j] = zi_load(qr + j);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATTN_ACC];
#pragma unroll
    for (int i = 0; i < ATTN_ACC; ++i) acc[i] = 0.f;

    for (int base = lo; base <= p; base += ZI_WAVE) {
        const int j = base + lane;
        bool valid = j <= p;
        float s = -INFINITY;
        int64_t row = -1, vrow = -1;
        if (valid) {
            const int pi = j / page_size;
            const int page = pi < max_pages ? bt[pi] : -1;
            if (page < 0 || page >= num_pages) {
                valid = false;  // a hole in the table: the host never schedules this; stay in bounds
            } else {
                row = (((int64_t)page * nkv + g) * page_size + (j % page_size)) * d;
                vrow = ((int64_t)page * nkv + g) * page_size * d + (j % page_size);
                const T* kr = kcache + row;
                float dot = 0.f;
                for (int x = 0; x < d; ++x) dot += qs[x] * zi_load(kr + x);
                s = dot * scale;
            }
        }
        const float mt = zi_wave_max(s);
        const float m_new = fmaxf(m, mt);
        const float pj = valid ? expf(s - m_new) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + zi_wave_sum(pj);
        ps[lane] = pj;
        vbase[lane] = vrow;
        __syncthreads();
        const int cnt = (p - base + 1 < ZI_WAVE) ? p - base + 1 : ZI_WAVE;
#pragma unroll
        for (int i = 0; i < ATTN_ACC; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const float pw = ps[jj];
            const int64_t vr = vbase[jj];
            if (vr < 0) continue;
#pragma unroll
            for (int i = 0; i < ATTN_ACC; ++i) {
                const int x = lane + i * ZI_WAVE;
                if (x < d) acc[i] += pw * zi_load(vcache + vr + (int64_t)x * page_size);
            }
        }
        m = m_new;
        __syncthreads();
    }
    T* orow = out + (int64_t)t * ldo + (int64_t)h * d;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < ATTN_ACC; ++i) {
        const int x = lane + i * ZI_WAVE;
        if (x < d) zi_store(orow + x, acc[i] * inv);
    }
}

extern "C" int zi_attention_generic(void* out, const void* q, int dt, int n, int64_t ldq, int64_t ldo,
                                    const void* kcache, const void* vcache, const int32_t* tok_index,
                                    const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables, int max_pages,
                                    int num_pages, int nh, int nkv, int d, int page_size, int window, float scale,
                                    hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0 && max_pages > 0 && num_pages > 0,
               "attention: bad sizes");
    ZI_REQUIRE(nh % nkv == 0, "attention: %d query heads are not a multiple of %d key/value heads", nh, nkv);
    ZI_REQUIRE(d <= ATTN_MAX_D, "attention: head_dim %d is larger than the %d this kernel holds", d, ATTN_MAX_D);
    ZI_REQUIRE(nh <= 65535, "attention: too many heads (%d)", nh);
    ZI_REQUIRE(window >= 0, "attention: negative window");
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldo >= (int64_t)nh * d, "attention: row stride too small");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        attention_generic_kernel<T><<<dim3(n, nh), ZI_WAVE, 0, stream>>>(
            (T*)out, (const T*)q, ldq, ldo, (const T*)kcache, (const T*)vcache, tok_index, tok_seq, tok_pos, block_tables,
            max_pages, num_pages, nh, nkv, d, page_size, window, scale);
    });
    return zi_check_launch("attention_generic");
}
