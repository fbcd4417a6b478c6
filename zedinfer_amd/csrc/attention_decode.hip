// Paged grouped-query attention for single query tokens, split over the keys.
//
// One wavefront per (token, key/value head, split of the keys).  It serves all
// G = heads / kv_heads query heads of its group from one pass over the keys and
// values, so each cached byte is read once per token.  A token at position p
// sees keys [lo, p] (lo = 0, or p - window + 1); that range, widened down to a
// multiple of 8, is cut into at most 64 splits of 64 keys (128, 256, ... when
// there are more than 4096 keys), which depends on the token alone, never on the
// rest of the batch.  Each split leaves a partial (running maximum, sum,
// unnormalised output) and a second kernel merges the splits; a token with one
// split is finished by the first kernel.
//
// Keys are read 16 bytes a lane, head_dim/8 lanes a key, and the dot products
// are finished with a butterfly over those lanes.  Values are stored transposed
// ([dim][slot]), so a lane owns output dimensions and reads eight consecutive
// positions of one dimension at a time.  Scores, the softmax and the sums are
// float32 (reference formulas: src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:15-72).
//
// bfloat16 only; head_dim 64, 128 or 256; group size up to 8; page size a multiple
// of 8.  Other shapes are the plain kernel's.
#include "zi_common.h"

#define DEC_MAXS 64      // most splits of one token
#define DEC_TILE 64      // keys a wavefront handles at a time

__device__ __forceinline__ void unpack8(const uint4& r, float* f) {
    f[0] = __uint_as_float(r.x << 16); f[1] = __uint_as_float(r.x & 0xffff0000u);
    f[2] = __uint_as_float(r.y << 16); f[3] = __uint_as_float(r.y & 0xffff0000u);
    f[4] = __uint_as_float(r.z << 16); f[5] = __uint_as_float(r.z & 0xffff0000u);
    f[6] = __uint_as_float(r.w << 16); f[7] = __uint_as_float(r.w & 0xffff0000u);
}

// The cut of a token's keys: first key seen, first key of split 0 (a multiple of 8),
// keys per split, number of splits.
struct DecSplit {
    int lo, lo_al, len, count;
};
__device__ __forceinline__ DecSplit dec_split(int p, int window) {
    DecSplit s;
    s.lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    s.lo_al = s.lo & ~7;
    const int nk = p - s.lo_al + 1;
    s.len = DEC_TILE;
    while (nk > s.len * DEC_MAXS) s.len *= 2;
    s.count = (nk + s.len - 1) / s.len;
    return s;
}

template <int D, int G>
__global__ void __launch_bounds__(ZI_WAVE)
attention_decode_kernel(zi_bf16* __restrict__ out, int64_t ldo, float* __restrict__ part_o,
                        float* __restrict__ part_ml, const zi_bf16* __restrict__ q, int64_t ldq,
                        const zi_bf16* __restrict__ kcache, const zi_bf16* __restrict__ vcache,
                        const int32_t* __restrict__ tok_index, const int32_t* __restrict__ tok_seq,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_tables,
                        int max_pages, int num_pages, int nh, int nkv, int ps, int window, float scale,
                        int max_splits) {
    constexpr int LPK = D / 8;          // lanes that share one key
    constexpr int KPI = ZI_WAVE / LPK;  // keys per load instruction
    constexpr int DV = D / ZI_WAVE;     // output dims per lane
    static_assert(D % ZI_WAVE == 0 && LPK <= ZI_WAVE, "head_dim must be 64, 128 or 256");
    __shared__ __attribute__((aligned(16))) float sc[G][DEC_TILE];

    const int x = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
    const int t = tok_index ? tok_index[x] : x;
    const int p = tok_pos[t];
    const DecSplit sp = dec_split(p, window);
    if (sp.count > max_splits) {
        // The host sized the launch (and the workspace) for fewer keys than this token sees.  Nothing
        // may be written to the workspace then; the token's output is made NaN so that it shows.
        if (split == 0)
            for (int i = lane; i < G * D; i += ZI_WAVE)
                zi_store(out + (int64_t)t * ldo + (int64_t)kvh * G * D + i, NAN);
        return;
    }
    if (split >= sp.count) return;
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const int k_begin = sp.lo_al + split * sp.len;
    const int k_stop = (k_begin + sp.len < p + 1) ? k_begin + sp.len : p + 1;   // one past the last key

    const int sub = lane / LPK, chunk = lane % LPK;
    float qr[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const uint4 raw = *reinterpret_cast<const uint4*>(q + (int64_t)t * ldq + (int64_t)(kvh * G + g) * D + chunk * 8);
        unpack8(raw, qr[g]);
    }
    float m[G], l[G], acc[G][DV];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int v = 0; v < DV; ++v) acc[g][v] = 0.f;
    }

    for (int base = k_begin; base < k_stop; base += DEC_TILE) {
        // ---- scores of up to 64 keys
#pragma unroll 2
        for (int i = 0; i < DEC_TILE / KPI; ++i) {
            const int key = base + i * KPI + sub;
            const bool valid = key >= sp.lo && key < k_stop;
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; ++g) dot[g] = 0.f;
            if (valid) {
                const int pi = key / ps;
                const int page = pi < max_pages ? bt[pi] : -1;
                if (page >= 0 && page < num_pages) {
                    const uint4 raw = *reinterpret_cast<const uint4*>(
                        kcache + (((int64_t)page * nkv + kvh) * ps + key % ps) * D + chunk * 8);
                    float kf[8];
                    unpack8(raw, kf);
#pragma unroll
                    for (int g = 0; g < G; ++g)
#pragma unroll
                        for (int e = 0; e < 8; ++e) dot[g] = fmaf(qr[g][e], kf[e], dot[g]);
                }
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
#pragma unroll
                for (int o = LPK / 2; o > 0; o >>= 1) dot[g] += __shfl_xor(dot[g], o, ZI_WAVE);
            }
            if (chunk == 0) {
#pragma unroll
                for (int g = 0; g < G; ++g) sc[g][i * KPI + sub] = valid ? dot[g] * scale : -INFINITY;
            }
        }
        __syncthreads();
        // ---- running softmax, one key a lane
        float corr[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float s = sc[g][lane];
            const float m_new = fmaxf(m[g], zi_wave_max(s));
            const float pj = (s == -INFINITY) ? 0.f : expf(s - m_new);
            corr[g] = (m[g] == -INFINITY) ? 0.f : expf(m[g] - m_new);
            l[g] = l[g] * corr[g] + zi_wave_sum(pj);
            m[g] = m_new;
            sc[g][lane] = pj;
#pragma unroll
            for (int v = 0; v < DV; ++v) acc[g][v] *= corr[g];
        }
        __syncthreads();
        // ---- values: eight positions of one dimension per load
        for (int grp = 0; grp < DEC_TILE / 8; ++grp) {
            const int key0 = base + grp * 8;
            if (key0 >= k_stop || key0 + 8 <= sp.lo) continue;
            const int pi = key0 / ps;
            const int page = pi < max_pages ? bt[pi] : -1;
            if (page < 0 || page >= num_pages) continue;
            const bool edge = key0 < sp.lo || key0 + 8 > k_stop;
            const int64_t vb = ((int64_t)page * nkv + kvh) * D * ps + key0 % ps;
#pragma unroll
            for (int v = 0; v < DV; ++v) {
                const uint4 raw = *reinterpret_cast<const uint4*>(vcache + vb + (int64_t)(lane + v * ZI_WAVE) * ps);
                float vf[8];
                unpack8(raw, vf);
                if (edge) {   // positions outside [lo, p] may hold anything: keep them out of the sum
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (key0 + e < sp.lo || key0 + e >= k_stop) vf[e] = 0.f;
                }
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const float4 p0 = *reinterpret_cast<const float4*>(&sc[g][grp * 8]);
                    const float4 p1 = *reinterpret_cast<const float4*>(&sc[g][grp * 8 + 4]);
                    float a = acc[g][v];
                    a = fmaf(p0.x, vf[0], a); a = fmaf(p0.y, vf[1], a); a = fmaf(p0.z, vf[2], a); a = fmaf(p0.w, vf[3], a);
                    a = fmaf(p1.x, vf[4], a); a = fmaf(p1.y, vf[5], a); a = fmaf(p1.z, vf[6], a); a = fmaf(p1.w, vf[7], a);
                    acc[g][v] = a;
                }
            }
        }
        __syncthreads();
    }

    if (sp.count == 1) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float inv = 1.f / l[g];
#pragma unroll
            for (int v = 0; v < DV; ++v)
                zi_store(out + (int64_t)t * ldo + (int64_t)(kvh * G + g) * D + lane + v * ZI_WAVE, acc[g][v] * inv);
        }
        return;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int64_t slot = ((int64_t)x * nh + kvh * G + g) * DEC_MAXS + split;
#pragma unroll
        for (int v = 0; v < DV; ++v) part_o[slot * D + lane + v * ZI_WAVE] = acc[g][v];
        if (lane == 0) {
            part_ml[slot * 2] = m[g];
            part_ml[slot * 2 + 1] = l[g];
        }
    }
}

// Merge the splits of one (token, head): out = sum_s e^(m_s - M) o_s / sum_s e^(m_s - M) l_s.
template <int D>
__global__ void __launch_bounds__(ZI_WAVE)
attention_decode_merge_kernel(zi_bf16* __restrict__ out, int64_t ldo, const float* __restrict__ part_o,
                              const float* __restrict__ part_ml, const int32_t* __restrict__ tok_index,
                              const int32_t* __restrict__ tok_pos, int nh, int window, int max_splits) {
    constexpr int DV = D / ZI_WAVE;
    const int x = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int t = tok_index ? tok_index[x] : x;
    const DecSplit sp = dec_split(tok_pos[t], window);
    if (sp.count == 1 || sp.count > max_splits) return;
    const int64_t slot0 = ((int64_t)x * nh + h) * DEC_MAXS;
    float M = -INFINITY;
    for (int s = 0; s < sp.count; ++s) M = fmaxf(M, part_ml[(slot0 + s) * 2]);
    float L = 0.f, acc[DV];
#pragma unroll
    for (int v = 0; v < DV; ++v) acc[v] = 0.f;
    for (int s = 0; s < sp.count; ++s) {
        const float ms = part_ml[(slot0 + s) * 2];
        const float w = (ms == -INFINITY) ? 0.f : expf(ms - M);
        L += w * part_ml[(slot0 + s) * 2 + 1];
#pragma unroll
        for (int v = 0; v < DV; ++v) acc[v] += w * part_o[(slot0 + s) * D + lane + v * ZI_WAVE];
    }
    const float inv = 1.f / L;
#pragma unroll
    for (int v = 0; v < DV; ++v) zi_store(out + (int64_t)t * ldo + (int64_t)h * D + lane + v * ZI_WAVE, acc[v] * inv);
}

template <int D>
static int launch_decode(int G, dim3 grid, hipStream_t stream, zi_bf16* out, int64_t ldo, float* po, float* pml,
                         const zi_bf16* q, int64_t ldq, const zi_bf16* kc, const zi_bf16* vc, const int32_t* ti,
                         const int32_t* ts, const int32_t* tp, const int32_t* bt, int max_pages, int num_pages,
                         int nh, int nkv, int ps, int window, float scale, int max_splits) {
#define ZI_DEC_CASE(GG)                                                                                          \
    case GG:                                                                                                     \
        attention_decode_kernel<D, GG><<<grid, ZI_WAVE, 0, stream>>>(out, ldo, po, pml, q, ldq, kc, vc, ti, ts, \
                                                                     tp, bt, max_pages, num_pages, nh, nkv, ps, \
                                                                     window, scale, max_splits);                \
        break;
    switch (G) {
        ZI_DEC_CASE(1) ZI_DEC_CASE(2) ZI_DEC_CASE(3) ZI_DEC_CASE(4) ZI_DEC_CASE(5) ZI_DEC_CASE(6) ZI_DEC_CASE(7)
        ZI_DEC_CASE(8)
        default: return zi_fail("attention_decode: group size %d is not supported (1..8)", G);
    }
#undef ZI_DEC_CASE
    return 0;
}

// Floats of workspace the split kernel needs for n tokens.
extern "C" int64_t zi_attention_decode_workspace(int n, int nh, int d) {
    return (int64_t)n * nh * DEC_MAXS * (d + 2);
}

// 1 when the shape is this kernel's, else 0.
extern "C" int zi_attention_decode_supported(int dt, int nh, int nkv, int d, int page_size) {
    if (dt != ZI_BF16 || nkv <= 0 || nh % nkv) return 0;
    const int G = nh / nkv;
    return (d == 64 || d == 128 || d == 256) && G >= 1 && G <= 8 && page_size % 8 == 0;
}

extern "C" int zi_attention_decode(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo,
                                   const void* kcache, const void* vcache, const int32_t* tok_index,
                                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables,
                                   int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window,
                                   float scale, int max_splits, float* workspace, int64_t workspace_floats,
                                   hipStream_t stream) {
    ZI_REQUIRE(zi_attention_decode_supported(dt, nh, nkv, d, page_size),
               "attention_decode: unsupported shape (bfloat16, head_dim 64/128/256, group <= 8, page size %% 8 == 0): "
               "dtype %d heads %d kv_heads %d head_dim %d page %d", dt, nh, nkv, d, page_size);
    ZI_REQUIRE(n_idx >= 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode: bad sizes");
    ZI_REQUIRE(max_splits >= 1 && max_splits <= DEC_MAXS, "attention_decode: max_splits %d outside 1..%d", max_splits, DEC_MAXS);
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldo >= (int64_t)nh * d && ldq % 8 == 0, "attention_decode: bad row stride");
    ZI_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0,
               "attention_decode: q and the caches must be 16-byte aligned");
    ZI_REQUIRE(nkv <= 65535, "attention_decode: too many kv heads");
    if (n_idx == 0) return 0;
    ZI_REQUIRE(max_splits == 1 || workspace_floats >= zi_attention_decode_workspace(n_idx, nh, d),
               "attention_decode: workspace of %lld floats is too small", (long long)workspace_floats);
    float* po = workspace;
    float* pml = workspace ? workspace + (int64_t)n_idx * nh * DEC_MAXS * d : nullptr;
    const dim3 grid(n_idx, nkv, max_splits);
    int rc = 0;
    const int G = nh / nkv;
#define ZI_DEC_D(DD)                                                                                               \
    rc = launch_decode<DD>(G, grid, stream, (zi_bf16*)out, ldo, po, pml, (const zi_bf16*)q, ldq,                   \
                           (const zi_bf16*)kcache, (const zi_bf16*)vcache, tok_index, tok_seq, tok_pos,            \
                           block_tables, max_pages, num_pages, nh, nkv, page_size, window, scale, max_splits);     \
    if (!rc && max_splits > 1)                                                                                     \
        attention_decode_merge_kernel<DD><<<dim3(n_idx, nh), ZI_WAVE, 0, stream>>>((zi_bf16*)out, ldo, po, pml,    \
                                                                                   tok_index, tok_pos, nh, window,  \
                                                                                   max_splits);
    if (d == 64) { ZI_DEC_D(64) } else if (d == 128) { ZI_DEC_D(128) } else { ZI_DEC_D(256) }
#undef ZI_DEC_D
    if (rc) return rc;
    return zi_check_launch("attention_decode");
}
