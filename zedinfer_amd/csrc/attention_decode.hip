// Paged grouped-query attention for single query tokens, split over the keys, on
// the matrix cores.
//
// One workgroup of four wavefronts per (token, key/value head, chunk of the keys).
// It serves all G = heads / kv_heads query heads of its group from one pass over
// the keys and values, so each cached byte is read once per token: the G heads
// stand in for the 16 "queries" of a v_mfma_f32_16x16x32_bf16 tile (rows beyond G
// are zero).  A token at position p sees keys [lo, p] (lo = 0, or p - window + 1);
// that range, widened down to a multiple of 8, is cut into at most 64 chunks of 256
// keys (512, 1024, ... when there are more than 16384 keys), which depends on the
// token alone, never on the rest of the batch.  Inside a chunk every wavefront takes
// a quarter, in blocks of 64 keys: it loads the block's keys and values straight
// from the cache into matrix-core operands (nothing is shared between wavefronts,
// so nothing goes through LDS), computes the scores transposed, S^T = K . Q^T, so
// that a lane holds the scores of one head, runs the softmax on them in float32,
// and accumulates O^T += V^T . P^T.  The four wavefronts' running (maximum, sum,
// output) are merged through LDS; a token with one chunk is finished there, else
// the chunk leaves a partial and a second kernel merges the chunks in rising order.
// (reference formulas: src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:15-72;
// the scale is applied after the dot product, :44.)
//
// Operand layout: as in the prompt kernel, the keys of a block are assigned to the
// rows of the four score tiles in a permuted order (tile t, row j*4 + e <-> key
// (t/2)*32 + j*8 + (t%2)*4 + e), which makes the eight probabilities a lane holds
// after two tiles the eight consecutive keys that the P.V product wants from it.
// Values are cached transposed ([dim][slot]), so a lane reads 16-byte runs of keys.
//
// bfloat16 only; head_dim a multiple of 16 up to 128; group size up to 16; page size
// a multiple of 8.  Other shapes are the plain kernel's.
#include "zi_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 dec_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float dec_f32x4_t;

#define DEC_MAXC 64       // most chunks of one token
#define DEC_CHUNK 256     // keys of the smallest chunk
#define DEC_WAVES 4
#define DEC_BLOCK 64      // keys a wavefront handles at a time

union dec_pack {
    uint4 u;
    dec_bf16x8_t b;
    uint16_t h[8];
};

// The cut of a token's keys: first key seen, first key of chunk 0 (a multiple of 8),
// keys per chunk, number of chunks.
struct DecSplit {
    int lo, lo_al, len, count;
};
__host__ __device__ __forceinline__ DecSplit dec_split(int p, int window) {
    DecSplit s;
    s.lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    s.lo_al = s.lo & ~7;
    const int nk = p - s.lo_al + 1;
    s.len = DEC_CHUNK;
    while (nk > s.len * DEC_MAXC) s.len *= 2;
    s.count = (nk + s.len - 1) / s.len;
    return s;
}

template <int D>
__global__ void __launch_bounds__(DEC_WAVES* ZI_WAVE, 2)
attention_decode_kernel(zi_bf16* __restrict__ out, int64_t ldo, float* __restrict__ part_o,
                        float* __restrict__ part_ml, const zi_bf16* __restrict__ q, int64_t ldq,
                        const zi_bf16* __restrict__ kcache, const zi_bf16* __restrict__ vcache,
                        const int32_t* __restrict__ tok_index, const int32_t* __restrict__ tok_seq,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_tables,
                        int max_pages, int num_pages, int nh, int nkv, int G, int ps, int window, float scale,
                        int max_chunks) {
    static_assert(D % 16 == 0 && D >= 16 && D <= 128, "head_dim must be a multiple of 16 up to 128");
    constexpr int DK = (D + 31) / 32;   // k-steps of the score product
    constexpr int DT = D / 16;          // output tiles of 16 dims
    __shared__ float sm[DEC_WAVES][16], sl[DEC_WAVES][16];
    __shared__ dec_f32x4_t so[DEC_WAVES][DT][ZI_WAVE];

    const int x = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int t = tok_index ? tok_index[x] : x;
    const int p = tok_pos[t];
    const DecSplit sp = dec_split(p, window);
    if (sp.count > max_chunks) {
        // The host sized the launch (and the workspace) for fewer keys than this token sees.  Nothing
        // may be written to the workspace then; the token's output is made NaN so that it shows.
        if (chunk == 0)
            for (int i = tid; i < G * D; i += DEC_WAVES * ZI_WAVE)
                zi_store(out + (int64_t)t * ldo + (int64_t)kvh * G * D + i, NAN);
        return;
    }
    if (chunk >= sp.count) return;
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const int ps_shift = (ps & (ps - 1)) == 0 ? __ffs(ps) - 1 : -1;   // no division for the usual page sizes
    const int quarter = sp.len / DEC_WAVES;
    const int k_begin = sp.lo_al + chunk * sp.len + wave * quarter;
    const int k_end = (k_begin + quarter < p + 1) ? k_begin + quarter : p + 1;   // one past the wavefront's last key
    const int p8 = p & ~7, pi_last = max_pages - 1;

    // the group's queries as the B operand: lane (r, j) holds head r, dims dk*32 + j*8 ..
    dec_bf16x8_t qop[DK];
#pragma unroll
    for (int dk = 0; dk < DK; ++dk) {
        dec_pack w;
        w.u = make_uint4(0, 0, 0, 0);
        if (r < G && dk * 32 + j * 8 < D)
            w.u = *reinterpret_cast<const uint4*>(q + (int64_t)t * ldq + (int64_t)(kvh * G + r) * D + dk * 32 + j * 8);
        qop[dk] = w.b;
    }
    dec_f32x4_t o[DT];
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) o[dd] = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, lsum = 0.f;   // m is in base-2 units: the maximum of s * scale * log2(e)
    const float scale_log2 = scale * 1.4426950408889634f;

    for (int base = k_begin; base < k_end; base += DEC_BLOCK) {
        // ---- all loads of the block first, in straight-line code: the six table lookups, then keys
        // (4 tiles x DK) and values (DT x 2) from addresses clamped into the sequence and the pool.  What
        // must not count is masked afterwards; with a branch around a load the compiler would wait for it
        // on the spot, one tile after the other.
        dec_pack kop[4][DK], vop[DT][2];
        int kpage[4], kslot[4], vpage[2], vslot[2];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const int key = base + (tt / 2) * 32 + (r / 4) * 8 + (tt % 2) * 4 + (r % 4);
            const int kc = key < p ? key : p;
            int pi = ps_shift >= 0 ? kc >> ps_shift : kc / ps;
            kslot[tt] = kc - pi * ps;
            kpage[tt] = bt[pi < pi_last ? pi : pi_last];
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int key0 = base + b * 32 + j * 8;
            const int kc = key0 < p8 ? key0 : p8;
            int pi = ps_shift >= 0 ? kc >> ps_shift : kc / ps;
            vslot[b] = kc - pi * ps;
            vpage[b] = bt[pi < pi_last ? pi : pi_last];
        }
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const int page = (unsigned)kpage[tt] < (unsigned)num_pages ? kpage[tt] : 0;   // a window may have freed it
            const zi_bf16* kr = kcache + (((int64_t)page * nkv + kvh) * ps + kslot[tt]) * D;
#pragma unroll
            for (int dk = 0; dk < DK; ++dk)
                kop[tt][dk].u = *reinterpret_cast<const uint4*>(kr + ((D % 32 == 0 || dk * 32 + j * 8 < D) ? dk * 32 + j * 8 : 0));
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int page = (unsigned)vpage[b] < (unsigned)num_pages ? vpage[b] : 0;
            const zi_bf16* vr = vcache + (((int64_t)page * nkv + kvh) * D + r) * ps + vslot[b];
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) vop[dd][b].u = *reinterpret_cast<const uint4*>(vr + (int64_t)dd * 16 * ps);
        }
        if (D % 32 != 0) {   // the padding of the last k-step must be zero: the query is, but 0 * NaN is not
            const unsigned keep = (DK - 1) * 32 + j * 8 < D ? ~0u : 0u;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                uint4& u = kop[tt][DK - 1].u;
                u.x &= keep; u.y &= keep; u.z &= keep; u.w &= keep;
            }
        }
        // Keys outside [lo, p] get the score -inf below, whatever was loaded for them.  Their values
        // must be zero, since 0 * NaN is NaN: slots outside the range may hold anything.
        if (base < sp.lo || base + DEC_BLOCK > k_end) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int key0 = base + b * 32 + j * 8;
                unsigned keep[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int ka = key0 + 2 * e, kb2 = ka + 1;
                    keep[e] = ((ka >= sp.lo && ka < k_end) ? 0xffffu : 0u) | ((kb2 >= sp.lo && kb2 < k_end) ? 0xffff0000u : 0u);
                }
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) {
                    uint4& u = vop[dd][b].u;
                    u.x &= keep[0]; u.y &= keep[1]; u.z &= keep[2]; u.w &= keep[3];
                }
            }
        }
        // ---- scores of 64 keys for this lane's head
        dec_f32x4_t s[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            s[tt] = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dk = 0; dk < DK; ++dk)
                s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[tt][dk].b, qop[dk], s[tt], 0, 0, 0);
        }
        // softmax in base 2: t = s * scale * log2(e), p = 2^(t - m)
        const bool whole = base >= sp.lo && base + DEC_BLOCK <= k_end;
        float mx = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = base + (tt / 2) * 32 + j * 8 + (tt % 2) * 4 + e;
                const float v = (whole || (key >= sp.lo && key < k_end)) ? s[tt][e] * scale_log2 : -INFINITY;
                s[tt][e] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_use);      // 2^(-inf) = 0 before the first key
        m = m_new;
        float psum = 0.f;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[tt][e] = __builtin_amdgcn_exp2f(s[tt][e] - m_use);   // 0 for keys not seen
                psum += s[tt][e];
            }
        dec_pack pb[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            pb[b].u.x = zi_pack_bf16x2(s[2 * b][0], s[2 * b][1]);
            pb[b].u.y = zi_pack_bf16x2(s[2 * b][2], s[2 * b][3]);
            pb[b].u.z = zi_pack_bf16x2(s[2 * b + 1][0], s[2 * b + 1][1]);
            pb[b].u.w = zi_pack_bf16x2(s[2 * b + 1][2], s[2 * b + 1][3]);
        }
        lsum = lsum * corr + psum;
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) {
            o[dd][0] *= corr; o[dd][1] *= corr; o[dd][2] *= corr; o[dd][3] *= corr;
#pragma unroll
            for (int b = 0; b < 2; ++b)
                o[dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[dd][b].b, pb[b].b, o[dd], 0, 0, 0);
        }
    }
    // ---- merge the four wavefronts: head r's (m, l) and this lane's outputs
    lsum += __shfl_xor(lsum, 16, ZI_WAVE);
    lsum += __shfl_xor(lsum, 32, ZI_WAVE);
    if (j == 0) {
        sm[wave][r] = m;
        sl[wave][r] = lsum;
    }
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) so[wave][dd][lane] = o[dd];
    __syncthreads();
    float M = sm[0][r];
#pragma unroll
    for (int w = 1; w < DEC_WAVES; ++w) M = fmaxf(M, sm[w][r]);
    float a[DEC_WAVES], L = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) {
        a[w] = (sm[w][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sm[w][r] - M);
        L += a[w] * sl[w][r];
    }
    const bool final = sp.count == 1;
    const float inv = final ? 1.f / L : 1.f;
    const int64_t slot = ((int64_t)x * nh + kvh * G + r) * DEC_MAXC + chunk;
    for (int dd = wave; dd < DT; dd += DEC_WAVES) {
        dec_f32x4_t acc = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const dec_f32x4_t v = so[w][dd][lane];
            acc[0] += a[w] * v[0]; acc[1] += a[w] * v[1]; acc[2] += a[w] * v[2]; acc[3] += a[w] * v[3];
        }
        if (r >= G) continue;
        if (final) {
            uint2 wv;
            wv.x = zi_pack_bf16x2(acc[0] * inv, acc[1] * inv);
            wv.y = zi_pack_bf16x2(acc[2] * inv, acc[3] * inv);
            *reinterpret_cast<uint2*>(out + (int64_t)t * ldo + (int64_t)(kvh * G + r) * D + dd * 16 + j * 4) = wv;
        } else {
            *reinterpret_cast<dec_f32x4_t*>(part_o + slot * D + dd * 16 + j * 4) = acc;
        }
    }
    if (!final && wave == 0 && j == 0 && r < G) {
        part_ml[slot * 2] = M;
        part_ml[slot * 2 + 1] = L;
    }
}

// Merge the chunks of one (token, head): out = sum_c e^(m_c - M) o_c / sum_c e^(m_c - M) l_c.
__global__ void __launch_bounds__(ZI_WAVE)
attention_decode_merge_kernel(zi_bf16* __restrict__ out, int64_t ldo, const float* __restrict__ part_o,
                              const float* __restrict__ part_ml, const int32_t* __restrict__ tok_index,
                              const int32_t* __restrict__ tok_pos, int nh, int D, int window, int max_chunks) {
    const int x = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int t = tok_index ? tok_index[x] : x;
    const DecSplit sp = dec_split(tok_pos[t], window);
    if (sp.count == 1 || sp.count > max_chunks) return;
    const int64_t slot0 = ((int64_t)x * nh + h) * DEC_MAXC;
    // chunk c's (m, l) sit in lane c
    const float mc = lane < sp.count ? part_ml[(slot0 + lane) * 2] : -INFINITY;
    const float lc = lane < sp.count ? part_ml[(slot0 + lane) * 2 + 1] : 0.f;
    const float M = zi_wave_max(mc);
    const float wc = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - M);   // maxima are in base-2 units
    float L = 0.f, acc[2] = {0.f, 0.f};
    for (int c0 = 0; c0 < sp.count; c0 += 8) {
        float po[8][2];   // eight chunks' loads are issued before the first is used
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int v = 0; v < 2; ++v)
                po[c][v] = (c0 + c < sp.count && lane + v * ZI_WAVE < D)
                               ? part_o[(slot0 + c0 + c) * D + lane + v * ZI_WAVE] : 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float w = __shfl(wc, (c0 + c) & (ZI_WAVE - 1), ZI_WAVE);   // 0 for chunks past the count
            L += w * __shfl(lc, (c0 + c) & (ZI_WAVE - 1), ZI_WAVE);
            acc[0] += w * po[c][0];
            acc[1] += w * po[c][1];
        }
    }
    const float inv = 1.f / L;
#pragma unroll
    for (int v = 0; v < 2; ++v)
        if (lane + v * ZI_WAVE < D) zi_store(out + (int64_t)t * ldo + (int64_t)h * D + lane + v * ZI_WAVE, acc[v] * inv);
}

// Floats of workspace the split kernel needs for n tokens.
extern "C" int64_t zi_attention_decode_workspace(int n, int nh, int d) {
    return (int64_t)n * nh * DEC_MAXC * (d + 2);
}

// Chunks the launch must cover when no token sees more than `keys` keys (position + 1, or the window).
extern "C" int zi_attention_decode_chunks(int keys) {
    if (keys < 1) keys = 1;
    // the range is widened down to a multiple of 8: up to 7 more keys.  Past DEC_CHUNK * DEC_MAXC keys
    // the chunks grow and their number drops again, but a token with fewer keys may still need them all.
    if (keys + 7 > DEC_CHUNK * DEC_MAXC) return DEC_MAXC;
    return dec_split(keys - 1 + 7, 0).count;
}

// 1 when the shape is this kernel's, else 0.
extern "C" int zi_attention_decode_supported(int dt, int nh, int nkv, int d, int page_size) {
    if (dt != ZI_BF16 || nkv <= 0 || nh <= 0 || nh % nkv) return 0;
    const int G = nh / nkv;
    return d >= 16 && d <= 128 && d % 16 == 0 && G <= 16 && page_size > 0 && page_size % 8 == 0;
}

extern "C" int zi_attention_decode(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo,
                                   const void* kcache, const void* vcache, const int32_t* tok_index,
                                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables,
                                   int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window,
                                   float scale, int max_chunks, float* workspace, int64_t workspace_floats,
                                   hipStream_t stream) {
    ZI_REQUIRE(zi_attention_decode_supported(dt, nh, nkv, d, page_size),
               "attention_decode: unsupported shape (bfloat16, head_dim a multiple of 16 up to 128, group <= 16, "
               "page size %% 8 == 0): dtype %d heads %d kv_heads %d head_dim %d page %d", dt, nh, nkv, d, page_size);
    ZI_REQUIRE(n_idx >= 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode: bad sizes");
    ZI_REQUIRE(max_chunks >= 1 && max_chunks <= DEC_MAXC, "attention_decode: max_chunks %d outside 1..%d", max_chunks,
               DEC_MAXC);
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldo >= (int64_t)nh * d && ldq % 8 == 0 && ldo % 4 == 0,
               "attention_decode: bad row stride");
    ZI_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 && ((uintptr_t)kcache % 16) == 0 &&
                   ((uintptr_t)vcache % 16) == 0,
               "attention_decode: q, out and the caches must be aligned to 16 bytes");
    ZI_REQUIRE(nkv <= 65535 && nh <= 65535, "attention_decode: too many heads");
    if (n_idx == 0) return 0;
    ZI_REQUIRE(max_chunks == 1 || (workspace && workspace_floats >= zi_attention_decode_workspace(n_idx, nh, d) &&
                                   ((uintptr_t)workspace % 16) == 0),
               "attention_decode: workspace of %lld floats is too small or not aligned", (long long)workspace_floats);
    float* po = workspace;
    float* pml = workspace ? workspace + (int64_t)n_idx * nh * DEC_MAXC * d : nullptr;
    const dim3 grid(n_idx, nkv, max_chunks);
    const int G = nh / nkv;
#define ZI_DEC(DD)                                                                                                   \
    attention_decode_kernel<DD><<<grid, DEC_WAVES * ZI_WAVE, 0, stream>>>(                                            \
        (zi_bf16*)out, ldo, po, pml, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache,         \
        tok_index, tok_seq, tok_pos, block_tables, max_pages, num_pages, nh, nkv, G, page_size, window, scale,       \
        max_chunks)
    switch (d) {
        case 16: ZI_DEC(16); break;
        case 32: ZI_DEC(32); break;
        case 48: ZI_DEC(48); break;
        case 64: ZI_DEC(64); break;
        case 80: ZI_DEC(80); break;
        case 96: ZI_DEC(96); break;
        case 112: ZI_DEC(112); break;
        default: ZI_DEC(128); break;
    }
#undef ZI_DEC
    if (max_chunks > 1)
        attention_decode_merge_kernel<<<dim3(n_idx, nh), ZI_WAVE, 0, stream>>>((zi_bf16*)out, ldo, po, pml, tok_index,
                                                                              tok_pos, nh, d, window, max_chunks);
    return zi_check_launch("attention_decode");
}
