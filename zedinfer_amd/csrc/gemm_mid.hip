// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for 17..64 rows of x: decoding at larger batches, still bound
// by the one pass over the weights.
//
// A workgroup of four wavefronts owns 64 weight rows (16 a wavefront) and a range of k.  It walks its
// k-blocks of 128: the block's slice of x (up to 64 rows x 128 values) is staged in LDS once for the four
// wavefronts, each wavefront reads its own 16 weight rows straight from memory into matrix-core operands
// (v_mfma_f32_16x16x32_bf16, float32 accumulation) and keeps the sums of its 16 x M outputs in registers,
// so nothing is added across wavefronts.  The next block's weights and x travel while the current one is
// worked on.  The k dimension is cut over gridDim.y workgroups when N alone gives too few of them; those
// leave float32 partial sums [split][M][N] that the consumer adds in rising order.  The cut depends on N
// and K only.  Epilogues as in the few-rows kernel: plain (bias), partial sums, SwiGLU over gate/up rows
// interleaved in blocks of 8.
#include "zi_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 gm_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float gm_f32x4_t;

#define GM_WAVES 4
#define GM_ROWS 64          // weight rows per workgroup
#define GM_KB 128
#define GM_XS (GM_KB + 8)   // LDS row stride of the x slice, in elements
#define GM_TARGET_WGS 384

#define GM_MODE_PLAIN 0
#define GM_MODE_PARTIAL 1
#define GM_MODE_SWIGLU 2

union gm_pack {
    uint4 u;
    gm_bf16x8_t b;
};

template <int MT>
__global__ void __launch_bounds__(GM_WAVES* ZI_WAVE)
gemm_mid_kernel(void* __restrict__ out, int mode, int out_f32, const zi_bf16* __restrict__ x,
                const zi_bf16* __restrict__ w, const zi_bf16* __restrict__ bias, int M, int N, int K, int64_t ldx,
                int64_t ldw, int64_t ldo, int kb_per_split, int vec_out) {
    __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 16 * GM_XS];
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int split = blockIdx.y;
    const int kb_total = (K + GM_KB - 1) / GM_KB;
    const int kb_lo = split * kb_per_split;
    const int kb_hi = (kb_lo + kb_per_split < kb_total) ? kb_lo + kb_per_split : kb_total;
    const int n0 = blockIdx.x * GM_ROWS + wave * 16;
    const int nrow = (n0 + r < N) ? n0 + r : N - 1;
    const zi_bf16* wrow = w + (int64_t)nrow * ldw + j * 8;

    // what this thread stages of a block's x slice: MT pieces of 16 bytes (row srow + 16 * t, piece spc)
    const int srow = tid / 16, spc = tid % 16;
    uint4 a_cur[4], a_next[4], xr[MT];
    auto fetch = [&](uint4 (&a)[4], int kb) {
        const int k0 = kb * GM_KB;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            a[c] = (k0 + c * 32 + j * 8 < K) ? *reinterpret_cast<const uint4*>(wrow + k0 + c * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + srow;
            xr[t] = (m < M && k0 + spc * 8 < K) ? *reinterpret_cast<const uint4*>(x + (int64_t)m * ldx + k0 + spc * 8)
                                                : make_uint4(0, 0, 0, 0);
        }
    };
    auto stash = [&](int b) {
#pragma unroll
        for (int t = 0; t < MT; ++t) *reinterpret_cast<uint4*>(&xs[b][(t * 16 + srow) * GM_XS + spc * 8]) = xr[t];
    };
    gm_f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};

    fetch(a_cur, kb_lo);
    stash(0);
    __syncthreads();
    int cur = 0;
    for (int kb = kb_lo; kb < kb_hi; ++kb, cur ^= 1) {
        const bool has_next = kb + 1 < kb_hi;
        if (has_next) fetch(a_next, kb + 1);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            gm_pack a;
            a.u = a_cur[c];
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                gm_pack b;
                b.u = *reinterpret_cast<const uint4*>(&xs[cur][(t * 16 + r) * GM_XS + c * 32 + j * 8]);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, acc[t], 0, 0, 0);
            }
        }
        if (has_next) {
            stash(cur ^ 1);
#pragma unroll
            for (int c = 0; c < 4; ++c) a_cur[c] = a_next[c];
        }
        __syncthreads();
    }
    // C[n = n0 + j*4 + e][m = t*16 + r]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        gm_f32x4_t s = acc[t];
        const int m = t * 16 + r;
        if (mode == GM_MODE_SWIGLU) {
            // lanes j = 0,1 hold gate rows j*4 + e, lanes j = 2,3 the up rows of the same columns
            gm_f32x4_t up;
            up[0] = __shfl_xor(s[0], 32, ZI_WAVE); up[1] = __shfl_xor(s[1], 32, ZI_WAVE);
            up[2] = __shfl_xor(s[2], 32, ZI_WAVE); up[3] = __shfl_xor(s[3], 32, ZI_WAVE);
            if (j >= 2 || m >= M || n0 >= N) continue;
            const int col = (n0 / 16) * 8 + j * 4;     // N / 2 columns of output; N % 16 == 0
            float act[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) act[e] = up[e] * (s[e] / (1.f + expf(-s[e])));
            zi_bf16* dst = (zi_bf16*)out + (int64_t)m * ldo + col;
            if (vec_out) {
                uint2 pk;
                pk.x = zi_pack_bf16x2(act[0], act[1]);
                pk.y = zi_pack_bf16x2(act[2], act[3]);
                *reinterpret_cast<uint2*>(dst) = pk;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) zi_store(dst + e, act[e]);
            }
            continue;
        }
        if (m >= M) continue;
        const int nb = n0 + j * 4;
        if (nb + 3 < N && vec_out) {
            if (mode == GM_MODE_PARTIAL) {
                *reinterpret_cast<gm_f32x4_t*>((float*)out + ((int64_t)split * M + m) * N + nb) = s;
            } else {
                if (bias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) s[e] += zi_load(bias + nb + e);
                }
                if (out_f32) {
                    *reinterpret_cast<gm_f32x4_t*>((float*)out + (int64_t)m * ldo + nb) = s;
                } else {
                    uint2 pk;
                    pk.x = zi_pack_bf16x2(s[0], s[1]);
                    pk.y = zi_pack_bf16x2(s[2], s[3]);
                    *reinterpret_cast<uint2*>((zi_bf16*)out + (int64_t)m * ldo + nb) = pk;
                }
            }
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = nb + e;
            if (n >= N) continue;
            if (mode == GM_MODE_PARTIAL) {
                ((float*)out)[((int64_t)split * M + m) * N + n] = s[e];
            } else {
                const float v = s[e] + (bias ? zi_load(bias + n) : 0.f);
                if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = v;
                else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, v);
            }
        }
    }
}

// Splits of k and k-blocks per split for a weight matrix [N, K]: enough workgroups to fill the chip,
// at least two k-blocks a workgroup where K allows, at most 16 splits (what the consumers add at once).
void zi_gemm_mid_plan(int N, int K, int* splits, int* kb_per_split) {
    const int groups = (N + GM_ROWS - 1) / GM_ROWS;
    const int kb_total = (K + GM_KB - 1) / GM_KB;
    int s = (GM_TARGET_WGS + groups - 1) / groups;
    if (s > 16) s = 16;
    if (s > kb_total / 2) s = kb_total / 2;
    if (s < 1) s = 1;
    const int per = (kb_total + s - 1) / s;
    *kb_per_split = per;
    *splits = (kb_total + per - 1) / per;
}

// The launch; the checks are the caller's (zi_gemm_skinny).
int zi_gemm_mid_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                       int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream) {
    int splits, per;
    zi_gemm_mid_plan(N, K, &splits, &per);
    const dim3 grid((N + GM_ROWS - 1) / GM_ROWS, splits);
    const int mt = (M + 15) / 16;
#define ZI_GM(MT)                                                                                                  \
    gemm_mid_kernel<MT><<<grid, GM_WAVES * ZI_WAVE, 0, stream>>>(out, mode, out_f32, x, w, bias, M, N, K, ldx, ldw, \
                                                                 ldo, per, vec_out)
    switch (mt) {
        case 1: ZI_GM(1); break;
        case 2: ZI_GM(2); break;
        case 3: ZI_GM(3); break;
        default: ZI_GM(4); break;
    }
#undef ZI_GM
    return zi_check_launch("gemm_mid");
}
