// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for 17..64 rows of x: decoding at larger batches, still bound
// by the one pass over the weights.
//
// A workgroup of four wavefronts owns 64 weight rows (16 a wavefront) and a range of k.  It walks its
// k-blocks of 128: the block's slice of x (up to 64 rows x 128 values) is staged in LDS once for the four
// wavefronts, each wavefront reads its own 16 weight rows straight from memory into matrix-core operands
// (v_mfma_f32_16x16x32_bf16, float32 accumulation) and keeps the sums of its 16 x M outputs in registers,
// so nothing is added across wavefronts.  The next block's weights and x travel while the current one is
// worked on (a ring of register buffers; loads are issued without branches so that they stay in
// flight).  The k dimension is cut over gridDim.y workgroups when N alone gives too few of them; those
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
#define GM_RING 3           // k-blocks of weights in flight per wavefront

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
    const zi_bf16* wrow_base = w + (int64_t)nrow * ldw;

    // what this thread stages of a block's x slice: MT pieces of 16 bytes (row srow + 16 * t, piece spc)
    const int srow = tid / 16, spc = tid % 16;
    // the weights of GM_RING k-blocks are in flight at once (a ring of register buffers); the x slice of
    // the next block is fetched while this one is worked on
    uint4 ring[GM_RING][4], xring[GM_RING][MT];
    // Loads are issued without branches (addresses are clamped into the matrix, what lies outside is
    // zeroed afterwards): only then does the compiler let several blocks' loads stay in flight.
    const int xm_last = M - 1;
    auto fetch = [&](uint4 (&a)[4], uint4 (&xr)[MT], int kb) {
        const int k0 = kb * GM_KB;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int k = k0 + c * 32 + j * 8;
            const uint4 v = *reinterpret_cast<const uint4*>(wrow_base + (k < K ? k : K - 8));
            a[c] = k < K ? v : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + srow, k = k0 + spc * 8;
            const uint4 v = *reinterpret_cast<const uint4*>(x + (int64_t)(m < M ? m : xm_last) * ldx + (k < K ? k : K - 8));
            xr[t] = (m < M && k < K) ? v : make_uint4(0, 0, 0, 0);
        }
    };
    auto stash = [&](const uint4 (&xr)[MT], int b) {
#pragma unroll
        for (int t = 0; t < MT; ++t) *reinterpret_cast<uint4*>(&xs[b][(t * 16 + srow) * GM_XS + spc * 8]) = xr[t];
    };
    gm_f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};

    // blocks kb_lo .. kb_lo + GM_RING - 2 are requested up front; block kb's x goes to LDS one iteration
    // before it is used, GM_RING - 2 iterations after it was requested
    const int kb_last = kb_hi - 1;    // requests past the last block fetch it again: no branch around a load
#pragma unroll
    for (int b = 0; b < GM_RING - 1; ++b) fetch(ring[b], xring[b], kb_lo + b < kb_hi ? kb_lo + b : kb_last);
    stash(xring[0], 0);
    __syncthreads();
    int cur = 0;
    for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += GM_RING) {
#pragma unroll
        for (int b = 0; b < GM_RING; ++b) {
            const int kb = kb0 + b;
            if (kb >= kb_hi) break;
            fetch(ring[(b + GM_RING - 1) % GM_RING], xring[(b + GM_RING - 1) % GM_RING],
                  kb + GM_RING - 1 < kb_hi ? kb + GM_RING - 1 : kb_last);
            // all of the block's x operands are read from LDS before the first product: the reads' latency
            // is paid once, not once per product
            gm_pack bb[4][MT];
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    bb[c][t].u = *reinterpret_cast<const uint4*>(&xs[cur][(t * 16 + r) * GM_XS + c * 32 + j * 8]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                gm_pack a;
                a.u = ring[b][c];
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, bb[c][t].b, acc[t], 0, 0, 0);
            }
            if (kb + 1 < kb_hi) stash(xring[(b + 1) % GM_RING], cur ^ 1);
            __syncthreads();
            cur ^= 1;
        }
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
    int s = (GM_TARGET_WGS + groups / 2) / groups;    // to the nearest: 280 groups are enough by themselves
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
