// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for few rows of x (M <= 64): the decode-time
// matrix product, bound by the one pass over the weights.
//
// bfloat16 x and w, float32 accumulation on the matrix cores
// (v_mfma_f32_16x16x32_bf16), output bfloat16 or float32.  A workgroup of four
// wavefronts owns a tile of 16 weight rows; the wavefronts take the k-blocks of 128
// in turn and their sums are added through LDS in a fixed order.  Small weight
// matrices are additionally cut along k over several workgroups (gridDim.y) so
// that enough loads are in flight to fill HBM; those write float32 partials that a
// second kernel adds, again in a fixed order.  The cut depends on N and K only, so
// a row's result does not depend on how many rows ride along.
//
// Operand layout.  For one MFMA the A operand is a 16 x 32 tile of w (lane l: row
// l%16, eight consecutive k) and the B operand the matching 32 x 16 tile of x^T
// (lane l: row l%16 of x, the same eight k).  Within a k-block of 128 the lane group
// j = l/16 reads k in [32j, 32j+32) as four 16-byte loads and MFMA i consumes load i:
// a permutation of k that both operands share, which turns every row's reads into
// 256 contiguous bytes per k-block.
#include "zi_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define SK_ROWS 16
#define SK_KB 128
#define SK_WAVES 4

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4& v) {
    union { uint4 u; bf16x8_t b; } c;
    c.u = v;
    return c.b;
}

template <int MT>
__global__ void __launch_bounds__(SK_WAVES* ZI_WAVE)
gemm_skinny_kernel(void* __restrict__ out, int out_f32, float* __restrict__ partial,
                   const zi_bf16* __restrict__ x, const zi_bf16* __restrict__ w, const zi_bf16* __restrict__ bias,
                   int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int kb_per_split) {
    __shared__ f32x4_t red[SK_WAVES][MT][ZI_WAVE];
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int n0 = blockIdx.x * SK_ROWS;
    const int nrow = (n0 + r < N) ? n0 + r : N - 1;
    const zi_bf16* wrow = w + (int64_t)nrow * ldw + j * 32;
    const zi_bf16* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;
        xrow[t] = x + (int64_t)(m < M ? m : M - 1) * ldx + j * 32;
    }
    f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const int kb_total = (K + SK_KB - 1) / SK_KB;
    const int kb_lo = blockIdx.y * kb_per_split;
    const int kb_hi = (kb_lo + kb_per_split < kb_total) ? kb_lo + kb_per_split : kb_total;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (int kb = kb_lo + wave; kb < kb_hi; kb += SK_WAVES) {
        const int k0 = kb * SK_KB;
        uint4 a[4], b[MT][4];
        if (k0 + SK_KB <= K) {
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const uint4*>(wrow + k0 + i * 8);
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) b[t][i] = *reinterpret_cast<const uint4*>(xrow[t] + k0 + i * 8);
        } else {   // the last, partial k-block (K is a multiple of 8)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool in = k0 + j * 32 + i * 8 < K;
                a[i] = in ? *reinterpret_cast<const uint4*>(wrow + k0 + i * 8) : zero;
#pragma unroll
                for (int t = 0; t < MT; ++t) b[t][i] = in ? *reinterpret_cast<const uint4*>(xrow[t] + k0 + i * 8) : zero;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[i]), as_bf16x8(b[t][i]), acc[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
    __syncthreads();
    // wave t of the workgroup finishes row tile t of x: C[n = (lane/16)*4 + e][m = lane%16]
    for (int t = wave; t < MT; t += SK_WAVES) {
        f32x4_t s = red[0][t][lane];
#pragma unroll
        for (int q = 1; q < SK_WAVES; ++q) {
            const f32x4_t o = red[q][t][lane];
            s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
        }
        const int m = t * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = n0 + j * 4 + e;
            if (n >= N) continue;
            if (partial) {
                partial[((int64_t)blockIdx.y * M + m) * N + n] = s[e];
            } else {
                const float v = s[e] + (bias ? zi_load(bias + n) : 0.f);
                if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = v;
                else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, v);
            }
        }
    }
}

// out[m,n] = sum_s partial[s,m,n] + bias[n], splits added in rising order.
__global__ void gemm_skinny_reduce_kernel(void* __restrict__ out, int out_f32, const float* __restrict__ partial,
                                          const zi_bf16* __restrict__ bias, int M, int N, int64_t ldo, int splits) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)M * N) return;
    const int m = (int)(i / N), n = (int)(i % N);
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += partial[(int64_t)k * M * N + i];
    if (bias) s += zi_load(bias + n);
    if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = s;
    else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, s);
}

// How the k dimension is cut for a weight matrix [N, K]: (splits, k-blocks per split).
static void skinny_plan(int N, int K, int* splits, int* kb_per_split) {
    const int tiles = (N + SK_ROWS - 1) / SK_ROWS;
    const int kb_total = (K + SK_KB - 1) / SK_KB;
    int s = (2048 + tiles * SK_WAVES - 1) / (tiles * SK_WAVES);      // aim at 2048 wavefronts
    const int most = kb_total / SK_WAVES > 0 ? kb_total / SK_WAVES : 1;   // keep every wavefront busy
    if (s > most) s = most;
    if (s < 1) s = 1;
    int per = (kb_total + s - 1) / s;
    s = (kb_total + per - 1) / per;
    *splits = s;
    *kb_per_split = per;
}

extern "C" int zi_gemm_skinny_supported(int M, int N, int K, int64_t ldx, int64_t ldw) {
    return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

// Floats of workspace for the split partials (0 when the product is not split).
extern "C" int64_t zi_gemm_skinny_workspace(int M, int N, int K) {
    int s, per;
    skinny_plan(N, K, &s, &per);
    return s > 1 ? (int64_t)s * M * N : 0;
}

extern "C" int zi_gemm_skinny(void* out, int out_dt, const void* x, const void* w, const void* bias, int M, int N,
                              int K, int64_t ldx, int64_t ldw, int64_t ldo, float* workspace,
                              int64_t workspace_floats, hipStream_t stream) {
    ZI_REQUIRE(zi_gemm_skinny_supported(M, N, K, ldx, ldw),
               "gemm_skinny: unsupported sizes M=%d N=%d K=%d (1 <= M <= 64, K and row strides multiples of 8)", M, N, K);
    ZI_REQUIRE(out_dt == ZI_F32 || out_dt == ZI_BF16, "gemm_skinny: unknown output dtype %d", out_dt);
    ZI_REQUIRE(ldx >= K && ldw >= K && ldo >= N, "gemm_skinny: leading dimension too small");
    ZI_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny: x and w must be 16-byte aligned");
    int splits, per;
    skinny_plan(N, K, &splits, &per);
    float* partial = nullptr;
    if (splits > 1) {
        ZI_REQUIRE(workspace && workspace_floats >= (int64_t)splits * M * N,
                   "gemm_skinny: workspace of %lld floats is too small (%lld needed)", (long long)workspace_floats,
                   (long long)splits * M * N);
        partial = workspace;
    }
    const dim3 grid((N + SK_ROWS - 1) / SK_ROWS, splits);
    const int mt = (M + 15) / 16;
#define ZI_SK(MT)                                                                                                   \
    gemm_skinny_kernel<MT><<<grid, SK_WAVES * ZI_WAVE, 0, stream>>>(out, out_dt == ZI_F32, partial, (const zi_bf16*)x, \
                                                                    (const zi_bf16*)w, (const zi_bf16*)bias, M, N, K, \
                                                                    ldx, ldw, ldo, per)
    switch (mt) {
        case 1: ZI_SK(1); break;
        case 2: ZI_SK(2); break;
        case 3: ZI_SK(3); break;
        default: ZI_SK(4); break;
    }
#undef ZI_SK
    if (splits > 1) {
        const int64_t total = (int64_t)M * N;
        gemm_skinny_reduce_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(out, out_dt == ZI_F32, partial,
                                                                                  (const zi_bf16*)bias, M, N, ldo, splits);
    }
    return zi_check_launch("gemm_skinny");
}
