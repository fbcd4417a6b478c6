// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for up to 256 rows of x: the decode-time matrix products, bound by the
// one pass over the weights.  This file holds their entry points, the cut's bookkeeping and the kernel that
// adds partial sums; the product kernels are in gemm_mid.hip (up to 128 rows: x staged in LDS, a workgroup's
// wavefronts take 16 weight rows each, the cut over workgroups balanced over the compute units) and in
// gemm_rows32.hip (more rows, and the SwiGLU epilogue from 65 rows on: 32 weight rows a wavefront).
//
// When the weight matrix gives too few workgroups the k dimension is cut over several of them (gridDim.y
// "splits"); those write float32 partial sums [split][M][N] that the consumer adds in rising order (the next
// norm, the rotary kernel, the SwiGLU kernel, or the reduce kernel here).  The cut depends on N and K only,
// so a row's result does not depend on how many rows ride along.
//
// Epilogues: plain (bias, bfloat16 or float32 out), partial sums, and SwiGLU: when the weight rows are gate
// and up rows interleaved in blocks of 8 (tile = 8 gate rows, then the 8 up rows of the same columns), the
// tile's lanes exchange halves and write act = up * gate / (1 + exp(-gate))
// (reference: src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).
//
// A kernel that kept x in registers and cut k over a workgroup's wavefronts served up to 16 rows before the
// other one's cut was balanced; since then it was slower at every size from one row on (1.5B gate/up at 8 rows
// 12.9 against 11.7 us, 32B gate/up 111 against 95 us) and is gone.
#include "zi_common.h"
#include "zi_api.h"

#define SK_MODE_PLAIN 0
#define SK_MODE_PARTIAL 1
#define SK_MODE_SWIGLU 2

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

#define SK_MAX_ROWS 256
#define SK_MID_MAX_ROWS 128        // up to here the kernels of gemm_mid.hip, beyond gemm_rows32.hip
#define SK_MID_MAX_ROWS_SWIGLU 64  // ... with the SwiGLU epilogue (measured: see gemm_rows32.hip)

extern "C" int zi_gemm_skinny_supported(int M, int N, int K, int64_t ldx, int64_t ldw) {
    return M >= 1 && M <= SK_MAX_ROWS && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

// most rows the products take
extern "C" int zi_gemm_skinny_max_rows() { return SK_MAX_ROWS; }

// 1 when these kernels are the faster way to partial sums than the library's product of the same operands, as
// measured: always up to 128 rows; beyond, for large weights with at least twice as many columns as rows (a down
// projection: 7B sizes at 256 rows 71 against 126 us, 32B 136 against 263), not for square ones (an output
// projection: 7B at 256 rows 24.6 against 16.9 us), and not for small ones (1.5B down at 256 rows 25.5 against
// 31 us, which the 25 MB of partial sums that the next kernel then adds take back: the decode step of 256
// requests got 3 % slower with it).
extern "C" int zi_gemm_skinny_pays(int M, int N, int K) {
    if (M <= SK_MID_MAX_ROWS) return 1;
    return M <= SK_MAX_ROWS && (int64_t)K >= 2 * (int64_t)N && (int64_t)N * K >= ((int64_t)1 << 25);
}

// The product kernel (gemm_mid.hip): its cut and its launch.
void zi_gemm_mid_plan(int N, int K, int* splits, int* kb_per_split, int* waves);
int zi_gemm_mid_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                       int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream);

void zi_gemm_rows32_plan(int N, int K, int many_rows, int whole, int* splits, int* kb_per_split, int* waves);
int zi_gemm_rows32_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                          int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream);

static bool sk_rows32(int M, int mode) { return M > (mode == SK_MODE_SWIGLU ? SK_MID_MAX_ROWS_SWIGLU : SK_MID_MAX_ROWS); }

// Splits of k for a weight matrix [N, K]: the leading dimension of the partial sums.  A function of N and K and
// of which of the two kernels the rows go to (up to 128, or more).
extern "C" int zi_gemm_skinny_splits(int M, int N, int K) {
    int s, per, waves;
    if (sk_rows32(M, SK_MODE_PARTIAL)) zi_gemm_rows32_plan(N, K, M > 128, 0, &s, &per, &waves);
    else zi_gemm_mid_plan(N, K, &s, &per, &waves);
    return s;
}

// Floats of workspace for the split partials (0 when the product is not split).
extern "C" int64_t zi_gemm_skinny_workspace(int M, int N, int K) {
    const int s = zi_gemm_skinny_splits(M, N, K);
    return s > 1 ? (int64_t)s * M * N : 0;
}

// mode 0: out[M,N] (+ bias), reduced through `workspace` when the product is split.
// mode 1: out = float32 partial sums [splits][M][N] (no bias; splits from zi_gemm_skinny_splits).
// mode 2: w holds gate and up rows interleaved in blocks of 8; out[M, N/2] (bfloat16) =
//         up * silu(gate); only for products that are not split.
extern "C" int zi_gemm_skinny(void* out, int out_dt, int mode, const void* x, const void* w, const void* bias, int M,
                              int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, float* workspace,
                              int64_t workspace_floats, hipStream_t stream) {
    ZI_REQUIRE(zi_gemm_skinny_supported(M, N, K, ldx, ldw),
               "gemm_skinny: unsupported sizes M=%d N=%d K=%d (1 <= M <= 256, K and row strides multiples of 8)", M, N, K);
    ZI_REQUIRE(out_dt == ZI_F32 || out_dt == ZI_BF16, "gemm_skinny: unknown output dtype %d", out_dt);
    ZI_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny: unknown mode %d", mode);
    ZI_REQUIRE(ldx >= K && ldw >= K, "gemm_skinny: leading dimension too small");
    ZI_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny: x and w must be 16-byte aligned");
    int splits, per, waves;
    const bool rows32 = sk_rows32(M, mode);
    if (rows32) zi_gemm_rows32_plan(N, K, M > 128, mode == SK_MODE_SWIGLU, &splits, &per, &waves);
    else zi_gemm_mid_plan(N, K, &splits, &per, &waves);
    void* dst = out;
    int kmode = mode;
    if (mode == SK_MODE_PLAIN) {
        ZI_REQUIRE(ldo >= N, "gemm_skinny: leading dimension of out too small");
        if (splits > 1) {
            ZI_REQUIRE(workspace && workspace_floats >= (int64_t)splits * M * N,
                       "gemm_skinny: workspace of %lld floats is too small (%lld needed)", (long long)workspace_floats,
                       (long long)splits * M * N);
            dst = workspace;
            kmode = SK_MODE_PARTIAL;
        }
    } else if (mode == SK_MODE_PARTIAL) {
        ZI_REQUIRE(out_dt == ZI_F32, "gemm_skinny: partial sums are float32");
    } else {
        ZI_REQUIRE(splits == 1, "gemm_skinny: the SwiGLU epilogue needs a product that is not split (N=%d K=%d has %d)",
                   N, K, splits);
        ZI_REQUIRE(N % 16 == 0 && out_dt == ZI_BF16 && ldo >= N / 2,
                   "gemm_skinny: the SwiGLU epilogue needs N %% 16 == 0 and a bfloat16 out of N/2 columns");
    }
    const zi_bf16* b = kmode == SK_MODE_PLAIN ? (const zi_bf16*)bias : nullptr;
    // four columns go out as one store when every row of the destination keeps them aligned
    int vec_out;
    if (kmode == SK_MODE_PARTIAL) vec_out = N % 4 == 0 && ((uintptr_t)dst % 16) == 0;
    else if (kmode == SK_MODE_SWIGLU) vec_out = ldo % 4 == 0 && ((uintptr_t)dst % 8) == 0;
    else vec_out = ldo % 4 == 0 && ((uintptr_t)dst % (out_dt == ZI_F32 ? 16 : 8)) == 0;
    const int of32 = out_dt == ZI_F32;
    const int rc = (rows32 ? zi_gemm_rows32_launch : zi_gemm_mid_launch)(dst, of32, kmode, (const zi_bf16*)x, (const zi_bf16*)w, b,
                                                                         M, N, K, ldx, ldw, ldo, vec_out, stream);
    if (rc) return rc;
    if (mode == SK_MODE_PLAIN && splits > 1) {
        const int64_t total = (int64_t)M * N;
        gemm_skinny_reduce_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(out, of32, workspace,
                                                                                  (const zi_bf16*)bias, M, N, ldo, splits);
    }
    return zi_check_launch("gemm_skinny");
}

// out[m,n] = sum_s sums[s,m,n] + bias[n] for float32 sums [splits][M][N], added in rising order.
extern "C" int zi_reduce_splits(void* out, int out_dt, const float* sums, const void* bias, int M, int N, int64_t ldo,
                                int splits, hipStream_t stream) {
    ZI_REQUIRE(M >= 0 && N > 0 && splits >= 1 && ldo >= N, "reduce_splits: bad sizes");
    ZI_REQUIRE(out_dt == ZI_F32 || out_dt == ZI_BF16, "reduce_splits: unknown output dtype %d", out_dt);
    if (M == 0) return 0;
    const int64_t total = (int64_t)M * N;
    gemm_skinny_reduce_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(out, out_dt == ZI_F32, sums,
                                                                              (const zi_bf16*)bias, M, N, ldo, splits);
    return zi_check_launch("reduce_splits");
}
