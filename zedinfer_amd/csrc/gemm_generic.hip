// out[M,N] = x[M,K] . w[N,K]^T (+ bias[N]): the plain matrix product.
//
// Every storage type pairing (float32 or bfloat16 for x, w, bias and out), every
// size; products and sums in float32 FMA, no matrix cores, no reduced-precision
// mode.  Each output element is one thread's sequential sum over k in rising
// order, so its value does not depend on M, on the tile it falls in or on the
// rest of the batch.  This is the matrix product of the float32 path, and of
// any layer whose checkpoint tensor is stored in 32-bit.
// (reference: src/backend/ops/linear/cpu/linear_cpu.cpp:26-85.)
#include "zi_common.h"
#include "zi_api.h"

#define GT 64   // output tile edge
#define GK 16   // k step

template <typename TX, typename TW, typename TB, typename TO>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(TO* __restrict__ out, const TX* __restrict__ x, const TW* __restrict__ w,
                    const TB* __restrict__ bias, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo) {
    __shared__ float xs[GK][GT + 4];
    __shared__ float ws[GK][GT + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int64_t m0 = (int64_t)blockIdx.y * GT, n0 = (int64_t)blockIdx.x * GT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    const int lr = tid / 4, lk = (tid % 4) * 4;  // this thread loads row lr, k offsets lk..lk+3 of each tile
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int64_t m = m0 + lr, n = n0 + lr;
            xs[lk + i][lr] = (m < M && k < K) ? zi_load(x + m * ldx + k) : 0.f;
            ws[lk + i][lr] = (n < N && k < K) ? zi_load(w + n * ldw + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += zi_load(bias + n);
            zi_store(out + m * ldo + n, v);
        }
    }
}

extern "C" int zi_gemm_generic(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt,
                               const void* bias, int bias_dt, int M, int N, int K, int64_t ldx, int64_t ldw,
                               int64_t ldo, hipStream_t stream) {
    ZI_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    ZI_REQUIRE(ldx >= K && ldw >= K && ldo >= N, "gemm: leading dimension too small");
    if (M == 0) return 0;
    const dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    ZI_REQUIRE(grid.y <= 65535, "gemm: M=%d is too large for one launch", M);
    if (!bias) bias_dt = ZI_F32;
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(bias_dt, TB, ZI_DISPATCH_DTYPE(out_dt, TO, {
        gemm_generic_kernel<TX, TW, TB, TO><<<grid, 256, 0, stream>>>(
            (TO*)out, (const TX*)x, (const TW*)w, (const TB*)bias, M, N, K, ldx, ldw, ldo);
    }))));
    return zi_check_launch("gemm_generic");
}
