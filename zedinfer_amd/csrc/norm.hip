// RMSNorm, alone and fused with the residual add that precedes it.
//   y = w * x * rsqrt(mean(x^2) + eps)      (eps inside the root)
// (reference: src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:14-29; the fused
// form res += x; y = norm(res) * w at src/backend/ops/rms_norm/op.cpp:39-68).
// Sum of squares, rstd and the products are float32; one workgroup per row, so
// a row's result does not depend on which other rows are in the batch.
#include "zi_common.h"

#define NORM_THREADS 256

template <typename TX, typename TW, typename TO>
__global__ void rmsnorm_kernel(TO* __restrict__ out, const TX* __restrict__ x, const TW* __restrict__ w, int H,
                               int64_t ldx, int64_t ldo, float eps, float w_offset) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const TX* xr = x + row * ldx;
    TO* orow = out + row * ldo;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        const float v = zi_load(xr + j);
        ss += v * v;
    }
    ss = zi_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    for (int j = threadIdx.x; j < H; j += blockDim.x)
        zi_store(orow + j, (zi_load(w + j) + w_offset) * zi_load(xr + j) * rstd);
}

extern "C" int zi_rmsnorm(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt, int n, int hidden,
                          int64_t ldx, int64_t ldo, float eps, int add_one, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && ldx >= hidden && ldo >= hidden, "rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
    ZI_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        rmsnorm_kernel<TX, TW, TO><<<n, NORM_THREADS, 0, stream>>>((TO*)out, (const TX*)x, (const TW*)w, hidden, ldx,
                                                                   ldo, eps, add_one ? 1.f : 0.f);
    })));
    return zi_check_launch("rmsnorm");
}

// resid (float32, in place) += delta;  out = norm(resid) * w.  delta may come as `splits` partial
// sums (split s at delta + s * split_stride), which are added in rising order.
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(TO* __restrict__ out, float* __restrict__ resid, const TD* __restrict__ delta,
                                   int splits, int64_t split_stride, const TW* __restrict__ w, int H, float eps,
                                   float w_offset) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float* rr = resid + row * H;
    const TD* dr = delta + row * H;
    TO* orow = out + row * H;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float d = zi_load(dr + j);
        for (int s = 1; s < splits; ++s) d += zi_load(dr + s * split_stride + j);
        const float v = rr[j] + d;
        rr[j] = v;
        ss += v * v;
    }
    ss = zi_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    // Each thread re-reads only what it wrote itself.
    for (int j = threadIdx.x; j < H; j += blockDim.x) zi_store(orow + j, (zi_load(w + j) + w_offset) * rr[j] * rstd);
}

extern "C" int zi_add_rmsnorm(void* out, int out_dt, float* resid, const void* delta, int delta_dt, int splits,
                              int64_t split_stride, const void* w, int w_dt, int n, int hidden, float eps, int add_one,
                              hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
    ZI_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || split_stride >= (int64_t)n * hidden),
               "add_rmsnorm: bad partial sums (splits %d, stride %lld)", splits, (long long)split_stride);
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(delta_dt, TD, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        add_rmsnorm_kernel<TD, TW, TO><<<n, NORM_THREADS, 0, stream>>>((TO*)out, resid, (const TD*)delta, splits,
                                                                       split_stride, (const TW*)w, hidden, eps,
                                                                       add_one ? 1.f : 0.f);
    })));
    return zi_check_launch("add_rmsnorm");
}
