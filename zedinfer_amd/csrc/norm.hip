// RMSNorm, alone and fused with the residual add that precedes it.
//   y = w * x * rsqrt(mean(x^2) + eps)      (eps inside the root)
// (reference: src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:14-29; the fused
// form res += x; y = norm(res) * w at src/backend/ops/rms_norm/op.cpp:39-68).
// Sum of squares, rstd and the products are float32; one workgroup per row, so
// a row's result does not depend on which other rows are in the batch.
#include "zi_common.h"
#include "zi_api.h"

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

__device__ __forceinline__ float4 zi_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 zi_load4(const zi_bf16* p) {
    const uint2 r = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                       __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ void zi_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void zi_store4(zi_bf16* p, float4 v) {
    uint2 r;
    r.x = (uint32_t)zi_float_to_bf16(v.x) | ((uint32_t)zi_float_to_bf16(v.y) << 16);
    r.y = (uint32_t)zi_float_to_bf16(v.z) | ((uint32_t)zi_float_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = r;
}

// The same for rows of H = 4 * blockDim.x * IT values at most (H % 4 == 0): a thread owns IT groups of four
// consecutive values, loads everything it needs at once (up to 16 splits) and keeps the sums in
// registers, so the row is read once and nothing is read back.
template <typename TD, typename TW, typename TO, int IT>
__global__ void add_rmsnorm_vec_kernel(TO* __restrict__ out, float* __restrict__ resid, const TD* __restrict__ delta,
                                       int splits, int64_t split_stride, const TW* __restrict__ w, int H, float eps,
                                       float w_offset) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float4 v[IT], wv[IT];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int j = (it * blockDim.x + threadIdx.x) * 4;
        v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        wv[it] = v[it];
        if (j >= H) continue;
        v[it] = zi_load4(resid + row * H + j);
        wv[it] = zi_load4(w + j);
        const TD* dr = delta + row * H + j;
        float4 d[16];   // every split's load is issued before the first is used
#pragma unroll
        for (int sp = 0; sp < 16; ++sp)
            d[sp] = (sp < splits) ? zi_load4(dr + (int64_t)sp * split_stride) : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 t = d[0];
#pragma unroll
        for (int sp = 1; sp < 16; ++sp) { t.x += d[sp].x; t.y += d[sp].y; t.z += d[sp].z; t.w += d[sp].w; }
        v[it].x += t.x; v[it].y += t.y; v[it].z += t.z; v[it].w += t.w;
        zi_store4(resid + row * H + j, v[it]);
        ss += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
    }
    ss = zi_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int j = (it * blockDim.x + threadIdx.x) * 4;
        if (j >= H) continue;
        zi_store4(out + row * H + j, make_float4((wv[it].x + w_offset) * v[it].x * rstd, (wv[it].y + w_offset) * v[it].y * rstd,
                                                 (wv[it].z + w_offset) * v[it].z * rstd, (wv[it].w + w_offset) * v[it].w * rstd));
    }
}

// Many rows (prompt portions), one addend: a wavefront per row, four rows a workgroup.  A lane owns NV
// groups of four consecutive values, 256 values apart, so every load instruction of the wavefront reads
// 1 KB of the row; all loads are issued before the first use, the sum of squares is taken within the
// wavefront (no barrier), and the row is read once.  H <= 1024 * NV, H % 4 == 0.
template <typename TD, typename TW, typename TO, int NV>
__global__ void __launch_bounds__(4 * ZI_WAVE)
add_rmsnorm_rows_kernel(TO* __restrict__ out, float* __restrict__ resid, const TD* __restrict__ delta,
                        const TW* __restrict__ w, int n, int H, float eps, float w_offset) {
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= n) return;
    float* rr = resid + row * H;
    const TD* dr = delta + row * H;
    float4 v[NV], d[NV], wv[NV];
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4, jc = j < H ? j : 0;     // past the row: its start again, unused
        v[c] = zi_load4(rr + jc);
        d[c] = zi_load4(dr + jc);
        wv[c] = zi_load4(w + jc);
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4;
        v[c].x += d[c].x; v[c].y += d[c].y; v[c].z += d[c].z; v[c].w += d[c].w;
        if (j < H) {
            zi_store4(rr + j, v[c]);
            ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
        }
    }
    ss = zi_wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    TO* orow = out + row * H;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4;
        if (j < H)
            zi_store4(orow + j, make_float4((wv[c].x + w_offset) * v[c].x * rstd, (wv[c].y + w_offset) * v[c].y * rstd,
                                            (wv[c].z + w_offset) * v[c].z * rstd, (wv[c].w + w_offset) * v[c].w * rstd));
    }
}

#define NORM_MANY_ROWS 64     // from this many rows on, a wavefront per row

extern "C" int zi_add_rmsnorm(void* out, int out_dt, float* resid, const void* delta, int delta_dt, int splits,
                              int64_t split_stride, const void* w, int w_dt, int n, int hidden, float eps, int add_one,
                              hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
    ZI_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || split_stride >= (int64_t)n * hidden),
               "add_rmsnorm: bad partial sums (splits %d, stride %lld)", splits, (long long)split_stride);
    if (n == 0) return 0;
    const bool aligned = ((uintptr_t)out % 16) == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)delta % 16) == 0 &&
                         ((uintptr_t)w % 16) == 0 && split_stride % 4 == 0;
    if (n >= NORM_MANY_ROWS && splits == 1 && hidden % 4 == 0 && hidden <= 8192 && aligned) {
        const int nv = (hidden + 4 * ZI_WAVE - 1) / (4 * ZI_WAVE);
        const int wgs = (n + 3) / 4;
#define ZI_NORM_ROWS(NV)                                                                                            \
    add_rmsnorm_rows_kernel<TD, TW, TO, NV><<<wgs, 4 * ZI_WAVE, 0, stream>>>(                                       \
        (TO*)out, resid, (const TD*)delta, (const TW*)w, n, hidden, eps, add_one ? 1.f : 0.f)
        ZI_DISPATCH_DTYPE(delta_dt, TD, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
            if (nv <= 2) ZI_NORM_ROWS(2);
            else if (nv <= 4) ZI_NORM_ROWS(4);
            else if (nv <= 6) ZI_NORM_ROWS(6);
            else if (nv <= 8) ZI_NORM_ROWS(8);
            else if (nv <= 12) ZI_NORM_ROWS(12);
            else if (nv <= 16) ZI_NORM_ROWS(16);
            else if (nv <= 20) ZI_NORM_ROWS(20);
            else if (nv <= 24) ZI_NORM_ROWS(24);
            else ZI_NORM_ROWS(32);
        })));
#undef ZI_NORM_ROWS
        return zi_check_launch("add_rmsnorm");
    }
    if (hidden % 4 == 0 && hidden <= 8192 && splits <= 16 && aligned) {
        const int vecs = hidden / 4;
        const int it = vecs > 1024 ? 2 : 1;
        int threads = ((vecs + it - 1) / it + ZI_WAVE - 1) / ZI_WAVE * ZI_WAVE;
        ZI_DISPATCH_DTYPE(delta_dt, TD, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
            if (it == 1)
                add_rmsnorm_vec_kernel<TD, TW, TO, 1><<<n, threads, 0, stream>>>(
                    (TO*)out, resid, (const TD*)delta, splits, split_stride, (const TW*)w, hidden, eps, add_one ? 1.f : 0.f);
            else
                add_rmsnorm_vec_kernel<TD, TW, TO, 2><<<n, threads, 0, stream>>>(
                    (TO*)out, resid, (const TD*)delta, splits, split_stride, (const TW*)w, hidden, eps, add_one ? 1.f : 0.f);
        })));
        return zi_check_launch("add_rmsnorm");
    }
    ZI_DISPATCH_DTYPE(delta_dt, TD, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        add_rmsnorm_kernel<TD, TW, TO><<<n, NORM_THREADS, 0, stream>>>((TO*)out, resid, (const TD*)delta, splits,
                                                                       split_stride, (const TW*)w, hidden, eps,
                                                                       add_one ? 1.f : 0.f);
    })));
    return zi_check_launch("add_rmsnorm");
}
