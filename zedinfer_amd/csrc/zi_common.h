// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave and block reductions, and the host-side error channel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <math.h>

#define ZI_F32 0
#define ZI_BF16 1
#define ZI_WAVE 64

// bfloat16 is stored as its 16 raw bits.
struct zi_bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float zi_bf16_to_float(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// Round to nearest, ties to even; NaN stays NaN (the quiet bit is forced).
__device__ __forceinline__ uint16_t zi_float_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Two floats to two bfloat16 in one word (first in the low half), rounded to nearest even by the
// hardware convert (v_cvt_pk_bf16_f32).
typedef __attribute__((ext_vector_type(2))) __bf16 zi_bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float zi_f32x2_t;
__device__ __forceinline__ uint32_t zi_pack_bf16x2(float a, float b) {
    zi_f32x2_t v;
    v[0] = a;
    v[1] = b;
    union { zi_bf16x2_t h; uint32_t u; } c;
    c.h = __builtin_convertvector(v, zi_bf16x2_t);
    return c.u;
}

__device__ __forceinline__ float zi_load(const float* p) { return *p; }
__device__ __forceinline__ float zi_load(const zi_bf16* p) { return zi_bf16_to_float(p->bits); }
__device__ __forceinline__ void zi_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void zi_store(zi_bf16* p, float v) { p->bits = zi_float_to_bf16(v); }

__device__ __forceinline__ float zi_wave_sum(float v) {
#pragma unroll
    for (int o = ZI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, ZI_WAVE);
    return v;
}
__device__ __forceinline__ float zi_wave_max(float v) {
#pragma unroll
    for (int o = ZI_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, ZI_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS.  The order of additions is fixed
// by the thread layout alone, so a row's sum does not depend on the batch.
__device__ __forceinline__ float zi_block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int nwaves = (blockDim.x + ZI_WAVE - 1) / ZI_WAVE;
    v = zi_wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nwaves; ++i) r += scratch[i];
    return r;
}
__device__ __forceinline__ float zi_block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int nwaves = (blockDim.x + ZI_WAVE - 1) / ZI_WAVE;
    v = zi_wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int i = 1; i < nwaves; ++i) r = fmaxf(r, scratch[i]);
    return r;
}

// ---- host side -------------------------------------------------------------
// Every entry point returns 0 on success.  On failure it returns non-zero and
// leaves a message that zi_last_error() hands out.
extern "C" const char* zi_last_error();
#define ZI_DEFAULT_COMPUTE_UNITS 256      // an MI355X
extern "C" int zi_compute_units();
int zi_fail(const char* fmt, ...);
int zi_check_launch(const char* what);

#define ZI_REQUIRE(cond, ...)              \
    do {                                   \
        if (!(cond)) return zi_fail(__VA_ARGS__); \
    } while (0)

// Run BODY with T bound to the storage type that `dt` names.
#define ZI_DISPATCH_DTYPE(dt, T, ...)                                  \
    do {                                                               \
        if ((dt) == ZI_F32) { using T = float; __VA_ARGS__; }          \
        else if ((dt) == ZI_BF16) { using T = zi_bf16; __VA_ARGS__; }  \
        else return zi_fail("unknown dtype code %d", (int)(dt));       \
    } while (0)
