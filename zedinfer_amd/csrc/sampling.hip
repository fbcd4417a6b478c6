// Choosing the next token on the device: argmax, and temperature / top-k /
// top-p / repetition-penalty sampling.
//
// The sampled token is the one the reference's host sampler would pick from the
// same logits and the same uniform draw u (reference:
// src/frontend/sampler/sampler.cpp:195-265 truncatedDist + sampleFromDist,
// :410-490 the steps): repetition penalty on raw logits (l > 0 ? l/p : l*p, once
// per listed token), division by the temperature, softmax, order by falling
// probability, keep the first top_k, then the smallest prefix whose sum reaches
// top_p, renormalise, and take the first entry whose running sum exceeds u.
// Instead of sorting the vocabulary the kernel finds each cut by bisection on
// the probability's bit pattern (non-negative floats order like their bits);
// equal probabilities are ordered by rising token id.  One workgroup per row.
#include "zi_common.h"
#include "zi_api.h"
#include "zi_no_alloc.h"
#include <mutex>

#define SAMPLE_THREADS 1024

// Highest value, lowest index among equals (reference:
// src/backend/ops/argmax/cpu/argmax_cpu.cpp:17-19).  NaNs never win.
template <typename T>
__device__ int block_argmax(const T* v, int V, float* out_val, float* fred, int* ired) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float x = zi_load(v + i);
        if (x > best || (x == best && i < bi)) { best = x; bi = i; }
    }
#pragma unroll
    for (int o = ZI_WAVE / 2; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, ZI_WAVE);
        const int oi = __shfl_xor(bi, o, ZI_WAVE);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int nwaves = (blockDim.x + ZI_WAVE - 1) / ZI_WAVE;
    __syncthreads();
    if (lane == 0) { fred[wave] = best; ired[wave] = bi; }
    __syncthreads();
    best = fred[0];
    bi = ired[0];
    for (int i = 1; i < nwaves; ++i)
        if (fred[i] > best || (fred[i] == best && ired[i] < bi)) { best = fred[i]; bi = ired[i]; }
    if (bi == 0x7fffffff) bi = 0;
    if (out_val) *out_val = best;
    return bi;
}

template <typename T>
__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_kernel(int32_t* __restrict__ out_idx, float* __restrict__ out_val, const T* __restrict__ logits,
              int64_t ld, int V) {
    __shared__ float fred[16];
    __shared__ int ired[16];
    const int64_t row = blockIdx.x;
    float bv;
    const int bi = block_argmax<T>(logits + row * ld, V, &bv, fred, ired);
    if (threadIdx.x == 0) {
        out_idx[row] = bi;
        if (out_val) out_val[row] = bv;
    }
}

// Stage one of the argmax of long rows: part `blockIdx.y` of row `blockIdx.x` leaves its best (value, index).
template <typename T>
__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_part_kernel(float* __restrict__ part_val, int32_t* __restrict__ part_idx, const T* __restrict__ logits,
                   int64_t ld, int V, int part_len) {
    __shared__ float fred[16];
    __shared__ int ired[16];
    const int64_t row = blockIdx.x;
    const int lo = blockIdx.y * part_len;
    const int n = (lo + part_len < V) ? part_len : V - lo;
    float bv;
    const int bi = block_argmax<T>(logits + row * ld + lo, n, &bv, fred, ired);
    if (threadIdx.x == 0) {
        part_val[row * gridDim.y + blockIdx.y] = bv;
        part_idx[row * gridDim.y + blockIdx.y] = lo + bi;
    }
}

// Stage two: the best of a row's parts; the lowest index among equals (parts are in rising order of index).
__global__ void argmax_merge_kernel(int32_t* __restrict__ out_idx, float* __restrict__ out_val,
                                    const float* __restrict__ part_val, const int32_t* __restrict__ part_idx,
                                    int parts) {
    const int row = blockIdx.x, lane = threadIdx.x;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < parts; i += ZI_WAVE) {
        const float v = part_val[row * parts + i];
        const int x = part_idx[row * parts + i];
        if (v > best || (v == best && x < bi)) { best = v; bi = x; }
    }
#pragma unroll
    for (int o = ZI_WAVE / 2; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, ZI_WAVE);
        const int oi = __shfl_xor(bi, o, ZI_WAVE);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (lane == 0) {
        out_idx[row] = bi == 0x7fffffff ? 0 : bi;
        if (out_val) out_val[row] = best;
    }
}

#define ARGMAX_PART 8192   // values one workgroup scans when a row is cut

// Floats of workspace that let a row be cut over several workgroups (0: rows are short).
extern "C" int64_t zi_argmax_workspace(int rows, int vocab) {
    const int parts = (vocab + ARGMAX_PART - 1) / ARGMAX_PART;
    return parts > 1 ? 2 * (int64_t)rows * parts : 0;
}

extern "C" int zi_argmax(int32_t* out_idx, float* out_val, const void* logits, int dt, int rows, int vocab,
                         int64_t ld, float* workspace, int64_t workspace_floats, hipStream_t stream) {
    ZI_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    const int parts = (vocab + ARGMAX_PART - 1) / ARGMAX_PART;
    if (parts > 1 && workspace && workspace_floats >= 2 * (int64_t)rows * parts && rows <= 65535 && parts <= 65535) {
        float* pv = workspace;
        int32_t* pi = reinterpret_cast<int32_t*>(workspace + (int64_t)rows * parts);
        ZI_DISPATCH_DTYPE(dt, T, {
            argmax_part_kernel<T><<<dim3(rows, parts), SAMPLE_THREADS, 0, stream>>>(pv, pi, (const T*)logits, ld, vocab,
                                                                                    ARGMAX_PART);
        });
        argmax_merge_kernel<<<rows, ZI_WAVE, 0, stream>>>(out_idx, out_val, pv, pi, parts);
        return zi_check_launch("argmax");
    }
    ZI_DISPATCH_DTYPE(dt, T, {
        argmax_kernel<T><<<rows, SAMPLE_THREADS, 0, stream>>>(out_idx, out_val, (const T*)logits, ld, vocab);
    });
    return zi_check_launch("argmax");
}

// ---- the argmax that allocates nothing ------------------------------------------------------------
// The parts' (value, index) pairs live in this array instead of a workspace.  In host code the array's
// name is only a stand-in for the symbol; the memory's address on a device comes from
// hipGetSymbolAddress, once per device, with that device current (every GPU has its own copy).
static __device__ __align__(256) unsigned char scratch[ZI_ARGMAX_STATIC_MAX_PARTS * 8];

#define ZI_MAX_DEVICES 64
static void* scratch_of_device[ZI_MAX_DEVICES];
static std::mutex scratch_lock;

// The address of `scratch` on the current device; nullptr (with the error set) when it cannot be had.
static void* scratch_address() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= ZI_MAX_DEVICES) {
        zi_fail("argmax_static: no current device (%s, device %d)", hipGetErrorString(e), dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_of_device[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            zi_fail("argmax_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        scratch_of_device[dev] = ptr;
    }
    return scratch_of_device[dev];
}

extern "C" int zi_argmax_static_max_parts() { return ZI_ARGMAX_STATIC_MAX_PARTS; }

extern "C" int zi_argmax_static(int32_t* out_idx, float* out_val, const void* logits, int dt, int rows, int vocab,
                                int64_t ld, hipStream_t stream) {
    ZI_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
    ZI_REQUIRE(out_idx && logits, "argmax_static: null argument");
    if (rows == 0) return 0;
    const int parts = (vocab + ARGMAX_PART - 1) / ARGMAX_PART;
    if (parts == 1) {      // short rows need no memory beside the result
        ZI_DISPATCH_DTYPE(dt, T, {
            argmax_kernel<T><<<rows, SAMPLE_THREADS, 0, stream>>>(out_idx, out_val, (const T*)logits, ld, vocab);
        });
        return zi_check_launch("argmax_static");
    }
    ZI_REQUIRE((int64_t)rows * parts <= ZI_ARGMAX_STATIC_MAX_PARTS && rows <= 65535,
               "argmax_static: %d rows of %d values are %lld parts, the library's array holds %d "
               "(use zi_argmax with a workspace)", rows, vocab, (long long)rows * parts, ZI_ARGMAX_STATIC_MAX_PARTS);
    void* ptr = scratch_address();
    if (!ptr) return 1;
    float* pv = reinterpret_cast<float*>(ptr);
    int32_t* pi = reinterpret_cast<int32_t*>(pv + (int64_t)rows * parts);
    ZI_DISPATCH_DTYPE(dt, T, {
        argmax_part_kernel<T><<<dim3(rows, parts), SAMPLE_THREADS, 0, stream>>>(pv, pi, (const T*)logits, ld, vocab,
                                                                                ARGMAX_PART);
    });
    argmax_merge_kernel<<<rows, ZI_WAVE, 0, stream>>>(out_idx, out_val, pv, pi, parts);
    return zi_check_launch("argmax_static");
}

// Sum and count of the probabilities whose bit pattern is >= tau.
__device__ void mass_count_ge(const float* p, int V, uint32_t tau, float* mass, float* count, float* fred) {
    float m = 0.f, c = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float x = p[i];
        if (__float_as_uint(x) >= tau) { m += x; c += 1.f; }
    }
    *mass = zi_block_sum(m, fred);
    *count = zi_block_sum(c, fred);
}

// Number of entries with bits == v and index <= x.
__device__ float count_eq_upto(const float* p, int V, uint32_t v, int x, float* fred) {
    float c = 0.f;
    for (int i = threadIdx.x; i < V && i <= x; i += blockDim.x)
        if (__float_as_uint(p[i]) == v) c += 1.f;
    return zi_block_sum(c, fred);
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(int32_t* __restrict__ out, const float* __restrict__ logits, int64_t ld, float* __restrict__ work,
              int V, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ penalty, const float* __restrict__ uniform,
              const int32_t* __restrict__ recent, const int32_t* __restrict__ recent_len, int max_recent) {
    __shared__ float fred[16];
    __shared__ int ired[16];
    const int64_t row = blockIdx.x;
    const float* lg = logits + row * ld;
    float* w = work + row * (int64_t)V;
    const float T = temperature[row];
    const float pen = penalty[row];
    const int nrec = recent_len ? recent_len[row] : 0;

    for (int i = threadIdx.x; i < V; i += blockDim.x) w[i] = lg[i];
    __syncthreads();
    if (pen != 1.0f && nrec > 0) {
        if (threadIdx.x == 0) {
            const int32_t* rc = recent + row * (int64_t)max_recent;
            for (int r = 0; r < nrec; ++r) {
                const int t = rc[r];
                if (t < 0 || t >= V) continue;
                const float lv = w[t];
                w[t] = lv > 0.f ? lv / pen : lv * pen;
            }
        }
        __syncthreads();
    }
    if (!(T > 0.f)) {  // greedy row
        const int bi = block_argmax<float>(w, V, nullptr, fred, ired);
        if (threadIdx.x == 0) out[row] = bi;
        return;
    }
    // temperature and softmax
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        float x = w[i];
        if (T != 1.0f) { x = x / T; w[i] = x; }
        mx = fmaxf(mx, x);
    }
    mx = zi_block_max(mx, fred);
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float e = expf(w[i] - mx);
        w[i] = e;
        sum += e;
    }
    sum = zi_block_sum(sum, fred);
    for (int i = threadIdx.x; i < V; i += blockDim.x) w[i] = w[i] / sum;
    __syncthreads();

    const uint32_t TOP = 0x7f800000u;  // +inf: above every probability
    float mass, cnt;
    // ---- top-k: value of the k-th entry and how many of its equals are kept
    uint32_t v_keep = 0;
    float c_keep, Z;
    const int k = top_k[row];
    if (k > 0 && k < V) {
        uint32_t lo = 0, hi = TOP;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo + 1) / 2;
            mass_count_ge(w, V, mid, &mass, &cnt, fred);
            if (cnt >= (float)k) lo = mid; else hi = mid - 1;
        }
        v_keep = lo;
        mass_count_ge(w, V, v_keep + 1, &mass, &cnt, fred);
        c_keep = (float)k - cnt;
        Z = mass + c_keep * __uint_as_float(v_keep);
    } else {
        mass_count_ge(w, V, 0, &mass, &cnt, fred);
        Z = mass;
        float mgt, cgt;
        mass_count_ge(w, V, 1, &mgt, &cgt, fred);
        c_keep = cnt - cgt;
    }
    // ---- top-p: smallest prefix (inside the top-k prefix) whose sum reaches top_p
    const float pp = top_p[row];
    if (pp < 1.0f && Z >= pp) {
        uint32_t lo = v_keep, hi = TOP;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo + 1) / 2;
            mass_count_ge(w, V, mid, &mass, &cnt, fred);
            if (mass >= pp) lo = mid; else hi = mid - 1;
        }
        float mgt, cgt;
        mass_count_ge(w, V, lo + 1, &mgt, &cgt, fred);
        float nt;
        if (lo == v_keep) nt = c_keep;
        else { mass_count_ge(w, V, lo, &mass, &cnt, fred); nt = cnt - cgt; }
        const float v = __uint_as_float(lo);
        float c = v > 0.f ? ceilf((pp - mgt) / v) : nt;
        c = fminf(fmaxf(c, 1.f), nt);
        v_keep = lo;
        c_keep = c;
        Z = mgt + c * v;
    }
    // ---- draw: first entry whose running sum exceeds u * Z
    const float target = uniform[row] * Z;
    uint32_t lo = v_keep, hi = TOP;
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo + 1) / 2;
        mass_count_ge(w, V, mid, &mass, &cnt, fred);
        if (mass > target) lo = mid; else hi = mid - 1;
    }
    float mgt, cgt;
    mass_count_ge(w, V, lo + 1, &mgt, &cgt, fred);
    float nt;
    if (lo == v_keep) nt = c_keep;
    else { mass_count_ge(w, V, lo, &mass, &cnt, fred); nt = cnt - cgt; }
    const float v = __uint_as_float(lo);
    float c = v > 0.f ? floorf((target - mgt) / v) + 1.f : 1.f;
    c = fminf(fmaxf(c, 1.f), fmaxf(nt, 1.f));
    // the c-th entry, by rising token id, among those equal to v
    int xlo = 0, xhi = V - 1;
    while (xlo < xhi) {
        const int mid = xlo + (xhi - xlo) / 2;
        if (count_eq_upto(w, V, lo, mid, fred) >= c) xhi = mid; else xlo = mid + 1;
    }
    if (threadIdx.x == 0) out[row] = xlo;
}

extern "C" int zi_sample(int32_t* out, const float* logits, int64_t ld, float* work, int rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p, const float* penalty,
                         const float* uniform, const int32_t* recent, const int32_t* recent_len, int max_recent,
                         hipStream_t stream) {
    ZI_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    ZI_REQUIRE(vocab < (1 << 24), "sample: vocabulary %d too large for exact counting", vocab);
    ZI_REQUIRE(max_recent >= 0, "sample: negative history length");
    if (rows == 0) return 0;
    sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, work, vocab, temperature, top_k, top_p, penalty,
                                                       uniform, recent, recent_len, max_recent);
    return zi_check_launch("sample");
}
