// Rotary position encoding (split-half, "NeoX" pairing) fused with the write of
// keys and values into the paged cache.
//
// For k < R/2 (R = rotary dims, R = head_dim for full rotation):
//   angle = float(pos) * inv_freq[k]          (float32; inv_freq[k] = theta^(-2k/R), made on the host)
//   out[k]       = a cos(angle) - b sin(angle)
//   out[k + R/2] = b cos(angle) + a sin(angle)     with a = in[k], b = in[k + R/2]
// (reference: src/backend/ops/rope/cpu/rope_cpu.cpp:33,47-52,62-65).  Queries are
// rotated in place; keys are rotated on their way into the cache, values copied
// (reference: K is stored after rotation, V raw, src/frontend/models/transformer_forward.cpp:99-104).
//
// Cache layout of one layer.  Keys: [page][kv_head][slot_in_page][head_dim].  Values are
// stored transposed: [page][kv_head][head_dim][slot_in_page], so that a run of consecutive
// positions of one dimension is contiguous, which is the order the matrix cores want for
// the P.V product.  Token slot s lives in page s / page_size at offset s % page_size.
// A negative slot skips the write.
#include "zi_common.h"

template <typename T>
__global__ void rope_kv_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                     int64_t ldq, int64_t ldk, int64_t ldv, const int32_t* __restrict__ pos,
                                     const int32_t* __restrict__ slots, const float* __restrict__ inv_freq,
                                     T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv, int d,
                                     int rot, int page_size, int write_kv, int64_t cache_slots) {
    extern __shared__ float cs[];  // cos[rot/2], sin[rot/2]
    const int64_t t = blockIdx.x;
    const int half = rot / 2;
    const float p = (float)pos[t];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s, c;
        sincosf(p * inv_freq[i], &s, &c);
        cs[i] = c;
        cs[half + i] = s;
    }
    __syncthreads();
    // queries, in place
    T* qr = q + t * ldq;
    for (int i = threadIdx.x; i < nh * half; i += blockDim.x) {
        const int h = i / half, j = i % half;
        T* base = qr + (int64_t)h * d;
        const float a = zi_load(base + j), b = zi_load(base + j + half);
        const float c = cs[j], s = cs[half + j];
        zi_store(base + j, a * c - b * s);
        zi_store(base + j + half, b * c + a * s);
    }
    if (!write_kv) return;
    const int slot = slots[t];
    if (slot < 0 || slot >= cache_slots) return;  // the host checks the range; never write outside the pool
    const int64_t page = slot / page_size, off = slot % page_size;
    const T* kr = k + t * ldk;
    const T* vr = v + t * ldv;
    for (int i = threadIdx.x; i < nkv * d; i += blockDim.x) {
        const int h = i / d, j = i % d;
        const int64_t dst = ((page * nkv + h) * page_size + off) * d + j;
        float kv;
        if (j < half) {
            kv = zi_load(kr + h * d + j) * cs[j] - zi_load(kr + h * d + j + half) * cs[half + j];
        } else if (j < rot) {
            const int jj = j - half;
            kv = zi_load(kr + h * d + j) * cs[jj] + zi_load(kr + h * d + jj) * cs[half + jj];
        } else {
            kv = zi_load(kr + h * d + j);
        }
        zi_store(kcache + dst, kv);
        vcache[((page * nkv + h) * d + j) * page_size + off] = vr[h * d + j];
    }
}

extern "C" int zi_rope_kv_store(void* q, const void* k, const void* v, int dt, int n, int64_t ldq, int64_t ldk,
                                int64_t ldv, const int32_t* pos, const int32_t* slots, const float* inv_freq,
                                void* kcache, void* vcache, int64_t cache_slots, int nh, int nkv, int d, int rot,
                                int page_size, int write_kv, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv >= 0 && d > 0, "rope_kv_store: bad sizes");
    ZI_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "rope_kv_store: rotary dims %d must be even and <= head_dim %d", rot, d);
    ZI_REQUIRE(ldq >= (int64_t)nh * d, "rope_kv_store: query row stride %lld < heads*head_dim", (long long)ldq);
    if (write_kv) {
        ZI_REQUIRE(page_size > 0 && cache_slots > 0 && cache_slots % page_size == 0,
                   "rope_kv_store: cache of %lld slots is not a whole number of pages of %d", (long long)cache_slots, page_size);
        ZI_REQUIRE(ldk >= (int64_t)nkv * d && ldv >= (int64_t)nkv * d, "rope_kv_store: key/value row stride too small");
        ZI_REQUIRE(k && v && kcache && vcache && slots, "rope_kv_store: null cache or key/value pointer");
    }
    ZI_REQUIRE(rot * sizeof(float) <= 48 * 1024, "rope_kv_store: rotary dims %d too large", rot);
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        rope_kv_store_kernel<T><<<n, 256, rot * sizeof(float), stream>>>(
            (T*)q, (const T*)k, (const T*)v, ldq, ldk, ldv, pos, slots, inv_freq, (T*)kcache, (T*)vcache, nh, nkv, d,
            rot, page_size, write_kv, cache_slots);
    });
    return zi_check_launch("rope_kv_store");
}

// The same for q, k, v that arrive as float32 partial sums of one fused projection: columns
// [0, nh*d) of a row are q, the next nkv*d are k, the last nkv*d are v; split s of row t starts at
// part + s * split_stride + t * ldp.  The splits are added in rising order, the bias is added, and
// the row is rotated from float32: q goes to q_out (rounded once), k and v into the cache.
template <typename T, typename TB>
__global__ void rope_kv_store_split_kernel(T* __restrict__ q_out, int64_t ldq, const float* __restrict__ part,
                                           int splits, int64_t split_stride, int64_t ldp,
                                           const TB* __restrict__ bias, const int32_t* __restrict__ pos,
                                           const int32_t* __restrict__ slots, const float* __restrict__ inv_freq,
                                           T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv, int d,
                                           int rot, int page_size, int write_kv, int64_t cache_slots, int vec4) {
    extern __shared__ __attribute__((aligned(16))) float sh[];  // cos[rot/2], sin[rot/2], then the summed row
    const int64_t t = blockIdx.x;
    const int half = rot / 2;
    const int qd = nh * d, kvd = nkv * d;
    const int width = qd + (write_kv ? 2 * kvd : 0);
    float* cs = sh;
    float* row = sh + ((rot + 3) & ~3);
    const float p = (float)pos[t];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s, c;
        sincosf(p * inv_freq[i], &s, &c);
        cs[i] = c;
        cs[half + i] = s;
    }
    const float* pr = part + t * ldp;
    if (vec4) {
        // every split's load is issued before the first is used (host: splits <= 16, 16-byte alignment)
        for (int i = threadIdx.x * 4; i < width; i += blockDim.x * 4) {
            float4 d[16];
#pragma unroll
            for (int s = 0; s < 16; ++s)
                d[s] = (s < splits) ? *reinterpret_cast<const float4*>(pr + (int64_t)s * split_stride + i)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
            float4 v = d[0];
#pragma unroll
            for (int s = 1; s < 16; ++s) { v.x += d[s].x; v.y += d[s].y; v.z += d[s].z; v.w += d[s].w; }
            if (bias) {
                v.x += zi_load(bias + i); v.y += zi_load(bias + i + 1); v.z += zi_load(bias + i + 2);
                v.w += zi_load(bias + i + 3);
            }
            *reinterpret_cast<float4*>(row + i) = v;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float v = pr[i];
            for (int s = 1; s < splits; ++s) v += pr[s * split_stride + i];
            if (bias) v += zi_load(bias + i);
            row[i] = v;
        }
    }
    __syncthreads();
    T* qr = q_out + t * ldq;
    for (int i = threadIdx.x; i < qd; i += blockDim.x) {
        const int h = i / d, j = i % d;
        const float* base = row + h * d;
        float v;
        if (j < half) v = base[j] * cs[j] - base[j + half] * cs[half + j];
        else if (j < rot) v = base[j] * cs[j - half] + base[j - half] * cs[j];
        else v = base[j];
        zi_store(qr + i, v);
    }
    if (!write_kv) return;
    const int slot = slots[t];
    if (slot < 0 || slot >= cache_slots) return;  // the host checks the range; never write outside the pool
    const int64_t page = slot / page_size, off = slot % page_size;
    for (int i = threadIdx.x; i < kvd; i += blockDim.x) {
        const int h = i / d, j = i % d;
        const float* base = row + qd + h * d;
        float kv;
        if (j < half) kv = base[j] * cs[j] - base[j + half] * cs[half + j];
        else if (j < rot) kv = base[j] * cs[j - half] + base[j - half] * cs[j];
        else kv = base[j];
        zi_store(kcache + ((page * nkv + h) * page_size + off) * d + j, kv);
        zi_store(vcache + ((page * nkv + h) * d + j) * page_size + off, row[qd + kvd + i]);
    }
}

extern "C" int zi_rope_kv_store_split(void* q_out, int dt, int64_t ldq, const float* part, int splits,
                                      int64_t split_stride, int64_t ldp, const void* bias, int bias_dt, int n,
                                      const int32_t* pos, const int32_t* slots, const float* inv_freq, void* kcache,
                                      void* vcache, int64_t cache_slots, int nh, int nkv, int d, int rot,
                                      int page_size, int write_kv, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv >= 0 && d > 0, "rope_kv_store_split: bad sizes");
    ZI_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "rope_kv_store_split: rotary dims %d must be even and <= head_dim %d",
               rot, d);
    const int64_t width = (int64_t)nh * d + (write_kv ? 2 * (int64_t)nkv * d : 0);
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldp >= width, "rope_kv_store_split: row stride too small");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || split_stride >= (int64_t)n * ldp),
               "rope_kv_store_split: bad partial sums (splits %d, stride %lld)", splits, (long long)split_stride);
    ZI_REQUIRE(rot == 0 || inv_freq, "rope_kv_store_split: no frequency table");
    if (write_kv) {
        ZI_REQUIRE(page_size > 0 && cache_slots > 0 && cache_slots % page_size == 0,
                   "rope_kv_store_split: cache of %lld slots is not a whole number of pages of %d", (long long)cache_slots,
                   page_size);
        ZI_REQUIRE(kcache && vcache && slots, "rope_kv_store_split: null cache pointer");
    }
    const size_t lds = (size_t)(((rot + 3) & ~3) + width + 4) * sizeof(float);
    const int vec4 = width % 4 == 0 && ldp % 4 == 0 && split_stride % 4 == 0 && ((uintptr_t)part % 16) == 0 && splits <= 16;
    ZI_REQUIRE(lds <= 60 * 1024, "rope_kv_store_split: a row of %lld values does not fit in LDS", (long long)width);
    if (n == 0) return 0;
    if (!bias) bias_dt = ZI_F32;
    ZI_DISPATCH_DTYPE(dt, T, ZI_DISPATCH_DTYPE(bias_dt, TB, {
        rope_kv_store_split_kernel<T, TB><<<n, 256, lds, stream>>>(
            (T*)q_out, ldq, part, splits, split_stride, ldp, (const TB*)bias, pos, slots, inv_freq, (T*)kcache,
            (T*)vcache, nh, nkv, d, rot, page_size, write_kv, cache_slots, vec4);
    }));
    return zi_check_launch("rope_kv_store_split");
}

// Rotation alone, out of place: out[t,h,:] = rotate(in[t,h,:], pos[t])  (op-level entry, and the
// form a layer uses that reads another layer's cache and therefore stores nothing).
template <typename T>
__global__ void rope_kernel(T* __restrict__ out, const T* __restrict__ in, int64_t ld_in, int64_t ld_out,
                            const int32_t* __restrict__ pos, const float* __restrict__ inv_freq, int nh, int d,
                            int rot) {
    extern __shared__ float cs[];
    const int64_t t = blockIdx.x;
    const int half = rot / 2;
    const float p = (float)pos[t];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s, c;
        sincosf(p * inv_freq[i], &s, &c);
        cs[i] = c;
        cs[half + i] = s;
    }
    __syncthreads();
    const T* ir = in + t * ld_in;
    T* orow = out + t * ld_out;
    for (int i = threadIdx.x; i < nh * half; i += blockDim.x) {
        const int h = i / half, j = i % half;
        const float a = zi_load(ir + (int64_t)h * d + j), b = zi_load(ir + (int64_t)h * d + j + half);
        zi_store(orow + (int64_t)h * d + j, a * cs[j] - b * cs[half + j]);
        zi_store(orow + (int64_t)h * d + j + half, b * cs[j] + a * cs[half + j]);
    }
    for (int i = threadIdx.x; i < nh * (d - rot); i += blockDim.x) {
        const int h = i / (d - rot), j = rot + i % (d - rot);
        orow[(int64_t)h * d + j] = ir[(int64_t)h * d + j];
    }
}

extern "C" int zi_rope(void* out, const void* in, int dt, int n, int64_t ld_in, int64_t ld_out, const int32_t* pos,
                       const float* inv_freq, int nh, int d, int rot, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && d > 0, "rope: bad sizes");
    ZI_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "rope: rotary dims %d must be even and <= head_dim %d", rot, d);
    ZI_REQUIRE(ld_in >= (int64_t)nh * d && ld_out >= (int64_t)nh * d, "rope: row stride too small");
    ZI_REQUIRE(rot * sizeof(float) <= 48 * 1024, "rope: rotary dims %d too large", rot);
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        rope_kernel<T><<<n, 256, rot * sizeof(float), stream>>>((T*)out, (const T*)in, ld_in, ld_out, pos, inv_freq, nh,
                                                                d, rot);
    });
    return zi_check_launch("rope");
}
