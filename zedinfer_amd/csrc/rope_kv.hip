// Rotary position encoding (split-half, "NeoX" pairing) fused with the write of
// keys and values into the paged cache.
//
// For k < R/2 (R = rotary dims, R = head_dim for full rotation):
//   angle = float(pos) * inv_freq[k]          (float32; inv_freq[k] = theta^(-2k/R), made on the host)
//   out[k]       = a cos(angle) - b sin(angle)
//   out[k + R/2] = b cos(angle) + a sin(angle)     with a = in[k], b = in[k + R/2]
// (reference: src/backend/ops/rope/cpu/rope_cpu.cpp:33,47-52,62-65).  The kernels that store take the step's
// (cos, sin) of every (token, k) as a table [n][R/2][2] (zi_rope_table makes it once per step, every layer
// reads it): whoever encodes positions decides the angles, the store only turns by them.  Queries are
// rotated in place; keys are rotated on their way into the cache, values copied
// (reference: K is stored after rotation, V raw, src/frontend/models/transformer_forward.cpp:99-104).
//
// Cache layout of one layer.  Keys: [page][kv_head][slot_in_page][head_dim].  Values are
// stored transposed: [page][kv_head][head_dim][slot_in_page], so that a run of consecutive
// positions of one dimension is contiguous, which is the order the matrix cores want for
// the P.V product.  Token slot s lives in page s / page_size at offset s % page_size.
// A negative slot skips the write.
#include "zi_common.h"
#include "zi_api.h"
#include "zi_paging.h"

template <typename T>
__global__ void rope_kv_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                     int64_t ldq, int64_t ldk, int64_t ldv, const int32_t* __restrict__ slots,
                                     const float2* __restrict__ table, T* __restrict__ kcache,
                                     T* __restrict__ vcache, int nh, int nkv, int d, int rot, int page_size,
                                     int write_kv, int64_t cache_slots) {
    extern __shared__ float cs[];  // cos[rot/2], sin[rot/2]
    const int64_t t = blockIdx.x;
    const int half = rot / 2;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const float2 e = table[t * half + i];
        cs[i] = e.x;
        cs[half + i] = e.y;
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
    const ZiSlotPlace place = zi_slot_place(slots[t], cache_slots, page_size);
    if (!place.ok) return;  // padding, or out of range (the host checks the range; never write outside the pool)
    const int64_t page = place.page;
    const int off = place.off;
    const T* kr = k + t * ldk;
    const T* vr = v + t * ldv;
    for (int i = threadIdx.x; i < nkv * d; i += blockDim.x) {
        const int h = i / d, j = i % d;
        const int64_t dst = zi_key_offset(page, h, off, nkv, page_size, d) + j;
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
        vcache[zi_value_offset(page, h, j, off, nkv, page_size, d)] = vr[h * d + j];
    }
}

// The same for many tokens (prompt portions) in bfloat16: a workgroup takes eight consecutive tokens, the
// angles of their positions go to LDS once, and everything moves in 16-byte pieces: a thread rotates
// eight dims of a head and their eight partners at a time.  Values are staged in LDS; when the eight
// tokens' slots are eight consecutive slots of one page that start at a multiple of eight (the usual case
// inside a prompt), a thread writes the eight tokens' values of one dim as one 16-byte run of the
// transposed value cache, else value by value.  half = rot / 2 must be a multiple of 8 (or 0).
#define RKT_TOKENS 8
__global__ void __launch_bounds__(256)
rope_kv_store_tile_kernel(zi_bf16* __restrict__ q, const zi_bf16* __restrict__ k, const zi_bf16* __restrict__ v,
                          int64_t ldq, int64_t ldk, int64_t ldv, const int32_t* __restrict__ slots,
                          const float2* __restrict__ table, zi_bf16* __restrict__ kcache, zi_bf16* __restrict__ vcache, int n, int nh, int nkv, int d,
                          int rot, int page_size, int write_kv, int64_t cache_slots) {
    extern __shared__ __attribute__((aligned(16))) unsigned char rkt_lds[];
    const int half = rot / 2, kvd = nkv * d;
    float* cs = reinterpret_cast<float*>(rkt_lds);                                   // [token][cos[half], sin[half]]
    uint16_t* vt = reinterpret_cast<uint16_t*>(rkt_lds + (size_t)RKT_TOKENS * rot * sizeof(float));   // [token][kvd]
    const int t0 = blockIdx.x * RKT_TOKENS, tid = threadIdx.x;
    const int nt = (n - t0 < RKT_TOKENS) ? n - t0 : RKT_TOKENS;
    for (int i = tid; i < nt * half; i += 256) {
        const int tt = i / half, jj = i % half;
        const float2 e = table[(int64_t)(t0 + tt) * half + jj];
        cs[tt * rot + jj] = e.x;
        cs[tt * rot + half + jj] = e.y;
    }
    if (write_kv)
        for (int i = tid; i < nt * (kvd / 8); i += 256) {
            const int tt = i / (kvd / 8), c8 = i % (kvd / 8);
            *reinterpret_cast<uint4*>(vt + tt * kvd + c8 * 8) =
                *reinterpret_cast<const uint4*>(v + (int64_t)(t0 + tt) * ldv + c8 * 8);
        }
    __syncthreads();
    auto unpack = [](uint4 u, float (&f)[8]) {
        f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
        f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
        f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
        f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
    };
    auto pack = [](const float (&f)[8]) {
        return make_uint4(zi_pack_bf16x2(f[0], f[1]), zi_pack_bf16x2(f[2], f[3]), zi_pack_bf16x2(f[4], f[5]),
                          zi_pack_bf16x2(f[6], f[7]));
    };
    // queries, in place: (token, head, eight dims of the first half and their partners)
    const int hp = half / 8;
    for (int i = tid; i < nt * nh * hp; i += 256) {
        const int tt = i / (nh * hp), rem = i % (nh * hp), h = rem / hp, j0 = (rem % hp) * 8;
        zi_bf16* base = q + (int64_t)(t0 + tt) * ldq + (int64_t)h * d + j0;
        float a[8], b[8], lo[8], hi[8];
        unpack(*reinterpret_cast<const uint4*>(base), a);
        unpack(*reinterpret_cast<const uint4*>(base + half), b);
        const float* c = cs + tt * rot + j0;
        const float* sn = c + half;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            lo[x] = a[x] * c[x] - b[x] * sn[x];
            hi[x] = b[x] * c[x] + a[x] * sn[x];
        }
        *reinterpret_cast<uint4*>(base) = pack(lo);
        *reinterpret_cast<uint4*>(base + half) = pack(hi);
    }
    if (!write_kv) return;
    // keys into the cache: (token, kv head, eight dims)
    const int dp = d / 8;
    for (int i = tid; i < nt * nkv * dp; i += 256) {
        const int tt = i / (nkv * dp), rem = i % (nkv * dp), h = rem / dp, j0 = (rem % dp) * 8;
        const ZiSlotPlace place = zi_slot_place(slots[t0 + tt], cache_slots, page_size);
        if (!place.ok) continue;     // the host checks the range; never write outside the pool
        const int64_t page = place.page;
        const int off = place.off;
        const zi_bf16* kr = k + (int64_t)(t0 + tt) * ldk + (int64_t)h * d;
        float a[8], o8[8];
        unpack(*reinterpret_cast<const uint4*>(kr + j0), a);
        if (j0 < rot) {
            const bool first = j0 < half;
            const int jj = first ? j0 : j0 - half;
            float b[8];
            unpack(*reinterpret_cast<const uint4*>(kr + (first ? j0 + half : jj)), b);
            const float* c = cs + tt * rot + jj;
            const float* sn = c + half;
#pragma unroll
            for (int x = 0; x < 8; ++x) o8[x] = first ? a[x] * c[x] - b[x] * sn[x] : a[x] * c[x] + b[x] * sn[x];
        } else {
#pragma unroll
            for (int x = 0; x < 8; ++x) o8[x] = a[x];
        }
        *reinterpret_cast<uint4*>(kcache + zi_key_offset(page, h, off, nkv, page_size, d) + j0) = pack(o8);
    }
    // values: transposed.  Eight tokens in eight consecutive slots from a multiple of eight: one run per dim.
    bool run = nt == RKT_TOKENS;
    const int s0 = slots[t0];
    if (run) {
#pragma unroll
        for (int x = 1; x < RKT_TOKENS; ++x) run = run && slots[t0 + x] == s0 + x;
        run = run && s0 >= 0 && (s0 & 7) == 0 && s0 + RKT_TOKENS <= cache_slots;
    }
    if (run) {
        const int64_t page = s0 / page_size, off = s0 % page_size;
        for (int i = tid; i < kvd; i += 256) {
            const int h = i / d, dim = i % d;
            uint4 u;
            u.x = (uint32_t)vt[0 * kvd + i] | ((uint32_t)vt[1 * kvd + i] << 16);
            u.y = (uint32_t)vt[2 * kvd + i] | ((uint32_t)vt[3 * kvd + i] << 16);
            u.z = (uint32_t)vt[4 * kvd + i] | ((uint32_t)vt[5 * kvd + i] << 16);
            u.w = (uint32_t)vt[6 * kvd + i] | ((uint32_t)vt[7 * kvd + i] << 16);
            *reinterpret_cast<uint4*>(vcache + zi_value_offset(page, h, dim, (int)off, nkv, page_size, d)) = u;
        }
    } else {
        for (int i = tid; i < nt * kvd; i += 256) {
            const int tt = i / kvd, col = i % kvd, h = col / d, dim = col % d;
            const ZiSlotPlace place = zi_slot_place(slots[t0 + tt], cache_slots, page_size);
            if (!place.ok) continue;
            vcache[zi_value_offset(place.page, h, dim, place.off, nkv, page_size, d)].bits = vt[i];
        }
    }
}

// From this many tokens on, the tile kernel (bfloat16, 16-byte pieces).  Below, a workgroup a token is
// faster (256 tokens with scattered slots, a large decode batch: 4.2 against 8.3 us; the two meet at 1,024
// tokens in one run of slots, and 2,048 take 7.0 against 8.8 us).
#define ROPE_MANY_TOKENS 1024

extern "C" int zi_rope_kv_store(void* q, const void* k, const void* v, int dt, int n, int64_t ldq, int64_t ldk,
                                int64_t ldv, const int32_t* slots, const float* table,
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
    ZI_REQUIRE(rot == 0 || (table && ((uintptr_t)table % 8) == 0), "rope_kv_store: no table of angles");
    if (n == 0) return 0;
    const float2* tb = reinterpret_cast<const float2*>(table);
    {
        // the tile kernel: bfloat16, rows and pointers that allow 16-byte pieces, eight rotated dims on one side
        const bool al = ((uintptr_t)q % 16) == 0 && ldq % 8 == 0 && d % 8 == 0 && (rot / 2) % 8 == 0 &&
                        (!write_kv || (((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 && ((uintptr_t)kcache % 16) == 0 &&
                                       ((uintptr_t)vcache % 16) == 0 && ldk % 8 == 0 && ldv % 8 == 0 && page_size % 8 == 0));
        const size_t lds = (size_t)RKT_TOKENS * rot * sizeof(float) + (write_kv ? (size_t)RKT_TOKENS * nkv * d * 2 : 0);
        if (dt == ZI_BF16 && n >= ROPE_MANY_TOKENS && al && lds <= 48 * 1024) {
            rope_kv_store_tile_kernel<<<(n + RKT_TOKENS - 1) / RKT_TOKENS, 256, lds, stream>>>(
                (zi_bf16*)q, (const zi_bf16*)k, (const zi_bf16*)v, ldq, ldk, ldv, slots, tb, (zi_bf16*)kcache,
                (zi_bf16*)vcache, n, nh, nkv, d, rot, page_size, write_kv, cache_slots);
            return zi_check_launch("rope_kv_store");
        }
    }
    ZI_DISPATCH_DTYPE(dt, T, {
        rope_kv_store_kernel<T><<<n, 256, rot * sizeof(float), stream>>>(
            (T*)q, (const T*)k, (const T*)v, ldq, ldk, ldv, slots, tb, (T*)kcache, (T*)vcache, nh, nkv, d,
            rot, page_size, write_kv, cache_slots);
    });
    return zi_check_launch("rope_kv_store");
}

// The same for q, k, v that arrive as float32 partial sums of one fused projection: columns
// [0, nh*d) of a row are q, the next nkv*d are k, the last nkv*d are v; split s of row t starts at
// part + s * split_stride + t * ldp.  The splits are added in rising order, the bias is added, and
// the row is rotated from float32: q goes to q_out (rounded once), k and v into the cache.
// One wavefront per (token, head): blockIdx.y < nh is a query head, the others are key heads, which
// bring their value head along.  A lane owns the pairs (j, j + rot/2) it rotates and reads their
// (cos, sin) itself, so nothing is shared and nothing waits at a barrier.  SP is the number of splits
// rounded up to a power of two: that many loads are issued at once per value.
template <typename T, typename TB, int SP>
__global__ void __launch_bounds__(ZI_WAVE)
rope_kv_store_split_kernel(T* __restrict__ q_out, int64_t ldq, const float* __restrict__ part, int splits,
                           int64_t split_stride, int64_t ldp, const TB* __restrict__ bias,
                           const int32_t* __restrict__ slots, const float2* __restrict__ table,
                           T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv, int d, int rot,
                           int page_size, int64_t cache_slots) {
    const int64_t t = blockIdx.x;
    const int hs = blockIdx.y, lane = threadIdx.x;
    const int half = rot / 2;
    const int qd = nh * d, kvd = nkv * d;
    const bool is_q = hs < nh;
    const int g = hs - nh;
    const int col0 = is_q ? hs * d : qd + g * d;
    const float* pr = part + t * ldp;
    auto value = [&](int col) {
        float v[SP];
#pragma unroll
        for (int s = 0; s < SP; ++s) v[s] = pr[(int64_t)(s < splits ? s : 0) * split_stride + col];
        float acc = v[0];
#pragma unroll
        for (int s = 1; s < SP; ++s) acc += s < splits ? v[s] : 0.f;
        if (bias) acc += zi_load(bias + col);
        return acc;
    };
    T* dst;
    int64_t vbase = 0;
    bool store_v = false;
    if (is_q) {
        dst = q_out + t * ldq + (int64_t)hs * d;
    } else {
        const ZiSlotPlace place = zi_slot_place(slots[t], cache_slots, page_size);
        if (!place.ok) return;  // the host checks the range; never write outside the pool
        dst = kcache + zi_key_offset(place.page, g, place.off, nkv, page_size, d);
        vbase = zi_value_offset(place.page, g, 0, place.off, nkv, page_size, d);
        store_v = true;
    }
    for (int j = lane; j < half; j += ZI_WAVE) {
        const float a = value(col0 + j), b = value(col0 + j + half);
        const float2 e = table[t * half + j];
        zi_store(dst + j, a * e.x - b * e.y);
        zi_store(dst + j + half, b * e.x + a * e.y);
    }
    for (int j = rot + lane; j < d; j += ZI_WAVE) zi_store(dst + j, value(col0 + j));
    if (store_v)
        for (int j = lane; j < d; j += ZI_WAVE) zi_store(vcache + vbase + (int64_t)j * page_size, value(qd + kvd + g * d + j));
}

extern "C" int zi_rope_kv_store_split(void* q_out, int dt, int64_t ldq, const float* part, int splits,
                                      int64_t split_stride, int64_t ldp, const void* bias, int bias_dt, int n,
                                      const int32_t* slots, const float* table, void* kcache,
                                      void* vcache, int64_t cache_slots, int nh, int nkv, int d, int rot,
                                      int page_size, int write_kv, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv >= 0 && d > 0, "rope_kv_store_split: bad sizes");
    ZI_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "rope_kv_store_split: rotary dims %d must be even and <= head_dim %d",
               rot, d);
    const int64_t width = (int64_t)nh * d + (write_kv ? 2 * (int64_t)nkv * d : 0);
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldp >= width, "rope_kv_store_split: row stride too small");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || split_stride >= (int64_t)n * ldp),
               "rope_kv_store_split: bad partial sums (splits %d, stride %lld)", splits, (long long)split_stride);
    ZI_REQUIRE(rot == 0 || (table && ((uintptr_t)table % 8) == 0), "rope_kv_store_split: no table of angles");
    if (write_kv) {
        ZI_REQUIRE(page_size > 0 && cache_slots > 0 && cache_slots % page_size == 0,
                   "rope_kv_store_split: cache of %lld slots is not a whole number of pages of %d", (long long)cache_slots,
                   page_size);
        ZI_REQUIRE(kcache && vcache && slots, "rope_kv_store_split: null cache pointer");
    }
    ZI_REQUIRE(splits <= 16, "rope_kv_store_split: at most 16 splits (%d)", splits);
    ZI_REQUIRE(nh + nkv <= 65535, "rope_kv_store_split: too many heads");
    if (n == 0) return 0;
    if (!bias) bias_dt = ZI_F32;
    const dim3 grid(n, nh + (write_kv ? nkv : 0));
#define ZI_RKS(SP)                                                                                                  \
    rope_kv_store_split_kernel<T, TB, SP><<<grid, ZI_WAVE, 0, stream>>>(                                            \
        (T*)q_out, ldq, part, splits, split_stride, ldp, (const TB*)bias, slots, reinterpret_cast<const float2*>(table), \
        (T*)kcache, (T*)vcache, \
        nh, nkv, d, rot, page_size, cache_slots)
    ZI_DISPATCH_DTYPE(dt, T, ZI_DISPATCH_DTYPE(bias_dt, TB, {
        if (splits <= 1) ZI_RKS(1);
        else if (splits <= 2) ZI_RKS(2);
        else if (splits <= 4) ZI_RKS(4);
        else if (splits <= 8) ZI_RKS(8);
        else ZI_RKS(16);
    }));
#undef ZI_RKS
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

// cos and sin of every (token, pair) angle: out[t][k] = (cos, sin)(pos[t] * inv_freq[k]), float32.  The
// angles of a step do not depend on the layer; kernels that take this table skip their own sincosf.
__global__ void rope_table_kernel(float* __restrict__ out, const int32_t* __restrict__ pos,
                                  const float* __restrict__ inv_freq, int64_t total, int half) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t t = i / half;
    const int k = (int)(i % half);
    float s, c;
    sincosf((float)pos[t] * inv_freq[k], &s, &c);
    out[2 * i] = c;
    out[2 * i + 1] = s;
}

extern "C" int zi_rope_table(float* out, const int32_t* pos, const float* inv_freq, int n, int half,
                             hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && half >= 0, "rope_table: bad sizes");
    ZI_REQUIRE(half == 0 || (out && pos && inv_freq), "rope_table: null pointer");
    const int64_t total = (int64_t)n * half;
    if (total == 0) return 0;
    rope_table_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(out, pos, inv_freq, total, half);
    return zi_check_launch("rope_table");
}
