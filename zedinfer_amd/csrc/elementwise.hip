// Row gathers and elementwise ops: embedding lookup, row gather, residual add,
// SwiGLU.  Arithmetic is done in float32 and rounded once on store.
#include "zi_common.h"
#include "zi_api.h"

// out[i,:] = table[ids[i],:]   (reference: src/backend/ops/embedding/cpu/embedding_cpu.cpp:10-23).
// An id outside [0, V) writes NaN into the row so that the fault shows.
template <typename TW, typename TO>
__global__ void embedding_kernel(TO* __restrict__ out, const TW* __restrict__ table,
                                 const int32_t* __restrict__ ids, int H, int V) {
    const int64_t row = blockIdx.x;
    const int id = ids[row];
    const bool ok = id >= 0 && id < V;
    const TW* src = table + (int64_t)(ok ? id : 0) * H;
    TO* dst = out + row * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) zi_store(dst + j, ok ? zi_load(src + j) : NAN);
}

extern "C" int zi_embedding(void* out, int out_dt, const void* table, int table_dt, const int32_t* ids,
                            int n, int hidden, int vocab, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(table_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        embedding_kernel<TW, TO><<<n, 256, 0, stream>>>((TO*)out, (const TW*)table, ids, hidden, vocab);
    }));
    return zi_check_launch("embedding");
}

// out[i,:] = in[idx[i],:]
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ in,
                                   const int32_t* __restrict__ idx, int H, int n_in) {
    const int64_t row = blockIdx.x;
    const int s = idx[row];
    const bool ok = s >= 0 && s < n_in;
    const T* src = in + (int64_t)(ok ? s : 0) * H;
    T* dst = out + row * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) zi_store(dst + j, ok ? zi_load(src + j) : NAN);
}

extern "C" int zi_gather_rows(void* out, const void* in, int dt, const int32_t* idx, int n_out, int n_in,
                              int hidden, hipStream_t stream) {
    ZI_REQUIRE(n_out >= 0 && n_in >= 0 && hidden > 0, "gather_rows: bad sizes");
    if (n_out == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        gather_rows_kernel<T><<<n_out, 256, 0, stream>>>((T*)out, (const T*)in, idx, hidden, n_in);
    });
    return zi_check_launch("gather_rows");
}

// c = a + b, added in float32 (reference: src/backend/ops/add/cpu/add_cpu_opt.cpp:22-24,57-59).
template <typename TA, typename TB, typename TC>
__global__ void add_kernel(TC* __restrict__ c, const TA* __restrict__ a, const TB* __restrict__ b, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        zi_store(c + i, zi_load(a + i) + zi_load(b + i));
}

extern "C" int zi_add(void* c, int c_dt, const void* a, int a_dt, const void* b, int b_dt, int64_t n,
                      hipStream_t stream) {
    ZI_REQUIRE(n >= 0, "add: negative size");
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
    ZI_DISPATCH_DTYPE(a_dt, TA, ZI_DISPATCH_DTYPE(b_dt, TB, ZI_DISPATCH_DTYPE(c_dt, TC, {
        add_kernel<TA, TB, TC><<<blocks, 256, 0, stream>>>((TC*)c, (const TA*)a, (const TB*)b, n);
    })));
    return zi_check_launch("add");
}

// out[i,j] = up[i,j] * gate[i,j] / (1 + exp(-gate[i,j]))
// (reference: src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).  gate and up are read with their
// own row strides, so both halves of one fused [n, 2I] product can be passed.  With
// `interleave` = B > 0 they are columns of ONE matrix in blocks of B: gate column j sits at
// (j / B) * 2B + j % B of `gate`, up column j another B further (`up` is not used).  The input
// may come as `splits` partial sums (split s at + s * split_stride), added in rising order.
template <typename TI, typename TO>
__global__ void swiglu_kernel(TO* __restrict__ out, const TI* __restrict__ gate, const TI* __restrict__ up,
                              int inter, int64_t ld_gate, int64_t ld_up, int interleave, int splits,
                              int64_t split_stride) {
    const int64_t row = blockIdx.y;
    const TI* g = gate + row * ld_gate;
    const TI* u = interleave > 0 ? g + interleave : up + row * ld_up;
    TO* o = out + row * (int64_t)inter;
    for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < inter; j += gridDim.x * blockDim.x) {
        const int64_t c = interleave > 0 ? (int64_t)(j / interleave) * 2 * interleave + j % interleave : j;
        float gv = zi_load(g + c), uv = zi_load(u + c);
        for (int s = 1; s < splits; ++s) {
            gv += zi_load(g + s * split_stride + c);
            uv += zi_load(u + s * split_stride + c);
        }
        zi_store(o + j, uv * (gv / (1.f + expf(-gv))));
    }
}

// The common case at full speed: bfloat16 in and out, gate and up interleaved in blocks of 8, no
// partial sums.  A thread reads the 16 bytes of 8 gate values and the 16 bytes of their up values and
// writes 16 bytes.
__global__ void __launch_bounds__(256)
swiglu_il8_kernel(zi_bf16* __restrict__ out, const zi_bf16* __restrict__ gu, int64_t n_groups, int groups_per_row,
                  int64_t ld) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_groups; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / groups_per_row;
        const int grp = (int)(i - row * groups_per_row);
        const zi_bf16* src = gu + row * ld + (int64_t)grp * 16;
        const uint4 g = *reinterpret_cast<const uint4*>(src);
        const uint4 u = *reinterpret_cast<const uint4*>(src + 8);
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
        uint32_t ow[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
            ow[k] = zi_pack_bf16x2(u0 * (g0 / (1.f + expf(-g0))), u1 * (g1 / (1.f + expf(-g1))));
        }
        *reinterpret_cast<uint4*>(out + i * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
}

// The same from the transposed product: gut [2I, n] holds, for every block of 8 channels, 8 rows of gate
// values over the n tokens and then the 8 rows of their up values (the matrix product of the stacked
// weight with x^T, which the library sometimes makes faster than x with the weight transposed).  Writes
// out [n, I].  A workgroup takes 64 channels x 64 tokens: a thread reads 16 bytes (8 tokens) of the gate
// and up rows of two neighbouring channels, the tile turns in LDS (4-byte words of two channels, rows of
// 33 words), and every token's 64 channels leave as 128 contiguous bytes.  n % 8 == 0, I % 8 == 0.
__global__ void __launch_bounds__(256)
swiglu_il8_t_kernel(zi_bf16* __restrict__ out, const zi_bf16* __restrict__ gut, int n, int inter, int64_t ldt) {
    __shared__ uint32_t tile[64 * 33];
    const int c0 = blockIdx.x * 64, m0 = blockIdx.y * 64, tid = threadIdx.x;
    {
        const int tg = tid % 8, cp = tid / 8;                 // eight tokens, a pair of channels
        const int c = c0 + 2 * cp, m = m0 + tg * 8;
        if (c < inter && m < n) {                              // inter and n are multiples of 8: whole pieces
            const zi_bf16* g = gut + (int64_t)((c / 8) * 16 + c % 8) * ldt + m;
            const uint4 ga = *reinterpret_cast<const uint4*>(g), gb = *reinterpret_cast<const uint4*>(g + ldt);
            const uint4 ua = *reinterpret_cast<const uint4*>(g + 8 * ldt), ub = *reinterpret_cast<const uint4*>(g + 9 * ldt);
            const uint32_t gaw[4] = {ga.x, ga.y, ga.z, ga.w}, gbw[4] = {gb.x, gb.y, gb.z, gb.w};
            const uint32_t uaw[4] = {ua.x, ua.y, ua.z, ua.w}, ubw[4] = {ub.x, ub.y, ub.z, ub.w};
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int sh = (k & 1) * 16;
                const float g0 = __uint_as_float((gaw[k / 2] >> sh) << 16), g1 = __uint_as_float((gbw[k / 2] >> sh) << 16);
                const float u0 = __uint_as_float((uaw[k / 2] >> sh) << 16), u1 = __uint_as_float((ubw[k / 2] >> sh) << 16);
                tile[(tg * 8 + k) * 33 + cp] = zi_pack_bf16x2(u0 * (g0 / (1.f + expf(-g0))), u1 * (g1 / (1.f + expf(-g1))));
            }
        }
    }
    __syncthreads();
    {
        const int tok = tid / 4, q = tid % 4;                  // a token, 16 of the 64 channels
        const int m = m0 + tok, c = c0 + q * 16;
        if (m < n && c < inter) {
            const uint32_t* src = tile + tok * 33 + q * 8;
            zi_bf16* dst = out + (int64_t)m * inter + c;
            *reinterpret_cast<uint4*>(dst) = make_uint4(src[0], src[1], src[2], src[3]);
            if (c + 8 < inter) *reinterpret_cast<uint4*>(dst + 8) = make_uint4(src[4], src[5], src[6], src[7]);
        }
    }
}

// out [n, inter] from gut [2 * inter, n] (row stride ldt), bfloat16, gate and up rows in blocks of 8.
extern "C" int zi_swiglu_t(void* out, const void* gut, int dt, int n, int inter, int64_t ldt, hipStream_t stream) {
    ZI_REQUIRE(dt == ZI_BF16, "swiglu_t: bfloat16 only");
    ZI_REQUIRE(n >= 0 && inter > 0 && n % 8 == 0 && inter % 8 == 0 && ldt >= n && ldt % 8 == 0,
               "swiglu_t: tokens %d and channels %d must be multiples of 8 (row stride %lld)", n, inter, (long long)ldt);
    ZI_REQUIRE(((uintptr_t)out % 16) == 0 && ((uintptr_t)gut % 16) == 0, "swiglu_t: pointers must be aligned to 16 bytes");
    if (n == 0) return 0;
    const dim3 grid((inter + 63) / 64, (n + 63) / 64);
    ZI_REQUIRE(grid.y <= 65535, "swiglu_t: too many tokens");
    swiglu_il8_t_kernel<<<grid, 256, 0, stream>>>((zi_bf16*)out, (const zi_bf16*)gut, n, inter, ldt);
    return zi_check_launch("swiglu_t");
}

extern "C" int zi_swiglu(void* out, int out_dt, const void* gate, const void* up, int dt, int n, int inter,
                         int64_t ld_gate, int64_t ld_up, int interleave, int splits, int64_t split_stride,
                         hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && inter > 0 && ld_gate >= inter, "swiglu: bad sizes n=%d inter=%d", n, inter);
    ZI_REQUIRE(interleave >= 0 && (interleave == 0 ? (up != nullptr && ld_up >= inter)
                                                   : (inter % interleave == 0 && ld_gate >= 2 * (int64_t)inter)),
               "swiglu: bad layout (interleave %d)", interleave);
    ZI_REQUIRE(splits >= 1, "swiglu: bad number of partial sums");
    if (n == 0) return 0;
    if (interleave == 8 && splits == 1 && dt == ZI_BF16 && out_dt == ZI_BF16 && ld_gate % 8 == 0 &&
        ((uintptr_t)gate % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        const int64_t groups = (int64_t)n * (inter / 8);
        int64_t blocks = (groups + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        swiglu_il8_kernel<<<(int)blocks, 256, 0, stream>>>((zi_bf16*)out, (const zi_bf16*)gate, groups, inter / 8, ld_gate);
        return zi_check_launch("swiglu");
    }
    ZI_REQUIRE(n <= 65535 * 1024, "swiglu: too many rows");
    int bx = (inter + 255) / 256;
    if (bx > 64) bx = 64;
    // gridDim.y is limited to 65535: fold larger batches.
    for (int r0 = 0; r0 < n; r0 += 65535) {
        const int rows = n - r0 < 65535 ? n - r0 : 65535;
        ZI_DISPATCH_DTYPE(dt, TI, ZI_DISPATCH_DTYPE(out_dt, TO, {
            swiglu_kernel<TI, TO><<<dim3(bx, rows), 256, 0, stream>>>(
                (TO*)out + (int64_t)r0 * inter, (const TI*)gate + (int64_t)r0 * ld_gate,
                up ? (const TI*)up + (int64_t)r0 * ld_up : nullptr, inter, ld_gate, ld_up, interleave, splits,
                split_stride);
        }));
    }
    return zi_check_launch("swiglu");
}
