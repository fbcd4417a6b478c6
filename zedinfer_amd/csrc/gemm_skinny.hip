// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for few rows of x: the decode-time matrix product,
// bound by the one pass over the weights.  Up to 16 rows run on the kernel in this file, 17 to 64
// on the one in gemm_mid.hip; this file holds the entry point of both.
//
// bfloat16 x and w, float32 accumulation on the matrix cores
// (v_mfma_f32_16x16x32_bf16).  A workgroup of four wavefronts owns tiles of 16 weight
// rows and a range of k: each wavefront takes KPW consecutive k-blocks of 128, the
// four sums are added through LDS in the order of the wavefronts.  When the weight
// matrix is small the k dimension is additionally cut over several workgroups
// (gridDim.y "splits") so that enough loads are in flight to fill HBM; those write
// float32 partial sums [split][M][N] that the consumer adds in rising order (the next
// norm, the rotary kernel, the SwiGLU kernel, or the reduce kernel here).  The cut
// depends on N and K only, so a row's result does not depend on how many rows ride
// along.  With up to 16 rows of x a workgroup keeps its slice of x in registers and
// walks several weight tiles, prefetching the next tile's rows while the matrix
// cores work on the current one.
//
// Epilogues: plain (bias, bfloat16 or float32 out), partial sums, and SwiGLU: when the
// weight rows are gate and up rows interleaved in blocks of 8 (tile = 8 gate rows, then
// the 8 up rows of the same columns), the tile's lanes exchange halves and write
// act = up * gate / (1 + exp(-gate)) (reference: src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).
//
// Operand layout.  For one MFMA the A operand is a 16 x 32 tile of w (lane l: row l%16, the eight
// consecutive k starting at 8 * (l/16)) and the B operand the matching 32 x 16 tile of x^T (lane l: row
// l%16 of x, the same eight k).  A k-block of 128 is four such MFMAs.  x is loaded in that layout; the
// weights are loaded as whole cache lines and rearranged through LDS.
#include "zi_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define SK_ROWS 16
#define SK_KB 128
#define SK_WS (SK_KB + 8)   // LDS row stride of a weight tile, in elements
#define SK_WAVES 4
#define SK_MAX_KPW 4
#define SK_RESIDENT_WGS 480   // workgroups that are surely resident at once (256 compute units, two each)
#define SK_ENOUGH_WGS 256
#define SK_MAX_TPW 32

#define SK_MODE_PLAIN 0
#define SK_MODE_PARTIAL 1
#define SK_MODE_SWIGLU 2

// 16 bytes as a native vector (copies of the struct uint4 are memcpys to the compiler, and an array of
// them that is only copied may stay in memory instead of registers)
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t& v) {
    union { u32x4_t u; bf16x8_t b; } c;
    c.u = v;
    return c.b;
}

// The four 16-byte pieces of x row `row` this lane owns in k-block `kb`, in the matrix-core operand layout:
// piece c holds k = kb*128 + c*32 + j*8 .. +8.  Pieces past K, and all pieces when `live` is false, are zero.
__device__ __forceinline__ void sk_load_x(u32x4_t (&dst)[4], const zi_bf16* row, int kb, int j, int K, bool live) {
    const int k0 = kb * SK_KB + j * 8;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int k = k0 + c * 32;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(row + (k < K ? k : K - 8));
        dst[c] = (live && k < K) ? v : u32x4_t{0u, 0u, 0u, 0u};
    }
}

template <int KPW>
__global__ void __launch_bounds__(SK_WAVES* ZI_WAVE)
gemm_skinny_kernel(void* __restrict__ out, int mode, int out_f32, const zi_bf16* x, const zi_bf16* __restrict__ w,
                   const zi_bf16* __restrict__ bias, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                   int tiles_per_wg, int vec_out) {
    constexpr int MT = 1;              // up to 16 rows of x: one matrix-core tile
    __shared__ f32x4_t red[2][SK_WAVES][MT][ZI_WAVE];
    __shared__ __attribute__((aligned(16))) uint16_t wt[SK_WAVES][SK_ROWS * SK_WS];   // a wavefront's weight tile
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int split = blockIdx.y;
    const int kb_total = (K + SK_KB - 1) / SK_KB;
    const int kb0 = split * (SK_WAVES * KPW) + wave * KPW;
    const int n_tiles = (N + SK_ROWS - 1) / SK_ROWS;
    const int tile_lo = blockIdx.x * tiles_per_wg;
    const int tile_hi = (tile_lo + tiles_per_wg < n_tiles) ? tile_lo + tiles_per_wg : n_tiles;

    const zi_bf16* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r;
        xrow[t] = x + (int64_t)(m < M ? m : M - 1) * ldx;
    }
    // The slice of x stays in registers over the workgroup's tiles.  It is zero past K and for k-blocks past
    // the last one (a wavefront that has fewer than KPW blocks reads the last block again and multiplies
    // it by zero).
    const int kb_last = kb_total - 1;
    u32x4_t xr[KPW][4];
#pragma unroll
    for (int i = 0; i < KPW; ++i)
        sk_load_x(xr[i], xrow[0], kb0 + i < kb_total ? kb0 + i : kb_last, j, K, kb0 + i < kb_total);
    // Weights are read as whole cache lines: a load instruction takes 4 rows x 256 bytes (lane l: row
    // l / 16 of the four, 16-byte piece l % 16), four instructions a tile of 16 rows x one k-block.  Loads
    // in the operand layout (16 rows x 64 bytes an instruction) were measured a fifth slower.  A tile is
    // turned into operands through a piece of LDS that the wavefront owns.  No branch goes around a load
    // (pieces past K are read from the row's last piece instead, K % 8 == 0; x is zero there), so that the
    // compiler lets the loads of two tiles stay in flight.
    const int wq = lane & 15;
    int wk[KPW];
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
        const int k = (kb0 + i < kb_total ? kb0 + i : kb_last) * SK_KB + wq * 8;
        wk[i] = k < K ? k : K - 8;
    }
    uint16_t* wt_put = &wt[wave][j * SK_WS + wq * 8];        // + c * 4 rows
    const uint16_t* wt_get = &wt[wave][r * SK_WS + j * 8];   // + c * 32 values
    u32x4_t ring[2][KPW][4];
    auto issue = [&](u32x4_t (&dst)[KPW][4], int tile) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int n = tile * SK_ROWS + c * 4 + j;
            const zi_bf16* row = w + (int64_t)(n < N ? n : N - 1) * ldw;
#pragma unroll
            for (int i = 0; i < KPW; ++i) dst[i][c] = *reinterpret_cast<const u32x4_t*>(row + wk[i]);
        }
    };
    int buf = 0;
    auto process = [&](u32x4_t (&a)[KPW][4], int tile) {
        f32x4_t acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KPW; ++i) {
            // LDS serves a wavefront's instructions in order: no barrier between put and get, and the
            // next block's put cannot overtake this block's get
            u32x4_t b[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) *reinterpret_cast<u32x4_t*>(wt_put + c * 4 * SK_WS) = a[i][c];
#pragma unroll
            for (int c = 0; c < 4; ++c) b[c] = *reinterpret_cast<const u32x4_t*>(wt_get + c * 32);
#pragma unroll
            for (int c = 0; c < 4; ++c)
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(b[c]), as_bf16x8(xr[i][c]), acc[0], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) red[buf][wave][t][lane] = acc[t];
        __syncthreads();
        // wave t of the workgroup finishes row tile t of x: C[n = (lane/16)*4 + e][m = lane%16]
        const int n0 = tile * SK_ROWS;
        for (int t = wave; t < MT; t += SK_WAVES) {
            f32x4_t s = red[buf][0][t][lane];
#pragma unroll
            for (int q = 1; q < SK_WAVES; ++q) {
                const f32x4_t o = red[buf][q][t][lane];
                s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
            }
            const int m = t * 16 + r;
            if (mode == SK_MODE_SWIGLU) {
                // lanes j = 0,1 hold gate rows j*4 + e, lanes j = 2,3 the up rows of the same columns
                f32x4_t up;
                up[0] = __shfl_xor(s[0], 32, ZI_WAVE); up[1] = __shfl_xor(s[1], 32, ZI_WAVE);
                up[2] = __shfl_xor(s[2], 32, ZI_WAVE); up[3] = __shfl_xor(s[3], 32, ZI_WAVE);
                if (j >= 2 || m >= M) continue;
                const int col = tile * 8 + j * 4;     // N / 2 columns of output
                zi_bf16* dst = (zi_bf16*)out + (int64_t)m * ldo + col;
                float act[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) act[e] = up[e] * (s[e] / (1.f + expf(-s[e])));
                if (vec_out) {   // N % 16 == 0: the four columns exist
                    uint2 pk;
                    pk.x = (uint32_t)zi_float_to_bf16(act[0]) | ((uint32_t)zi_float_to_bf16(act[1]) << 16);
                    pk.y = (uint32_t)zi_float_to_bf16(act[2]) | ((uint32_t)zi_float_to_bf16(act[3]) << 16);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N / 2) zi_store(dst + e, act[e]);
                }
                continue;
            }
            if (m >= M) continue;
            const int nb = n0 + j * 4;   // this lane's four consecutive columns
            if (nb + 3 < N && vec_out) {
                if (mode == SK_MODE_PARTIAL) {
                    *reinterpret_cast<f32x4_t*>((float*)out + ((int64_t)split * M + m) * N + nb) = s;
                } else {
                    if (bias) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) s[e] += zi_load(bias + nb + e);
                    }
                    if (out_f32) {
                        *reinterpret_cast<f32x4_t*>((float*)out + (int64_t)m * ldo + nb) = s;
                    } else {
                        uint2 pk;
                        pk.x = (uint32_t)zi_float_to_bf16(s[0]) | ((uint32_t)zi_float_to_bf16(s[1]) << 16);
                        pk.y = (uint32_t)zi_float_to_bf16(s[2]) | ((uint32_t)zi_float_to_bf16(s[3]) << 16);
                        *reinterpret_cast<uint2*>((zi_bf16*)out + (int64_t)m * ldo + nb) = pk;
                    }
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = nb + e;
                if (n >= N) continue;
                if (mode == SK_MODE_PARTIAL) {
                    ((float*)out)[((int64_t)split * M + m) * N + n] = s[e];
                } else {
                    const float v = s[e] + (bias ? zi_load(bias + n) : 0.f);
                    if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = v;
                    else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, v);
                }
            }
        }
        buf ^= 1;
    };
    // Two buffers take turns: while one tile is worked on the next one's rows travel.  Every load sits in
    // straight-line code (the last tile is peeled off instead of guarding its prefetch), which is what lets
    // the compiler wait for the older loads only.
    issue(ring[0], tile_lo);
    int tile = tile_lo;
    for (; tile + 2 < tile_hi; tile += 2) {
        issue(ring[1], tile + 1);
        process(ring[0], tile);
        issue(ring[0], tile + 2);
        process(ring[1], tile + 1);
    }
    if (tile + 1 < tile_hi) {
        issue(ring[1], tile + 1);
        process(ring[0], tile);
        process(ring[1], tile + 1);
    } else {
        process(ring[0], tile);
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

// How the product with a weight matrix [N, K] is cut: k-blocks per wavefront, splits of k over
// workgroups, and weight tiles per workgroup.  A function of N and K alone.
//
// The kernel is bound by memory latency and bandwidth, so what counts is that all its workgroups are
// resident at once (two per compute unit fit: no second round that runs half empty) and that there are
// many of them.  Among the cuts with at most SK_RESIDENT_WGS workgroups the one with the fewest splits
// that still gives SK_ENOUGH_WGS workgroups is taken (fewer partial sums to write and add), then the one
// with the most workgroups.
static void skinny_plan(int N, int K, int* kpw, int* splits, int* tiles_per_wg) {
    const int tiles = (N + SK_ROWS - 1) / SK_ROWS;
    const int kb_total = (K + SK_KB - 1) / SK_KB;
    int best_k = 1, best_s = (kb_total + SK_WAVES - 1) / SK_WAVES, best_t = SK_MAX_TPW;
    int64_t best_w = -1;
    bool best_enough = false;
    for (int c = SK_MAX_KPW; c >= 1; --c) {
        const int s = (kb_total + SK_WAVES * c - 1) / (SK_WAVES * c);
        if (c > 1 && (kb_total + SK_WAVES * (c - 1) - 1) / (SK_WAVES * (c - 1)) == s)
            continue;   // fewer k-blocks a wavefront give the same splits: more wavefronts busy
        for (int t = 1; t <= SK_MAX_TPW; ++t) {
            const int64_t w = (int64_t)s * ((tiles + t - 1) / t);
            if (w > SK_RESIDENT_WGS && t < SK_MAX_TPW) continue;
            const bool enough = w >= SK_ENOUGH_WGS;
            bool better;
            if (best_w < 0) better = true;
            else if (enough != best_enough) better = enough;
            else if (enough) better = s < best_s || (s == best_s && w > best_w);
            else better = w > best_w || (w == best_w && s < best_s);
            if (better) { best_k = c; best_s = s; best_t = t; best_w = w; best_enough = enough; }
            break;   // larger t only gives fewer workgroups
        }
    }
    *kpw = best_k;
    *splits = best_s;
    *tiles_per_wg = best_t;
}

extern "C" int zi_gemm_skinny_supported(int M, int N, int K, int64_t ldx, int64_t ldw) {
    return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

// The kernel for 17..64 rows (gemm_mid.hip): its cut and its launch.
void zi_gemm_mid_plan(int N, int K, int* splits, int* kb_per_split, int* waves);
int zi_gemm_mid_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                       int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream);

// From how many rows of x on the kernel that stages x in LDS (gemm_mid.hip) is taken.  It must be taken
// beyond 16 rows (the kernel in this file holds one matrix-core tile of x); below, the choice is by speed.
static int g_mid_min_rows = 1;
extern "C" int zi_gemm_skinny_mid_min_rows(int rows) {
    const int before = g_mid_min_rows;
    if (rows >= 1 && rows <= 17) g_mid_min_rows = rows;
    return before;
}

// Splits of k for M rows against a weight matrix [N, K]: the leading dimension of the partial sums.  A
// function of N, K and of which of the two kernels takes M rows (they cut differently).
extern "C" int zi_gemm_skinny_splits(int M, int N, int K) {
    int kpw, s, tpw, waves;
    if (M >= g_mid_min_rows) zi_gemm_mid_plan(N, K, &s, &tpw, &waves);
    else skinny_plan(N, K, &kpw, &s, &tpw);
    return s;
}

// Floats of workspace for the split partials (0 when the product is not split).
extern "C" int64_t zi_gemm_skinny_workspace(int M, int N, int K) {
    const int s = zi_gemm_skinny_splits(M, N, K);
    return s > 1 ? (int64_t)s * M * N : 0;
}

static void sk_launch(int kpw, dim3 grid, hipStream_t stream, void* out, int mode, int out_f32, const zi_bf16* x,
                      const zi_bf16* w, const zi_bf16* bias, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                      int tpw, int vec_out) {
#define ZI_SK(KPW)                                                                                                  \
    gemm_skinny_kernel<KPW><<<grid, SK_WAVES * ZI_WAVE, 0, stream>>>(out, mode, out_f32, x, w, bias, M, N, K, ldx, ldw, \
                                                                     ldo, tpw, vec_out)
    switch (kpw) {
        case 1: ZI_SK(1); break;
        case 2: ZI_SK(2); break;
        case 3: ZI_SK(3); break;
        default: ZI_SK(4); break;
    }
#undef ZI_SK
}

// mode 0: out[M,N] (+ bias), reduced through `workspace` when the product is split.
// mode 1: out = float32 partial sums [splits][M][N] (no bias; splits from zi_gemm_skinny_splits).
// mode 2: w holds gate and up rows interleaved in blocks of 8; out[M, N/2] (bfloat16) =
//         up * silu(gate); only for products that are not split.
extern "C" int zi_gemm_skinny(void* out, int out_dt, int mode, const void* x, const void* w, const void* bias, int M,
                              int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, float* workspace,
                              int64_t workspace_floats, hipStream_t stream) {
    ZI_REQUIRE(zi_gemm_skinny_supported(M, N, K, ldx, ldw),
               "gemm_skinny: unsupported sizes M=%d N=%d K=%d (1 <= M <= 64, K and row strides multiples of 8)", M, N, K);
    ZI_REQUIRE(out_dt == ZI_F32 || out_dt == ZI_BF16, "gemm_skinny: unknown output dtype %d", out_dt);
    ZI_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny: unknown mode %d", mode);
    ZI_REQUIRE(ldx >= K && ldw >= K, "gemm_skinny: leading dimension too small");
    ZI_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny: x and w must be 16-byte aligned");
    int kpw = 1, splits, tpw, mid_waves;
    const int mt = (M + 15) / 16;
    const bool mid = M >= g_mid_min_rows;
    if (mid) zi_gemm_mid_plan(N, K, &splits, &tpw, &mid_waves);    // more than 16 rows: the kernel that stages x in LDS
    else skinny_plan(N, K, &kpw, &splits, &tpw);
    const int tiles = (N + SK_ROWS - 1) / SK_ROWS;
    const dim3 grid((tiles + tpw - 1) / tpw, splits);
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
    if (mid) {
        const int rc = zi_gemm_mid_launch(dst, of32, kmode, (const zi_bf16*)x, (const zi_bf16*)w, b, M, N, K, ldx, ldw, ldo,
                                          vec_out, stream);
        if (rc) return rc;
    } else {
        sk_launch(kpw, grid, stream, dst, kmode, of32, (const zi_bf16*)x, (const zi_bf16*)w, b, M, N, K, ldx, ldw, ldo, tpw,
                     vec_out);
    }
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
