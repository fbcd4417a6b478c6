// out[M,N] = x[M,K] . w[N,K]^T for 65 .. 256 rows of x: large decode batches, still bound by the one pass over
// the weights, where the kernels of gemm_mid.hip (16 weight rows a wavefront) are bound by their reads of x from
// LDS: every operand of x they read serves 16 weight rows.  Here a wavefront owns 32 weight rows and multiplies
// with v_mfma_f32_32x32x16_bf16 (a 32 x 32 tile of sums in 16 registers a lane), so an operand of x serves
// twice the weights, and a workgroup reads half as much of x for the same weights.
//
// A workgroup of 4 or 8 wavefronts walks its range of k in blocks of 64.  The block's slice of x (up to 256
// rows x 64 values) lies in LDS, in one of two buffers: the next block's slice is stored while this one is
// read, one barrier a block.  Each wavefront reads its 32 weight rows from memory as whole lines of 128 bytes
// (an instruction takes 8 rows), several blocks ahead (a ring of register buffers; loads are issued without
// branches so that they stay in flight), and turns a block into matrix-core operands through a piece of LDS of
// its own.  LDS rows are 128 bytes, the 16-byte piece c of row r at place c xor ((r / 2) mod 8): sixteen
// lanes that read one piece of sixteen rows then touch every bank once.
// k is cut over gridDim.y workgroups when N alone gives too few; the cut depends on N and K only (not on M
// within this kernel's range), the partial sums [split][M][N] are added by the consumer in rising order.
// Epilogues as in gemm_mid.hip: plain (bias), partial sums, SwiGLU over gate/up rows interleaved in blocks of
// 8 (in a tile of 32 rows a gate row and its up row are the same lane's registers v and v + 4).
// (reference: src/backend/ops/linear/cpu/linear_cpu.cpp:26-85 for what is computed.)
#include "zi_common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 g32_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float g32_f32x16_t;
typedef __attribute__((ext_vector_type(4))) float g32_f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned g32_u32x4_t;

#define G32_KB 64           // values of k a block
#define G32_ROW 64          // LDS row stride in elements (128 bytes, 8 pieces of 16 bytes)
#define G32_MODE_PLAIN 0
#define G32_MODE_PARTIAL 1
#define G32_MODE_SWIGLU 2

union g32_pack {
    g32_u32x4_t u;
    g32_bf16x8_t b;
};

__device__ __forceinline__ g32_u32x4_t g32_keep(g32_u32x4_t v, bool keep) { return v & (0u - (unsigned)keep); }
// where the 16-byte piece c of LDS row r lies, in elements from the tile's start
__device__ __forceinline__ int g32_at(int r, int c) { return r * G32_ROW + ((c ^ ((r >> 1) & 7)) << 3); }

template <int MT, int WAVES, int RING>
__global__ void __launch_bounds__(WAVES* ZI_WAVE)
gemm_rows32_kernel(void* __restrict__ out, int mode, int out_f32, const zi_bf16* __restrict__ x,
                   const zi_bf16* __restrict__ w, const zi_bf16* __restrict__ bias, int M, int N, int K, int64_t ldx,
                   int64_t ldw, int64_t ldo, int kb_per_split, int vec_out) {
    constexpr int THREADS = WAVES * ZI_WAVE;
    constexpr int XP = (MT * 32 * 8 + THREADS - 1) / THREADS;      // pieces of a block's x slice a thread stages
    __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 32 * G32_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t wt[WAVES][32 * G32_ROW];
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r32 = lane & 31, kh = lane >> 5;        // operand row, and which 8 of a k-step's 16 values
    const int split = blockIdx.y;
    const int kb_total = (K + G32_KB - 1) / G32_KB;
    const int kb_lo = split * kb_per_split;
    const int kb_hi = (kb_lo + kb_per_split < kb_total) ? kb_lo + kb_per_split : kb_total;
    const int n0 = (blockIdx.x * WAVES + wave) * 32;
    // weights: instruction q takes rows q * 8 + lane / 8, 16-byte piece lane % 8 of the block
    const int wr = lane >> 3, wc = lane & 7;
    const zi_bf16* wrow[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int n = n0 + q * 8 + wr;
        wrow[q] = w + (int64_t)(n < N ? n : N - 1) * ldw;
    }
    uint16_t* const wt_w = &wt[wave][0];
    // x: piece i = tid + p * THREADS of the slice is (row i / 8, piece i % 8); rows past M repeat the last
    const zi_bf16* xrow[XP];
    int xdst[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) {
        const int i = tid + p * THREADS, row = i >> 3;
        xrow[p] = x + (int64_t)(row < M ? row : M - 1) * ldx;
        xdst[p] = i < MT * 32 * 8 ? g32_at(row, i & 7) : -1;
    }
    const int xc = tid & 7;      // THREADS is a multiple of 8: the piece index is the same for every p
    g32_u32x4_t ring[RING][4], xnext[XP];
    auto fetch_x = [&](int kb) __attribute__((always_inline)) {
        const int k0 = (kb < kb_hi ? kb : kb_hi - 1) * G32_KB;
        const int kx = k0 + xc * 8 < K ? k0 + xc * 8 : K - 8;
#pragma unroll
        for (int p = 0; p < XP; ++p) xnext[p] = *reinterpret_cast<const g32_u32x4_t*>(xrow[p] + kx);
    };
    auto fetch_w = [&](const int slot, int kb) __attribute__((always_inline)) {
        const int k = kb * G32_KB + wc * 8;
#pragma unroll
        for (int q = 0; q < 4; ++q) ring[slot][q] = __builtin_nontemporal_load(reinterpret_cast<const g32_u32x4_t*>(wrow[q] + (k < K ? k : K - 8)));
    };
    auto stash = [&](int b) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < XP; ++p)
            if (xdst[p] >= 0) *reinterpret_cast<g32_u32x4_t*>(&xs[b][xdst[p]]) = xnext[p];
    };
    g32_f32x16_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    int cur = 0;
    // Block kb lives in ring slot (kb - kb_lo) % RING.  x of block kb + 1 was requested a step ago and goes to
    // the other buffer now; x of block kb + 2 is requested (the index is clamped: the last steps ask for the
    // last block again, which nobody reads).
    auto step = [&](const int slot, int kb, const bool request) __attribute__((always_inline)) {
        if (request) fetch_w((slot + RING - 1) % RING, kb + RING - 1);
        // the block's weights through the wavefront's piece of LDS (zeros past K: the last block only); LDS
        // serves a wavefront's instructions in order, so no barrier stands between put and get
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<g32_u32x4_t*>(wt_w + g32_at(q * 8 + wr, wc)) = g32_keep(ring[slot][q], kb * G32_KB + wc * 8 < K);
        g32_pack a[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) a[s].u = *reinterpret_cast<const g32_u32x4_t*>(wt_w + g32_at(r32, s * 2 + kh));
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            g32_pack b[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) b[t].u = *reinterpret_cast<const g32_u32x4_t*>(&xs[cur][g32_at(t * 32 + r32, s * 2 + kh)]);
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s].b, b[t].b, acc[t], 0, 0, 0);
        }
        stash(cur ^ 1);
        fetch_x(kb + 2);
        __syncthreads();
        cur ^= 1;
    };
    auto ending = [&](auto left_c, int kb0) __attribute__((always_inline)) {
        constexpr int LEFT = decltype(left_c)::value;
#pragma unroll
        for (int i = 0; i < LEFT + RING - 1; ++i) step(i % RING, kb0 + i, i < LEFT);
    };
    fetch_x(kb_lo);
#pragma unroll
    for (int b = 0; b < RING - 1; ++b) fetch_w(b, kb_lo + b < kb_hi ? kb_lo + b : kb_hi - 1);
    stash(0);
    fetch_x(kb_lo + 1);
    __syncthreads();
    int kb0 = kb_lo;
    for (; kb0 + 2 * RING - 1 <= kb_hi; kb0 += RING) {
#pragma unroll
        for (int b = 0; b < RING; ++b) step(b, kb0 + b, true);
    }
    const int left = kb_hi - kb0 - (RING - 1);       // < 0: fewer blocks than the ring requests up front
    if (left < 0) {
#pragma unroll
        for (int b = 0; b < RING - 1; ++b)
            if (kb0 + b < kb_hi) step(b, kb0 + b, false);
    } else {
        static_assert(RING >= 2 && RING <= 4, "one ending per residue");
        switch (left) {
            case 0: ending(std::integral_constant<int, 0>{}, kb0); break;
            case 1: ending(std::integral_constant<int, 1>{}, kb0); break;
            case 2: if (RING > 2) ending(std::integral_constant<int, 2>{}, kb0); break;
            default: if (RING > 3) ending(std::integral_constant<int, 3>{}, kb0); break;
        }
    }

    // ---- what the wavefront does with its sums: acc[t][v] is C[n = n0 + (v / 4) * 8 + kh * 4 + v % 4][m = t * 32 + r32]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 32 + r32;
        if (m >= M) continue;
        if (mode == G32_MODE_SWIGLU) {
            // rows 0-7 and 16-23 of the tile are gate rows, 8-15 and 24-31 the up rows of the same columns
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                if (n0 + g * 16 >= N) continue;
                const int col = (n0 / 16 + g) * 8 + kh * 4;
                float act[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float gate = acc[t][g * 8 + e], up = acc[t][g * 8 + 4 + e];
                    act[e] = up * (gate / (1.f + expf(-gate)));
                }
                zi_bf16* dst = (zi_bf16*)out + (int64_t)m * ldo + col;
                if (vec_out) {
                    uint2 pk;
                    pk.x = zi_pack_bf16x2(act[0], act[1]);
                    pk.y = zi_pack_bf16x2(act[2], act[3]);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) zi_store(dst + e, act[e]);
                }
            }
            continue;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nb = n0 + g * 8 + kh * 4;
            g32_f32x4_t s = g32_f32x4_t{acc[t][g * 4], acc[t][g * 4 + 1], acc[t][g * 4 + 2], acc[t][g * 4 + 3]};
            if (nb + 3 < N && vec_out) {
                if (mode == G32_MODE_PARTIAL) {
                    *reinterpret_cast<g32_f32x4_t*>((float*)out + ((int64_t)split * M + m) * N + nb) = s;
                } else {
                    if (bias) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) s[e] += zi_load(bias + nb + e);
                    }
                    if (out_f32) {
                        *reinterpret_cast<g32_f32x4_t*>((float*)out + (int64_t)m * ldo + nb) = s;
                    } else {
                        uint2 pk;
                        pk.x = zi_pack_bf16x2(s[0], s[1]);
                        pk.y = zi_pack_bf16x2(s[2], s[3]);
                        *reinterpret_cast<uint2*>((zi_bf16*)out + (int64_t)m * ldo + nb) = pk;
                    }
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = nb + e;
                if (n >= N) continue;
                if (mode == G32_MODE_PARTIAL) {
                    ((float*)out)[((int64_t)split * M + m) * N + n] = s[e];
                } else {
                    const float v = s[e] + (bias ? zi_load(bias + n) : 0.f);
                    if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = v;
                    else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, v);
                }
            }
        }
    }
}

// How the product with a weight matrix [N, K] is cut for this kernel: wavefronts a workgroup (32 weight rows
// each), splits of k over workgroups (at most 16) and blocks of 64 per split; a function of N and K and of
// whether there are more than 128 rows (`many_rows`: the sums of so many rows leave a wavefront registers
// enough only when a SIMD holds one wavefront, so the workgroups are of four).  As in zi_gemm_mid_plan what
// counts is the most work any compute unit gets when workgroups are dealt out in turn; `whole` forbids a split
// (the SwiGLU epilogue needs whole sums).
void zi_gemm_rows32_plan(int N, int K, int many_rows, int whole, int* splits, int* kb_per_split, int* waves) {
    const int tiles = (N + 31) / 32;
    const int kb_total = (K + G32_KB - 1) / G32_KB;
    const int cus = zi_compute_units();
    int64_t best_cost = -1;
    int best_s = 1, best_w = 4, best_per = kb_total;
    for (int w = 4; w <= (many_rows ? 4 : 8); w *= 2) {
        const int groups = (tiles + w - 1) / w;
        for (int s0 = 1; s0 <= (whole ? 1 : 16) && s0 <= (kb_total > 1 ? kb_total / 2 : 1); ++s0) {
            const int per = (kb_total + s0 - 1) / s0;
            const int s = (kb_total + per - 1) / per;
            if (s != s0) continue;
            const int64_t wgs = (int64_t)groups * s;
            const int64_t rounds = (wgs + cus - 1) / cus;
            const int64_t cost = rounds * ((int64_t)w * per + 16);
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && (s < best_s || (s == best_s && w > best_w)))) {
                best_cost = cost; best_s = s; best_w = w; best_per = per;
            }
        }
    }
    *splits = best_s;
    *kb_per_split = best_per;
    *waves = best_w;
}

// The launch; the checks are the caller's (zi_gemm_skinny).  M is 1 .. 256.
int zi_gemm_rows32_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                          int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream) {
    int splits, per, waves;
    zi_gemm_rows32_plan(N, K, M > 128, mode == G32_MODE_SWIGLU, &splits, &per, &waves);
    const int tiles = (N + 31) / 32;
    const dim3 grid((tiles + waves - 1) / waves, splits);
    const int mt = (M + 31) / 32;
    // Workgroups of four wavefronts (a wavefront a SIMD, all 512 registers its own) keep four blocks of weights
    // in flight; of eight, as many as the 256 registers beside the sums allow.
#define ZI_G32W(MT, WV, RG)                                                                                            \
    gemm_rows32_kernel<MT, WV, RG><<<grid, WV * ZI_WAVE, 0, stream>>>(out, mode, out_f32, x, w, bias, M, N, K, ldx, ldw, \
                                                                     ldo, per, vec_out)
#define ZI_G32(MT, RG8)                         \
    if (waves == 4) ZI_G32W(MT, 4, 4);          \
    else ZI_G32W(MT, 8, RG8)
    switch (mt) {
        case 1: ZI_G32(1, 4); break;
        case 2: ZI_G32(2, 4); break;
        case 3: ZI_G32(3, 3); break;
        case 4: ZI_G32(4, 3); break;
        case 5: ZI_G32W(5, 4, 4); break;
        case 6: ZI_G32W(6, 4, 4); break;
        case 7: ZI_G32W(7, 4, 4); break;
        default: ZI_G32W(8, 4, 4); break;
    }
#undef ZI_G32
#undef ZI_G32W
    return zi_check_launch("gemm_rows32");
}
