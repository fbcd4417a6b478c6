// out[M,N] = x[M,K] . w[N,K]^T (+ bias) for 1..128 rows of x: the decode-time products, bound by the one
// pass over the weights (the entry points are in gemm_skinny.hip).
//
// A workgroup of four to eight wavefronts owns 16 weight rows a wavefront and a range of k.  It walks its
// k-blocks of 128: the block's slice of x (up to 64 rows x 128 values) is staged in LDS once for the four
// wavefronts, each wavefront reads its own 16 weight rows from memory as whole cache lines, turns them
// into matrix-core operands through a piece of LDS of its own (v_mfma_f32_16x16x32_bf16, float32
// accumulation) and keeps the sums of its 16 x M outputs in registers, so nothing is added across
// wavefronts.  The next two blocks' weights and x travel while the current one is worked on (a ring of
// three register buffers; loads are issued without branches so that they stay in flight).  The k dimension is cut over gridDim.y workgroups when N alone gives too few of them; those
// leave float32 partial sums [split][M][N] that the consumer adds in rising order.  The cut depends on N
// and K only.  Epilogues as in the few-rows kernel: plain (bias), partial sums, SwiGLU over gate/up rows
// interleaved in blocks of 8.
#include "zi_common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 gm_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float gm_f32x4_t;
// 16 bytes as a native vector: copies of the struct uint4 are memcpys to the compiler, and an array of
// them that is only copied stays in memory instead of registers
typedef __attribute__((ext_vector_type(4))) unsigned gm_u32x4_t;

#define GM_MIN_WAVES 4      // wavefronts of a workgroup: 4 .. 8, 16 weight rows each
#define GM_MAX_WAVES 8
#define GM_KB 128
#define GM_XS GM_KB         // LDS row stride, in elements: rows of 16 pieces of 16 bytes, piece c of row r at place c xor (r mod 16)

#define GM_MODE_PLAIN 0
#define GM_MODE_PARTIAL 1
#define GM_MODE_SWIGLU 2

union gm_pack {
    gm_u32x4_t u;
    gm_bf16x8_t b;
};

// v where `keep` holds, else zeros, by arithmetic: after a select the compiler may move the load that
// made v under a branch, and wait for it there.
__device__ __forceinline__ gm_u32x4_t gm_keep(gm_u32x4_t v, bool keep) {
    const unsigned mask = 0u - (unsigned)keep;
    return v & mask;
}

// What a wavefront does with its sums: C[n = n0 + j*4 + e][m = t*16 + r] in acc[t][e].
template <int MT>
__device__ __forceinline__ void gm_epilogue(const gm_f32x4_t (&acc)[MT], void* __restrict__ out, int mode, int out_f32,
                                            const zi_bf16* __restrict__ bias, int M, int N, int64_t ldo, int split,
                                            int n0, int r, int j, int vec_out) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        gm_f32x4_t s = acc[t];
        const int m = t * 16 + r;
        if (mode == GM_MODE_SWIGLU) {
            // lanes j = 0,1 hold gate rows j*4 + e, lanes j = 2,3 the up rows of the same columns
            gm_f32x4_t up;
            up[0] = __shfl_xor(s[0], 32, ZI_WAVE); up[1] = __shfl_xor(s[1], 32, ZI_WAVE);
            up[2] = __shfl_xor(s[2], 32, ZI_WAVE); up[3] = __shfl_xor(s[3], 32, ZI_WAVE);
            if (j >= 2 || m >= M || n0 >= N) continue;
            const int col = (n0 / 16) * 8 + j * 4;     // N / 2 columns of output; N % 16 == 0
            float act[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) act[e] = up[e] * (s[e] / (1.f + expf(-s[e])));
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
            continue;
        }
        if (m >= M) continue;
        const int nb = n0 + j * 4;
        if (nb + 3 < N && vec_out) {
            if (mode == GM_MODE_PARTIAL) {
                *reinterpret_cast<gm_f32x4_t*>((float*)out + ((int64_t)split * M + m) * N + nb) = s;
            } else {
                if (bias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) s[e] += zi_load(bias + nb + e);
                }
                if (out_f32) {
                    *reinterpret_cast<gm_f32x4_t*>((float*)out + (int64_t)m * ldo + nb) = s;
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
            if (mode == GM_MODE_PARTIAL) {
                ((float*)out)[((int64_t)split * M + m) * N + n] = s[e];
            } else {
                const float v = s[e] + (bias ? zi_load(bias + n) : 0.f);
                if (out_f32) ((float*)out)[(int64_t)m * ldo + n] = v;
                else zi_store((zi_bf16*)out + (int64_t)m * ldo + n, v);
            }
        }
    }
}

template <int MT, int GM_RING, int GM_WAVES>
__global__ void __launch_bounds__(GM_WAVES* ZI_WAVE)
gemm_mid_kernel(void* __restrict__ out, int mode, int out_f32, const zi_bf16* __restrict__ x,
                const zi_bf16* __restrict__ w, const zi_bf16* __restrict__ bias, int M, int N, int K, int64_t ldx,
                int64_t ldw, int64_t ldo, int kb_per_split, int vec_out) {
    __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 16 * GM_XS];
    __shared__ __attribute__((aligned(16))) uint16_t wt[GM_WAVES][16 * GM_XS];   // a wavefront's weight tile
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int split = blockIdx.y;
    const int kb_total = (K + GM_KB - 1) / GM_KB;
    const int kb_lo = split * kb_per_split;
    const int kb_hi = (kb_lo + kb_per_split < kb_total) ? kb_lo + kb_per_split : kb_total;
    const int n0 = (blockIdx.x * GM_WAVES + wave) * 16;
    // Weights are read as whole cache lines: a load instruction takes 4 rows x 256 bytes (lane l: row
    // l / 16 of the four, 16-byte piece l % 16), four instructions a tile of 16 rows x 128 values.
    // Loads in the matrix-core operand layout (16 rows x 64 bytes an instruction) were measured a fifth
    // slower.  The tile is turned into that layout through a piece of LDS that the wavefront owns.
    const int wq = lane & 15;
    const zi_bf16* wrow[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int n = n0 + c * 4 + j;
        wrow[c] = w + (int64_t)(n < N ? n : N - 1) * ldw;
    }
    // LDS rows are not padded but swizzled (16-byte reads in operand order then run at the full LDS rate)
    uint16_t* const wt_w = &wt[wave][0];

    // what this thread stages of a block's x slice: XP pieces of 16 bytes (rows srow[p], piece spc).  The slice's
    // MT * 256 pieces are dealt out over all the workgroup's threads, a row of 16 pieces to 16 neighbours; the
    // last round may pass the slice's end (its loads repeat the last row and go nowhere).
    constexpr int THREADS = GM_WAVES * ZI_WAVE, XP = (MT * 256 + THREADS - 1) / THREADS;
    const int spc = tid % 16;
    int srow[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) srow[p] = p * (THREADS / 16) + tid / 16;
    // the weights of GM_RING k-blocks are in flight at once (a ring of register buffers); the x slice of
    // the next block is fetched while this one is worked on
    gm_u32x4_t ring[GM_RING][4], xring[GM_RING][XP];
    // Loads are issued without branches and their results are not touched before the products need
    // them: only then does the compiler let several blocks' loads stay in flight.  Addresses are
    // clamped into the matrices.  Rows of x past M repeat the last row and give outputs that nobody
    // stores; columns past K would count the last eight twice, so the weights are zeroed there, when
    // they are used.  A block's x is requested before its weights: loads return in order, and x, which
    // comes from the cache and is wanted a step earlier, must not queue behind weights from memory.
    const zi_bf16* xrow[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) xrow[p] = x + (int64_t)(srow[p] < M ? srow[p] : M - 1) * ldx;
    auto fetch = [&](const int slot, int kb) __attribute__((always_inline)) {
        const int k0 = kb * GM_KB;
        const int kx = k0 + spc * 8 < K ? k0 + spc * 8 : K - 8;
#pragma unroll
        for (int p = 0; p < XP; ++p) xring[slot][p] = *reinterpret_cast<const gm_u32x4_t*>(xrow[p] + kx);
        const int k = k0 + wq * 8;
        // a weight is read once a step and the weights of a step are many times the caches: non-temporal loads keep
        // them out of L2 (decode at batch 8, 1.5B sizes: 5,403 to 5,518 tok/s)
#pragma unroll
        for (int c = 0; c < 4; ++c) ring[slot][c] = __builtin_nontemporal_load(reinterpret_cast<const gm_u32x4_t*>(wrow[c] + (k < K ? k : K - 8)));
    };
    auto stash = [&](const int slot, int b) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < XP; ++p)
            if ((p + 1) * (THREADS / 16) <= MT * 16 || srow[p] < MT * 16)
                *reinterpret_cast<gm_u32x4_t*>(&xs[b][srow[p] * GM_XS + (spc ^ (srow[p] & 15)) * 8]) = xring[slot][p];
    };
    gm_f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Blocks kb_lo .. kb_lo + GM_RING - 2 are requested up front; block kb's x goes to LDS one step
    // before it is used, GM_RING - 2 steps after it was requested.  Block kb lives in ring slot
    // (kb - kb_lo) % GM_RING.  The compiler counts how many loads may stay in flight at each use only
    // in straight-line code; behind a branch that may or may not have issued loads it waits for all of
    // them.  So the walk is cut into pieces without such branches: a steady loop of GM_RING steps that
    // all request a block, and one of GM_RING straight-line endings, chosen by how many blocks are
    // left to request.
    int cur = 0;
    auto step = [&](const int slot, int kb, const bool request) __attribute__((always_inline)) {
        if (request) fetch((slot + GM_RING - 1) % GM_RING, kb + GM_RING - 1);
        // all of the block's x operands are read from LDS before the first product: the reads' latency
        // is paid once, not once per product
        // the weight tile goes through the wavefront's LDS piece (zeros past K: the last block only);
        // LDS serves a wavefront's instructions in order, so no barrier stands between put and get
#pragma unroll
        for (int c = 0; c < 4; ++c)
            *reinterpret_cast<gm_u32x4_t*>(wt_w + (c * 4 + j) * GM_XS + (wq ^ (c * 4 + j)) * 8) =
                gm_keep(ring[slot][c], kb * GM_KB + wq * 8 < K);
        gm_pack bb[4][MT], a[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                bb[c][t].u = *reinterpret_cast<const gm_u32x4_t*>(&xs[cur][(t * 16 + r) * GM_XS + ((c * 4 + j) ^ r) * 8]);
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c].u = *reinterpret_cast<const gm_u32x4_t*>(wt_w + r * GM_XS + ((c * 4 + j) ^ r) * 8);
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[c].b, bb[c][t].b, acc[t], 0, 0, 0);
        stash((slot + 1) % GM_RING, cur ^ 1);    // after the last block: something nobody reads
        __syncthreads();
        cur ^= 1;
    };
    // the ending for `left` blocks still to request: left + GM_RING - 1 blocks to work on
    auto ending = [&](auto left_c, int kb0) __attribute__((always_inline)) {
        constexpr int LEFT = decltype(left_c)::value;
#pragma unroll
        for (int i = 0; i < LEFT + GM_RING - 1; ++i) step(i % GM_RING, kb0 + i, i < LEFT);
    };
#pragma unroll
    for (int b = 0; b < GM_RING - 1; ++b) fetch(b, kb_lo + b < kb_hi ? kb_lo + b : kb_hi - 1);
    stash(0, 0);
    __syncthreads();
    int kb0 = kb_lo;
    for (; kb0 + 2 * GM_RING - 1 <= kb_hi; kb0 += GM_RING) {
#pragma unroll
        for (int b = 0; b < GM_RING; ++b) step(b, kb0 + b, true);
    }
    const int left = kb_hi - kb0 - (GM_RING - 1);    // < 0: fewer blocks than the ring requests up front
    if (left < 0) {
#pragma unroll
        for (int b = 0; b < GM_RING - 1; ++b)
            if (kb0 + b < kb_hi) step(b, kb0 + b, false);
    } else {
        static_assert(GM_RING >= 2 && GM_RING <= 4, "one ending per residue");
        switch (left) {
            case 0: ending(std::integral_constant<int, 0>{}, kb0); break;
            case 1: ending(std::integral_constant<int, 1>{}, kb0); break;
            case 2: if (GM_RING > 2) ending(std::integral_constant<int, 2>{}, kb0); break;
            default: if (GM_RING > 3) ending(std::integral_constant<int, 3>{}, kb0); break;
        }
    }
    gm_epilogue<MT>(acc, out, mode, out_f32, bias, M, N, ldo, split, n0, r, j, vec_out);
}

// The same product for 65 .. 128 rows of x (MT = 5 .. 8 tiles of 16 rows): one pass over the weights where two
// launches of the kernel above would make two, and where the library's products of so few rows stay far from the
// weights' stream.  The registers that the kernel above spends on rings of x and on all of a block's x operands
// do not stretch to eight tiles, so here a block's x is requested one step ahead only (it comes from the cache;
// the weights keep their ring of three), it lies in LDS once (two barriers a block instead of one; a second
// buffer for it, 96 KB of LDS in all, was measured and changed nothing), and the x operands
// are read a k-step at a time, just before their matrix instructions.  The cut, the order of the sums and the
// epilogues are the kernel's above: a row's result does not depend on which of the two kernels makes it.
template <int MT, int GM_WAVES>
__global__ void __launch_bounds__(GM_WAVES* ZI_WAVE)
gemm_wide_kernel(void* __restrict__ out, int mode, int out_f32, const zi_bf16* __restrict__ x,
                 const zi_bf16* __restrict__ w, const zi_bf16* __restrict__ bias, int M, int N, int K, int64_t ldx,
                 int64_t ldw, int64_t ldo, int kb_per_split, int vec_out) {
    constexpr int RING = 3;
    __shared__ __attribute__((aligned(16))) uint16_t xs[MT * 16 * GM_XS];
    __shared__ __attribute__((aligned(16))) uint16_t wt[GM_WAVES][16 * GM_XS];
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int split = blockIdx.y;
    const int kb_total = (K + GM_KB - 1) / GM_KB;
    const int kb_lo = split * kb_per_split;
    const int kb_hi = (kb_lo + kb_per_split < kb_total) ? kb_lo + kb_per_split : kb_total;
    const int n0 = (blockIdx.x * GM_WAVES + wave) * 16;
    const int wq = lane & 15;
    const zi_bf16* wrow[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int n = n0 + c * 4 + j;
        wrow[c] = w + (int64_t)(n < N ? n : N - 1) * ldw;
    }
    uint16_t* const wt_w = &wt[wave][0];
    // the block's x slice is dealt out over all the workgroup's threads (see the kernel above)
    constexpr int THREADS = GM_WAVES * ZI_WAVE, XP = (MT * 256 + THREADS - 1) / THREADS;
    const int spc = tid % 16;
    int srow[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) srow[p] = p * (THREADS / 16) + tid / 16;
    gm_u32x4_t ring[RING][4], xnext[XP];
    const zi_bf16* xrow[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) xrow[p] = x + (int64_t)(srow[p] < M ? srow[p] : M - 1) * ldx;
    // a block's x is requested before the weights that are requested in the same step: loads return in order,
    // and x is wanted first.  The block index is clamped: the last step asks for its own block again.
    auto fetch_x = [&](int kb) __attribute__((always_inline)) {
        const int k0 = (kb < kb_hi ? kb : kb_hi - 1) * GM_KB;
        const int kx = k0 + spc * 8 < K ? k0 + spc * 8 : K - 8;
#pragma unroll
        for (int p = 0; p < XP; ++p) xnext[p] = *reinterpret_cast<const gm_u32x4_t*>(xrow[p] + kx);
    };
    auto fetch_w = [&](const int slot, int kb) __attribute__((always_inline)) {
        const int k = kb * GM_KB + wq * 8;
#pragma unroll
        for (int c = 0; c < 4; ++c) ring[slot][c] = __builtin_nontemporal_load(reinterpret_cast<const gm_u32x4_t*>(wrow[c] + (k < K ? k : K - 8)));
    };
    auto stash = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < XP; ++p)
            if ((p + 1) * (THREADS / 16) <= MT * 16 || srow[p] < MT * 16)
                *reinterpret_cast<gm_u32x4_t*>(&xs[srow[p] * GM_XS + (spc ^ (srow[p] & 15)) * 8]) = xnext[p];
    };
    gm_f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};

    auto step = [&](const int slot, int kb, const bool request) __attribute__((always_inline)) {
        fetch_x(kb + 1);
        if (request) fetch_w((slot + RING - 1) % RING, kb + RING - 1);
#pragma unroll
        for (int c = 0; c < 4; ++c)
            *reinterpret_cast<gm_u32x4_t*>(wt_w + (c * 4 + j) * GM_XS + (wq ^ (c * 4 + j)) * 8) =
                gm_keep(ring[slot][c], kb * GM_KB + wq * 8 < K);
        gm_pack a[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c].u = *reinterpret_cast<const gm_u32x4_t*>(wt_w + r * GM_XS + ((c * 4 + j) ^ r) * 8);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            gm_pack bb[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t)
                bb[t].u = *reinterpret_cast<const gm_u32x4_t*>(&xs[(t * 16 + r) * GM_XS + ((c * 4 + j) ^ r) * 8]);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[c].b, bb[t].b, acc[t], 0, 0, 0);
        }
        __syncthreads();        // every wavefront has read this block's x
        stash();                // the next block's (after the last block: something nobody reads)
        __syncthreads();
    };
    auto ending = [&](auto left_c, int kb0) __attribute__((always_inline)) {
        constexpr int LEFT = decltype(left_c)::value;
#pragma unroll
        for (int i = 0; i < LEFT + RING - 1; ++i) step(i % RING, kb0 + i, i < LEFT);
    };
    fetch_x(kb_lo);
#pragma unroll
    for (int b = 0; b < RING - 1; ++b) fetch_w(b, kb_lo + b < kb_hi ? kb_lo + b : kb_hi - 1);
    stash();
    __syncthreads();
    int kb0 = kb_lo;
    for (; kb0 + 2 * RING - 1 <= kb_hi; kb0 += RING) {
#pragma unroll
        for (int b = 0; b < RING; ++b) step(b, kb0 + b, true);
    }
    const int left = kb_hi - kb0 - (RING - 1);
    if (left < 0) {
#pragma unroll
        for (int b = 0; b < RING - 1; ++b)
            if (kb0 + b < kb_hi) step(b, kb0 + b, false);
    } else {
        switch (left) {
            case 0: ending(std::integral_constant<int, 0>{}, kb0); break;
            case 1: ending(std::integral_constant<int, 1>{}, kb0); break;
            default: ending(std::integral_constant<int, 2>{}, kb0); break;
        }
    }
    gm_epilogue<MT>(acc, out, mode, out_f32, bias, M, N, ldo, split, n0, r, j, vec_out);
}

// How the product with a weight matrix [N, K] is cut: wavefronts a workgroup (16 weight rows each), splits
// of k over workgroups (at most 16: what the consumers add at once) and k-blocks per split.  A function of
// N and K alone.
//
// A compute unit works through the wavefronts it is given at a fixed rate (measured: 280 workgroups of
// four wavefronts on 256 compute units take almost twice as long as 140, because 24 units hold two), so
// what counts is the most work any unit gets when workgroups are dealt out in turn: rounds = ceil(workgroups
// / units), each of `waves * k-blocks` wavefront-blocks plus a start-up worth about ten of them.  Among
// the cuts the cheapest by that measure is taken, then the one with the fewest splits, then the fewest
// wavefronts.  A matrix with many times more rows than that keeps the units busy whatever the cut (its
// workgroups follow each other, two to a unit): four wavefronts, no split (measured on the 151,936 rows of
// the output head: 108 against 119 us with eight).
void zi_gemm_mid_plan(int N, int K, int* splits, int* kb_per_split, int* waves) {
    const int tiles = (N + 15) / 16;
    const int kb_total = (K + GM_KB - 1) / GM_KB;
    int64_t best_cost = -1;
    int best_s = 1, best_w = GM_MIN_WAVES, best_per = kb_total;
    const int cus = zi_compute_units();          // the cut is balanced over the device's compute units
    const bool many = (tiles + GM_MIN_WAVES - 1) / GM_MIN_WAVES > 4 * cus;
    for (int w = GM_MIN_WAVES; w <= (many ? GM_MIN_WAVES : GM_MAX_WAVES); ++w) {
        const int groups = (tiles + w - 1) / w;
        for (int s0 = 1; s0 <= (many ? 1 : 16) && s0 <= (kb_total > 1 ? kb_total / 2 : 1); ++s0) {
            const int per = (kb_total + s0 - 1) / s0;
            const int s = (kb_total + per - 1) / per;
            if (s != s0) continue;      // the same cut under another name
            const int64_t wgs = (int64_t)groups * s;
            const int64_t rounds = (wgs + cus - 1) / cus;
            const int64_t cost = rounds * ((int64_t)w * per + 10);
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && s < best_s)) {
                best_cost = cost; best_s = s; best_w = w; best_per = per;
            }
        }
    }
    *splits = best_s;
    *kb_per_split = best_per;
    *waves = best_w;
}

// The launch; the checks are the caller's (zi_gemm_skinny).
int zi_gemm_mid_launch(void* out, int out_f32, int mode, const zi_bf16* x, const zi_bf16* w, const zi_bf16* bias, int M,
                       int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int vec_out, hipStream_t stream) {
    int splits, per, waves;
    zi_gemm_mid_plan(N, K, &splits, &per, &waves);
    const int tiles = (N + 15) / 16;
    const dim3 grid((tiles + waves - 1) / waves, splits);
    const int mt = (M + 15) / 16;
#define ZI_GM2(MT, WV)                                                                                            \
    gemm_mid_kernel<MT, 3, WV><<<grid, WV * ZI_WAVE, 0, stream>>>(out, mode, out_f32, x, w, bias, M, N, K, ldx, ldw, \
                                                                  ldo, per, vec_out)
#define ZI_GM(MT)                               \
    switch (waves) {                            \
        case 4: ZI_GM2(MT, 4); break;           \
        case 5: ZI_GM2(MT, 5); break;           \
        case 6: ZI_GM2(MT, 6); break;           \
        case 7: ZI_GM2(MT, 7); break;           \
        default: ZI_GM2(MT, 8); break;          \
    }
#define ZI_GW2(MT, WV)                                                                                         \
    gemm_wide_kernel<MT, WV><<<grid, WV * ZI_WAVE, 0, stream>>>(out, mode, out_f32, x, w, bias, M, N, K, ldx, ldw, ldo, \
                                                               per, vec_out)
#define ZI_GW(MT)                               \
    switch (waves) {                            \
        case 4: ZI_GW2(MT, 4); break;           \
        case 5: ZI_GW2(MT, 5); break;           \
        case 6: ZI_GW2(MT, 6); break;           \
        case 7: ZI_GW2(MT, 7); break;           \
        default: ZI_GW2(MT, 8); break;          \
    }
    switch (mt) {
        case 1: ZI_GM(1); break;
        case 2: ZI_GM(2); break;
        case 3: ZI_GM(3); break;
        case 4: ZI_GM(4); break;
        case 5: ZI_GW(5); break;
        case 6: ZI_GW(6); break;
        case 7: ZI_GW(7); break;
        default: ZI_GW(8); break;
    }
#undef ZI_GM
#undef ZI_GM2
#undef ZI_GW
#undef ZI_GW2
    return zi_check_launch("gemm_mid");
}
