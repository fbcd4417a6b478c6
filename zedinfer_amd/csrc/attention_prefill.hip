// Paged causal grouped-query attention for prompt portions on the matrix cores.
//
// A workgroup of eight wavefronts owns a tile of 64 consecutive query tokens of one
// entry and one query head: four sub-tiles of 16 queries, each shared by two
// wavefronts that take alternate runs of 64 keys and merge their results at the end
// (the longest chain of dependent work, a late tile's walk over all earlier keys, is
// halved that way).  The tile's keys are walked in blocks of 128, aligned to absolute
// multiples of 128, so a query's blocks do not depend on how its prompt was cut into steps.  Each block of keys and values is
// staged once in LDS for the four wavefronts (two buffers: the next block travels
// from the cache into registers while the matrix cores work on this one); scores and the P.V product run on
// v_mfma_f32_16x16x32_bf16 with float32 accumulation, the running softmax
// (maximum, sum, rescaling) is float32, and s_j = (q . k_j) * scale is scaled after
// the dot product (reference formulas:
// src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:106-162).
//
// A tile that sees more than 2,048 keys is cut along the keys, at absolute multiples of 2,048, over several
// workgroups (gridDim.y), so that a portion of a long prompt, which has few tiles but a long walk each,
// still fills the chip; those workgroups leave (maximum, sum, unnormalised output) per query and a second
// kernel merges them in rising order of the keys.  The cut depends on the query's position alone.
//
// Operand layout.  Scores are computed transposed: the A operand is a 16-key tile of
// K, the B operand the 16 queries, so a lane ends up with the scores of ONE query
// (lane % 16) and four keys per tile.  Keys are placed in LDS rows in a permuted
// order (row t*16 + j*4 + e holds key (t/2)*32 + j*8 + (t%2)*4 + e of the block), which
// makes the eight probabilities a lane holds after two tiles exactly the eight
// consecutive keys j*8..j*8+7 that the B operand of the P.V product wants from that
// lane: no data moves between lanes.  Values are cached transposed ([dim][slot]),
// so the A operand of P.V (16 dims x 32 keys) is read as 16-byte runs of keys.
// LDS rows are padded by 16 bytes, which spreads a quarter-wave's 16-byte reads over
// all banks.
//
// bfloat16; head_dim a multiple of 16 up to 128 (a head_dim that is no multiple of 32 is
// padded with zeros for the score product); page size a power of two from 8.
// Other shapes are the plain kernel's.
#include "zi_common.h"
#include "zi_api.h"
#include "zi_paging.h"

typedef __attribute__((ext_vector_type(8))) __bf16 pf_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float pf_f32x4_t;

#define PF_KH 2                  // wavefronts that share a query sub-tile, each with its own 64 keys of a block
#define PF_WAVES (4 * PF_KH)
#define PF_BM ZI_PF_BM           // queries per workgroup
#define PF_BN 64                 // keys per wavefront and block
#define PF_BS (PF_BN * PF_KH)    // keys per block
#define PF_CHUNK ZI_PF_CHUNK     // keys one workgroup walks at most: a tile with more is cut over several
#define PF_MAXC ZI_PF_MAXC       // most such cuts of one tile
static_assert(PF_BS == ZI_PF_BS, "the block of keys is the one the shared cut is made for");

union pf_pack {
    uint4 u;
    pf_bf16x8_t b;
    uint16_t h[8];
};

// v where bit 0 of `keep` is set, else zeros (by value: a select between two register arrays' elements
// would be made through memory)
__device__ __forceinline__ uint4 pf_keep(uint4 v, int keep) {
    const unsigned mask = 0u - (unsigned)(keep & 1);
    return make_uint4(v.x & mask, v.y & mask, v.z & mask, v.w & mask);
}

template <int D>
__global__ void __launch_bounds__(PF_WAVES* ZI_WAVE)
attention_prefill_kernel(zi_bf16* __restrict__ out, int64_t ldo, const zi_bf16* __restrict__ q, int64_t ldq,
                         const zi_bf16* __restrict__ kcache, const zi_bf16* __restrict__ vcache,
                         const int32_t* __restrict__ tile_entry, const int32_t* __restrict__ tile_off,
                         const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                         const int32_t* __restrict__ entry_past, const int32_t* __restrict__ block_tables,
                         int max_pages, int num_pages, int nh, int nkv, int ps_shift, int window, float scale,
                         float* __restrict__ part_o, float* __restrict__ part_ml, int max_chunks, int chunk_keys) {
    static_assert(D % 16 == 0 && D >= 16 && D <= 128, "head_dim must be a multiple of 16 up to 128");
    constexpr int DK = (D + 31) / 32;   // k-steps of the score product
    constexpr int DP = DK * 32;         // head_dim padded to a multiple of 32
    constexpr int KS = DP + 8;          // LDS row stride of the key tile, in elements
    constexpr int VS = PF_BS + 8;       // LDS row stride of the transposed value tile
    constexpr int DT = D / 16;          // output tiles of 16 dims
    constexpr int CPR = DP / 8;         // 16-byte chunks per (padded) key row
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[2 * PF_BS * KS];   // two buffers each
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[2 * D * VS];

    // tiles come heaviest first; all heads of a tile are dispatched before the next tile
    const int tile = blockIdx.x / nh, h = blockIdx.x % nh;
    const int g = h / (nh / nkv);
    const int e = tile_entry[tile], off = tile_off[tile];
    const int start = entry_start[e], len = entry_len[e], past = entry_past[e];
    const int count = (len - off < PF_BM) ? len - off : PF_BM;
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int32_t* bt = block_tables + (int64_t)e * max_pages;
    const int pos0 = past + off;            // position of the tile's first query
    // this workgroup's cut of the tile's keys: [kb_begin, khi], between absolute multiples of PF_CHUNK
    const PfCut cut = zi_pf_cut(pos0, count, window, blockIdx.y, chunk_keys);
    if (!cut.live) return;
    const int kmax = cut.kmax;              // last key any query of the tile sees
    const int nc = cut.nc, kb_begin = cut.kb_begin, khi = cut.khi;

    // this wavefront's queries (sub-tile qs) and its share of every block's keys (kh)
    const int qs = wave % 4, kh = wave / 4;
    const int row = qs * 16 + r;
    const bool wave_active = qs * 16 < count;
    const bool qvalid = row < count;
    const int qrow = qvalid ? row : count - 1;
    const int qpos = pos0 + qrow;
    const int wave_first = pos0 + ((qs * 16 < count) ? qs * 16 : count - 1);
    const int wave_last = pos0 + ((qs * 16 + 15 < count) ? qs * 16 + 15 : count - 1);
    const float scale_log2 = scale * 1.4426950408889634f;
    const int wave_lo = (window > 0 && pos0 + qs * 16 - window + 1 > 0) ? pos0 + qs * 16 - window + 1 : 0;
    pf_bf16x8_t qop[DK];
    {
        const zi_bf16* qr = q + (int64_t)(start + off + qrow) * ldq + (int64_t)h * D + j * 8;
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            pf_pack p;
            p.u = (dk * 32 + j * 8 < D) ? *reinterpret_cast<const uint4*>(qr + dk * 32) : make_uint4(0, 0, 0, 0);
            qop[dk] = p.b;
        }
    }
    pf_f32x4_t o[DT];
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) o[dd] = pf_f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, lsum = 0.f;

    const int ps = 1 << ps_shift;
    const int vpart = ps < PF_BS ? ps : PF_BS;   // keys of one page inside a block
    const int gpp = vpart / 8;                   // 8-key groups of that part (a power of two)
    const int gshift = __ffs(gpp) - 1;
    constexpr int THREADS = PF_WAVES * ZI_WAVE;
    constexpr int KPASS = (PF_BS * CPR + THREADS - 1) / THREADS;      // 16-byte pieces of K a thread stages
    constexpr int VPASS = (D * (PF_BS / 8) + THREADS - 1) / THREADS;  // and of V
    uint4 kreg[KPASS], vreg[VPASS];
    // What a thread stages does not change from block to block: key row and 16-byte piece of K, and
    // (dim, column) of V.  Page sizes are powers of two here: no division in the loop.
    int k_kk[KPASS], k_c[KPASS], k_dst[KPASS], v_dim[VPASS], v_col[VPASS];
#pragma unroll
    for (int pass = 0; pass < KPASS; ++pass) {
        const int idx = pass * THREADS + tid;
        const int kk = idx / CPR, c = idx % CPR;
        const int k64 = kk % PF_BN;   // the 64 keys of one wavefront are permuted among themselves
        k_kk[pass] = idx < PF_BS * CPR ? kk : -1;
        k_c[pass] = c;
        k_dst[pass] = ((kk / PF_BN) * PF_BN + (2 * (k64 / 32) + ((k64 % 8) / 4)) * 16 + ((k64 % 32) / 8) * 4 + k64 % 4) * KS +
                      c * 8;
    }
#pragma unroll
    for (int pass = 0; pass < VPASS; ++pass) {
        const int idx = pass * THREADS + tid;
        const int part = (idx / D) >> gshift, rem = idx - part * (D << gshift);
        v_dim[pass] = idx < D * (PF_BS / 8) ? rem >> gshift : -1;
        v_col[pass] = part * vpart + (rem & (gpp - 1)) * 8;
    }
    const int ps_mask = ps - 1;

    // global -> registers: the block of keys [kb, kb + 128).  Straight-line code: every table lookup
    // is issued, then every load of keys and values, from addresses clamped into the sequence and the
    // pool; what a thread must not use is zeroed when it goes to LDS.  With a branch around a load the
    // compiler waits for it on the spot, and the block would not travel during the products.
    int kvalid = 0, vvalid = 0;
    const int kmax8 = kmax & ~7, pi_last = max_pages - 1;
    auto fetch = [&](int kb) {
        int kpage[KPASS], vpage[VPASS], kkey[KPASS], vkey[VPASS];
        kvalid = 0;
        vvalid = 0;
#pragma unroll
        for (int pass = 0; pass < KPASS; ++pass) {
            const int key = kb + (k_kk[pass] >= 0 ? k_kk[pass] : 0);
            const bool ok = k_kk[pass] >= 0 && key <= kmax && (D % 32 == 0 || k_c[pass] * 8 < D);
            kkey[pass] = key <= kmax ? key : kmax;
            const int pi = kkey[pass] >> ps_shift;
            kpage[pass] = bt[pi < pi_last ? pi : pi_last];
            kvalid |= (int)ok << pass;
        }
#pragma unroll
        for (int pass = 0; pass < VPASS; ++pass) {
            const int key0 = kb + v_col[pass];
            const bool ok = v_dim[pass] >= 0 && key0 <= kmax;
            vkey[pass] = key0 <= kmax ? key0 : kmax8;
            const int pi = vkey[pass] >> ps_shift;
            vpage[pass] = bt[pi < pi_last ? pi : pi_last];
            vvalid |= (int)ok << pass;
        }
#pragma unroll
        for (int pass = 0; pass < KPASS; ++pass) {
            const bool held = (unsigned)kpage[pass] < (unsigned)num_pages;   // a window may have freed the page
            const int page = held ? kpage[pass] : 0;
            const int c = (D % 32 == 0 || k_c[pass] * 8 < D) ? k_c[pass] : 0;
            kreg[pass] = *reinterpret_cast<const uint4*>(
                kcache + ((((int64_t)page * nkv + g) << ps_shift) + (kkey[pass] & ps_mask)) * D + c * 8);
            if (!held) kvalid &= ~(1 << pass);
        }
#pragma unroll
        for (int pass = 0; pass < VPASS; ++pass) {
            const bool held = (unsigned)vpage[pass] < (unsigned)num_pages;
            const int page = held ? vpage[pass] : 0;
            const int dim = v_dim[pass] >= 0 ? v_dim[pass] : 0;
            vreg[pass] = *reinterpret_cast<const uint4*>(
                vcache + ((((int64_t)page * nkv + g) * D + dim) << ps_shift) + (vkey[pass] & ps_mask));
            if (!held) vvalid &= ~(1 << pass);
        }
    };
    // registers -> LDS buffer `b`: key kb + kk goes to row rho(kk) of the key tile; values go in
    // transposed, row dim, column key - kb
    auto stash = [&](int kb, int b) {
        uint16_t* kl = k_lds + b * (PF_BS * KS);
        uint16_t* vl = v_lds + b * (D * VS);
#pragma unroll
        for (int pass = 0; pass < KPASS; ++pass)
            if (k_kk[pass] >= 0) *reinterpret_cast<uint4*>(&kl[k_dst[pass]]) = pf_keep(kreg[pass], kvalid >> pass);
        if (kb + PF_BS - 1 <= kmax) {     // all blocks but the last: no key past the end
#pragma unroll
            for (int pass = 0; pass < VPASS; ++pass)
                if (v_dim[pass] >= 0)
                    *reinterpret_cast<uint4*>(&vl[v_dim[pass] * VS + v_col[pass]]) = pf_keep(vreg[pass], vvalid >> pass);
        } else {
#pragma unroll
            for (int pass = 0; pass < VPASS; ++pass) {
                if (v_dim[pass] < 0) continue;
                const int key0 = kb + v_col[pass];
                pf_pack val;
                val.u = pf_keep(vreg[pass], vvalid >> pass);
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    if (key0 + x > kmax) val.h[x] = 0;    // slots past the last key may hold anything
                *reinterpret_cast<uint4*>(&vl[v_dim[pass] * VS + v_col[pass]]) = val.u;
            }
        }
    };

    fetch(kb_begin);
    stash(kb_begin, 0);
    __syncthreads();
    // one block of keys from LDS buffer `cur` into this wavefront's running softmax and output
    auto work = [&](int kb0, int cur) {
        const int kb = kb0 + kh * PF_BN;      // this wavefront's 64 keys of the block
        const uint16_t* kl = k_lds + cur * (PF_BS * KS) + kh * (PF_BN * KS);
        const uint16_t* vl = v_lds + cur * (D * VS) + kh * PF_BN;
        if (wave_active && kb <= wave_last && kb + PF_BN > wave_lo) {
        // ---- scores of 64 keys for this lane's query
        pf_f32x4_t s[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            s[t] = pf_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dk = 0; dk < DK; ++dk) {
                pf_pack a;
                a.u = *reinterpret_cast<const uint4*>(&kl[(t * 16 + r) * KS + dk * 32 + j * 8]);
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, qop[dk], s[t], 0, 0, 0);
            }
        }
        // softmax in base 2: t = s * scale * log2(e), p = 2^(t - m).  A block that every query of the
        // wavefront sees whole (all but those on the diagonal and at a window's edge) needs no mask.
        const bool whole = kb + PF_BN - 1 <= wave_first && (window <= 0 || kb > wave_last - window);
        float mx = -INFINITY;
        if (whole) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int x = 0; x < 4; ++x) mx = fmaxf(mx, s[t][x]);
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int key = kb + (t / 2) * 32 + j * 8 + (t % 2) * 4 + x;
                    const bool vis = key <= qpos && (window <= 0 || key > qpos - window);
                    const float v = vis ? s[t][x] : -INFINITY;
                    s[t][x] = v;
                    mx = fmaxf(mx, v);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
        // the scale is positive (the host checks): the largest scaled score is the largest score, scaled; the
        // scaling of every score is then one fused multiply-add with the subtraction of the maximum
        const float m_new = fmaxf(m, mx * scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_use);      // 2^(-inf) = 0 before the first key
        m = m_new;
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                s[t][x] = __builtin_amdgcn_exp2f(fmaf(s[t][x], scale_log2, -m_use));    // 0 for masked keys
                psum += s[t][x];
            }
        pf_pack pb[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            pb[b].u.x = zi_pack_bf16x2(s[2 * b][0], s[2 * b][1]);
            pb[b].u.y = zi_pack_bf16x2(s[2 * b][2], s[2 * b][3]);
            pb[b].u.z = zi_pack_bf16x2(s[2 * b + 1][0], s[2 * b + 1][1]);
            pb[b].u.w = zi_pack_bf16x2(s[2 * b + 1][2], s[2 * b + 1][3]);
        }
        lsum = lsum * corr + psum;
        if (__any(corr != 1.f)) {     // the running maximum seldom moves after the first blocks
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) {
                o[dd][0] *= corr; o[dd][1] *= corr; o[dd][2] *= corr; o[dd][3] *= corr;
            }
        }
        // ---- o^T += V^T . P^T
#pragma unroll
        for (int dd = 0; dd < DT; ++dd)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                pf_pack a;
                a.u = *reinterpret_cast<const uint4*>(&vl[(dd * 16 + r) * VS + b * 32 + j * 8]);
                o[dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, pb[b].b, o[dd], 0, 0, 0);
            }
        }
    };
    // The next block travels from the cache into registers while this one is worked on; it goes into
    // the other LDS buffer, which everyone has finished reading at the barrier before.  The last block
    // stands outside the loop, so that no branch surrounds the loop's loads.
    int cur = 0, kb0 = kb_begin;
    for (; kb0 + PF_BS <= khi; kb0 += PF_BS, cur ^= 1) {
        fetch(kb0 + PF_BS);
        work(kb0, cur);
        stash(kb0 + PF_BS, cur ^ 1);
        __syncthreads();
    }
    work(kb0, cur);
    __syncthreads();
    float l = lsum;
    l += __shfl_xor(l, 16, ZI_WAVE);
    l += __shfl_xor(l, 32, ZI_WAVE);
    if (PF_KH > 1) {
        // the wavefronts of a query sub-tile merge their (maximum, sum, output) through LDS, in the order
        // of the wavefronts; nobody reads the key tiles any more
        float* mo = reinterpret_cast<float*>(k_lds);                 // [kh-1][qs][DT][64][4]
        float* ml = mo + (PF_KH - 1) * 4 * DT * ZI_WAVE * 4;         // [kh-1][qs][64][2]
        if (kh > 0) {
            float* dst = mo + ((kh - 1) * 4 + qs) * (DT * ZI_WAVE * 4);
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) *reinterpret_cast<pf_f32x4_t*>(dst + (dd * ZI_WAVE + lane) * 4) = o[dd];
            ml[(((kh - 1) * 4 + qs) * ZI_WAVE + lane) * 2] = m;
            ml[(((kh - 1) * 4 + qs) * ZI_WAVE + lane) * 2 + 1] = l;
        }
        __syncthreads();
        if (kh > 0) return;
#pragma unroll
        for (int k2 = 1; k2 < PF_KH; ++k2) {
            const float* src = mo + ((k2 - 1) * 4 + qs) * (DT * ZI_WAVE * 4);
            const float m2 = ml[(((k2 - 1) * 4 + qs) * ZI_WAVE + lane) * 2];
            const float l2 = ml[(((k2 - 1) * 4 + qs) * ZI_WAVE + lane) * 2 + 1];
            const float mm = fmaxf(m, m2);
            const float mu = (mm == -INFINITY) ? 0.f : mm;
            const float a1 = __builtin_amdgcn_exp2f(m - mu), a2 = __builtin_amdgcn_exp2f(m2 - mu);
            l = l * a1 + l2 * a2;
            m = mm;
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) {
                const pf_f32x4_t v = *reinterpret_cast<const pf_f32x4_t*>(src + (dd * ZI_WAVE + lane) * 4);
                o[dd][0] = o[dd][0] * a1 + v[0] * a2; o[dd][1] = o[dd][1] * a1 + v[1] * a2;
                o[dd][2] = o[dd][2] * a1 + v[2] * a2; o[dd][3] = o[dd][3] * a1 + v[3] * a2;
            }
        }
    }
    if (!qvalid) return;
    if (nc > 1) {
        // one of several cuts of this tile's keys: leave (maximum, sum, unnormalised output) for the merge.
        // A launch sized for fewer cuts than the tile has must not write outside the workspace: the
        // query's output is made NaN instead, so that it shows.
        if (nc > max_chunks) {
            if (blockIdx.y == 0)
                for (int dd = 0; dd < DT; ++dd)
                    for (int x = 0; x < 4; ++x) zi_store(out + (int64_t)(start + off + row) * ldo + (int64_t)h * D + dd * 16 + j * 4 + x, NAN);
            return;
        }
        const int64_t slot = zi_pf_part_slot(start + off + row, nh, h, max_chunks, blockIdx.y);
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) *reinterpret_cast<pf_f32x4_t*>(part_o + slot * D + dd * 16 + j * 4) = o[dd];
        if (j == 0) {
            part_ml[slot * 2] = m;
            part_ml[slot * 2 + 1] = l;
        }
        return;
    }
    const float inv = 1.f / l;
    zi_bf16* orow = out + (int64_t)(start + off + row) * ldo + (int64_t)h * D;
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) {
        uint2 w;
        w.x = zi_pack_bf16x2(o[dd][0] * inv, o[dd][1] * inv);
        w.y = zi_pack_bf16x2(o[dd][2] * inv, o[dd][3] * inv);
        *reinterpret_cast<uint2*>(orow + dd * 16 + j * 4) = w;
    }
}

// ---------------------------------------------------------------------------------------------------
// The same attention for head sizes 64 and 128 with keys and values loaded straight into LDS
// (global_load_lds_dwordx4): no registers, no address arithmetic and no LDS stores are spent on staging.
// One load instruction of a wavefront fills 1 KB of LDS, lane l the 16 bytes at l * 16; which 16 bytes of
// the cache a lane asks for is free, so the tiles keep the order the matrix cores want (keys permuted as
// above, values transposed) and their rows are not padded but swizzled: the 16-byte piece c of row r sits
// at place c xor (r mod pieces-per-row) (rows of 128 bytes: c xor (r / 2 mod 8), two rows share the 64
// banks), which spreads a quarter-wave's reads over the banks without a conflict: 16-byte reads in this
// order run at the rate of consecutive ones, those of rows padded by 16 bytes or rotated by the row number
// an eighth slower.  Two buffers, each a pair of LDS arrays of its own, used in turn by an unrolled loop: the loads
// of the next block are issued right after the barrier that makes this block visible, so the compiler's
// wait before a barrier (it waits for every load into LDS there) never waits for a block that is still
// needed later.  Values of keys past the last key and of pages that a window has given back are loaded
// from 16 zero bytes instead (0 * NaN would be NaN); the one piece that straddles the last key is
// cleaned in LDS.  Keys need no such care: their scores are masked.
__device__ __attribute__((aligned(16))) const unsigned pf_zero16[4] = {0u, 0u, 0u, 0u};

// QW: sub-tiles of 16 queries a wavefront owns: 1 (tiles of 64 queries) or 2 (tiles of 128: every block of keys and
// values that is brought into LDS, and every operand read from there, serves twice the queries).
// KH: wavefronts that share a query group, each with its own 64 keys of a block: 2 (eight wavefronts, blocks of
// 128 keys, one workgroup on a compute unit) or 1 (four wavefronts, blocks of 64 keys, half the LDS: two
// workgroups on a compute unit, which are not in step with each other, so that one's matrix instructions run
// beside the other's softmax and loads; a tile's walk is one wavefront's per query group, so it takes longer:
// for launches with many tiles).
template <int D, int QW, int KH>
__global__ void __launch_bounds__(4 * KH * ZI_WAVE, KH == 1 ? 2 : 1)
attention_prefill_dma_kernel(zi_bf16* __restrict__ out, int64_t ldo, const zi_bf16* __restrict__ q, int64_t ldq,
                             const zi_bf16* __restrict__ kcache, const zi_bf16* __restrict__ vcache,
                             const int32_t* __restrict__ tile_entry, const int32_t* __restrict__ tile_off,
                             const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                             const int32_t* __restrict__ entry_past, const int32_t* __restrict__ block_tables,
                             int max_pages, int num_pages, int nh, int nkv, int ps_shift, int window, float scale,
                             float* __restrict__ part_o, float* __restrict__ part_ml, int max_chunks, int chunk_keys) {
    static_assert(D == 64 || D == 128, "this variant takes head sizes 64 and 128");
    static_assert(QW == 1 || QW == 2, "16 or 32 queries a wavefront");
    constexpr int BM = PF_BM * QW;                   // queries of a tile
    constexpr int QR = 16 * QW;                      // queries of a wavefront
    constexpr int DK = D / 32, DT = D / 16;
    constexpr int KC = D / 8;                        // 16-byte pieces of a key row
    static_assert(KH == 1 || KH == 2, "one or two wavefronts a query group");
    constexpr int WAVES = 4 * KH;
    constexpr int BS = PF_BN * KH;                   // keys of a block
    constexpr int VC = BS / 8;                       // and of a row of the transposed value tile: 8 or 16
    constexpr int VSW = 16 / VC;                     // value rows that share 256 bytes of LDS (and one swizzle)
    constexpr int KCH = BS * KC, VCH = D * VC;       // pieces of the two tiles
    constexpr int THREADS = WAVES * ZI_WAVE;
    constexpr int KI = KCH / THREADS, VI = VCH / THREADS;   // load instructions a wavefront issues per tile
    constexpr int KSW = 16 / KC;                     // key rows that share 256 bytes of LDS (and one swizzle)
    __shared__ __attribute__((aligned(16))) uint4 k_ab[2 * KCH];
    __shared__ __attribute__((aligned(16))) uint4 v_ab[2 * VCH];
    uint4* const k_a = k_ab;
    uint4* const k_b = k_ab + KCH;
    uint4* const v_a = v_ab;
    uint4* const v_b = v_ab + VCH;
    __shared__ int32_t bt_lds[ZI_PF_CHUNK_LONG / 8 + 8];     // the pages of this workgroup's keys (page size >= 8)

    const int tile = blockIdx.x / nh, h = blockIdx.x % nh;
    const int g = h / (nh / nkv);
    const int e = tile_entry[tile], off = tile_off[tile];
    const int start = entry_start[e], len = entry_len[e], past = entry_past[e];
    const int count = (len - off < BM) ? len - off : BM;
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int32_t* bt = block_tables + (int64_t)e * max_pages;
    const int pos0 = past + off;
    const PfCut cut = zi_pf_cut(pos0, count, window, blockIdx.y, chunk_keys);
    if (!cut.live) return;
    const int kmax = cut.kmax, nc = cut.nc, kb_begin = cut.kb_begin, khi = cut.khi;

    // wavefront (qs, kh): queries qs * QR .. + QR - 1 of the tile (sub-tile u: 16 of them), half kh of every block
    const int qs = wave % 4, kh = wave / 4;
    int row[QW], qpos[QW];
    bool qvalid[QW];
#pragma unroll
    for (int u = 0; u < QW; ++u) {
        row[u] = qs * QR + u * 16 + r;
        qvalid[u] = row[u] < count;
        qpos[u] = pos0 + (qvalid[u] ? row[u] : count - 1);
    }
    const bool wave_active = qs * QR < count;
    const int wave_first = pos0 + ((qs * QR < count) ? qs * QR : count - 1);
    const int wave_last = pos0 + ((qs * QR + QR - 1 < count) ? qs * QR + QR - 1 : count - 1);
    const float scale_log2 = scale * 1.4426950408889634f;
    const int wave_lo = (window > 0 && pos0 + qs * QR - window + 1 > 0) ? pos0 + qs * QR - window + 1 : 0;
    pf_bf16x8_t qop[QW][DK];
#pragma unroll
    for (int u = 0; u < QW; ++u) {
        const zi_bf16* qr = q + (int64_t)(start + off + (qvalid[u] ? row[u] : count - 1)) * ldq + (int64_t)h * D + j * 8;
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            pf_pack p;
            p.u = *reinterpret_cast<const uint4*>(qr + dk * 32);
            qop[u][dk] = p.b;
        }
    }
    pf_f32x4_t o[QW][DT];
    float m[QW], lsum[QW];
#pragma unroll
    for (int u = 0; u < QW; ++u) {
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) o[u][dd] = pf_f32x4_t{0.f, 0.f, 0.f, 0.f};
        m[u] = -INFINITY;
        lsum[u] = 0.f;
    }

    // the block table's entries for keys [kb_begin, khi], once
    const int ps = 1 << ps_shift, ps_mask = ps - 1;
    const int pi_last = max_pages - 1, pi_first = kb_begin >> ps_shift;
    for (int i = tid; i <= (khi >> ps_shift) - pi_first; i += blockDim.x)
        bt_lds[i] = bt[pi_first + i < pi_last ? pi_first + i : pi_last];
    // What a lane loads does not change from block to block: for its KI pieces of the key tile the key
    // (as an offset into the block) and the piece of its row, for its VI pieces of the value tile the
    // dim and the eight keys.  Place L of a tile is row L / pieces-per-row; the piece there is swizzled.
    int k_key[KI], k_piece[KI], v_dim[VI], v_key[VI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int L = (wave * KI + i) * ZI_WAVE + lane;
        const int rho = L / KC;
        const int t = (rho % PF_BN) / 16, rr = rho % 16;
        k_key[i] = (rho / PF_BN) * PF_BN + (t / 2) * 32 + (rr / 4) * 8 + (t % 2) * 4 + rr % 4;
        k_piece[i] = (L % KC) ^ ((rho / KSW) & (KC - 1));
    }
#pragma unroll
    for (int i = 0; i < VI; ++i) {
        const int L = (wave * VI + i) * ZI_WAVE + lane;
        v_dim[i] = L / VC;
        v_key[i] = ((L % VC) ^ ((v_dim[i] / VSW) & (VC - 1))) * 8;
    }
    const zi_bf16* kbase = kcache + (int64_t)g * ps * D;
    const zi_bf16* vbase = vcache + (int64_t)g * D * ps;
    const int64_t page_stride = (int64_t)nkv * ps * D;
    const int khi8 = khi & ~7;
    __syncthreads();      // the table is in LDS

    auto issue = [&](int kb, uint4* kl, uint4* vl) {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const int key = kb + k_key[i];
            const int kc = key <= khi ? key : khi;
            const int pg = bt_lds[(kc >> ps_shift) - pi_first];
            const int page = (unsigned)pg < (unsigned)num_pages ? pg : 0;     // not held: a window has passed it
            const zi_bf16* src = kbase + page * page_stride + (int64_t)(kc & ps_mask) * D + k_piece[i] * 8;
            __builtin_amdgcn_global_load_lds(src, kl + (wave * KI + i) * ZI_WAVE, 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < VI; ++i) {
            const int key0 = kb + v_key[i];
            const int kc = key0 <= khi ? key0 : khi8;
            const int pg = bt_lds[(kc >> ps_shift) - pi_first];
            const bool ok = key0 <= kmax && (unsigned)pg < (unsigned)num_pages;
            const zi_bf16* src = ok ? vbase + pg * page_stride + ((int64_t)v_dim[i] << ps_shift) + (kc & ps_mask)
                                    : reinterpret_cast<const zi_bf16*>(pf_zero16);
            __builtin_amdgcn_global_load_lds(src, vl + (wave * VI + i) * ZI_WAVE, 16, 0, 0);
        }
    };
    // The piece of every value row that holds the last key and keys past it: what lies past is cleared
    // (those slots of the page may hold anything).  Only in the block that holds the last key.
    auto clean = [&](int kb, uint4* vl) {
        if (kb + BS - 1 > kmax && ((kmax + 1) & 7) != 0) {
            if (tid < D) {
                const int piece = (kmax - kb) / 8, keep = (kmax + 1) & 7;
                pf_pack val;
                uint4* at = vl + tid * VC + (piece ^ ((tid / VSW) & (VC - 1)));
                val.u = *at;
#pragma unroll
                for (int x = 0; x < 8; ++x)
                    if (x >= keep) val.h[x] = 0;
                *at = val.u;
            }
            __syncthreads();
        }
    };
    auto work = [&](int kb0, const uint4* kl, const uint4* vl) {
        const int kb = kb0 + kh * PF_BN;      // this wavefront's 64 keys of the block
        if (wave_active && kb <= wave_last && kb + PF_BN > wave_lo) {
        pf_f32x4_t s[QW][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int u = 0; u < QW; ++u) s[u][t] = pf_f32x4_t{0.f, 0.f, 0.f, 0.f};
            const int rho = kh * PF_BN + t * 16 + r;
#pragma unroll
            for (int dk = 0; dk < DK; ++dk) {
                pf_pack a;
                a.u = kl[rho * KC + ((dk * 4 + j) ^ ((rho / KSW) & (KC - 1)))];
#pragma unroll
                for (int u = 0; u < QW; ++u)      // one read of the keys' operand serves every sub-tile
                    s[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, qop[u][dk], s[u][t], 0, 0, 0);
            }
        }
        const bool whole = kb + PF_BN - 1 <= wave_first && (window <= 0 || kb > wave_last - window);
        pf_pack pb[QW][2];
#pragma unroll
        for (int u = 0; u < QW; ++u) {
            float mx = -INFINITY;
            if (whole) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int x = 0; x < 4; ++x) mx = fmaxf(mx, s[u][t][x]);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const int key = kb + (t / 2) * 32 + j * 8 + (t % 2) * 4 + x;
                        const bool vis = key <= qpos[u] && (window <= 0 || key > qpos[u] - window);
                        const float v = vis ? s[u][t][x] : -INFINITY;
                        s[u][t][x] = v;
                        mx = fmaxf(mx, v);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
            const float m_new = fmaxf(m[u], mx * scale_log2);      // the scale is positive
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float corr = __builtin_amdgcn_exp2f(m[u] - m_use);
            m[u] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    s[u][t][x] = __builtin_amdgcn_exp2f(fmaf(s[u][t][x], scale_log2, -m_use));
                    psum += s[u][t][x];
                }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                pb[u][b].u.x = zi_pack_bf16x2(s[u][2 * b][0], s[u][2 * b][1]);
                pb[u][b].u.y = zi_pack_bf16x2(s[u][2 * b][2], s[u][2 * b][3]);
                pb[u][b].u.z = zi_pack_bf16x2(s[u][2 * b + 1][0], s[u][2 * b + 1][1]);
                pb[u][b].u.w = zi_pack_bf16x2(s[u][2 * b + 1][2], s[u][2 * b + 1][3]);
            }
            lsum[u] = lsum[u] * corr + psum;
            if (__any(corr != 1.f)) {
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) {
                    o[u][dd][0] *= corr; o[u][dd][1] *= corr; o[u][dd][2] *= corr; o[u][dd][3] *= corr;
                }
            }
        }
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) {
            const int dim = dd * 16 + r;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                pf_pack a;
                a.u = vl[dim * VC + ((kh * 8 + b * 4 + j) ^ ((dim / VSW) & (VC - 1)))];
#pragma unroll
                for (int u = 0; u < QW; ++u)      // and one read of the values' operand
                    o[u][dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, pb[u][b].b, o[u][dd], 0, 0, 0);
            }
        }
        }
    };
    // Two blocks a turn, buffer a then b.  At each barrier the block about to be worked on has arrived
    // (the compiler waits for all loads into LDS before a barrier) and everyone has finished with the
    // other buffer, so the block after it is requested into that one at once.
    issue(kb_begin, k_a, v_a);
    int kb0 = kb_begin;
    while (true) {
        __syncthreads();
        if (kb0 + BS <= khi) issue(kb0 + BS, k_b, v_b);
        clean(kb0, v_a);
        work(kb0, k_a, v_a);
        if (kb0 + BS > khi) break;
        kb0 += BS;
        __syncthreads();
        if (kb0 + BS <= khi) issue(kb0 + BS, k_a, v_a);
        clean(kb0, v_b);
        work(kb0, k_b, v_b);
        if (kb0 + BS > khi) break;
        kb0 += BS;
    }
    __syncthreads();
    float l[QW];
#pragma unroll
    for (int u = 0; u < QW; ++u) {
        l[u] = lsum[u];
        l[u] += __shfl_xor(l[u], 16, ZI_WAVE);
        l[u] += __shfl_xor(l[u], 32, ZI_WAVE);
    }
    if constexpr (KH > 1) {
        // the two wavefronts of a query group merge their (maximum, sum, output) through LDS; nobody reads
        // the tiles any more
        float* mo = reinterpret_cast<float*>(k_ab);                  // [qs][QW][DT][64][4]: within the two key tiles
        float* ml = reinterpret_cast<float*>(v_ab);                  // [qs][QW][64][2]
        static_assert(sizeof(float) * 4 * QW * DT * ZI_WAVE * 4 <= sizeof(uint4) * 2 * KCH, "the key tiles hold the merge");
        if (kh > 0) {
#pragma unroll
            for (int u = 0; u < QW; ++u) {
                float* dst = mo + (qs * QW + u) * (DT * ZI_WAVE * 4);
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) *reinterpret_cast<pf_f32x4_t*>(dst + (dd * ZI_WAVE + lane) * 4) = o[u][dd];
                ml[((qs * QW + u) * ZI_WAVE + lane) * 2] = m[u];
                ml[((qs * QW + u) * ZI_WAVE + lane) * 2 + 1] = l[u];
            }
        }
        __syncthreads();
        if (kh > 0) return;
#pragma unroll
        for (int u = 0; u < QW; ++u) {
            const float* src = mo + (qs * QW + u) * (DT * ZI_WAVE * 4);
            const float m2 = ml[((qs * QW + u) * ZI_WAVE + lane) * 2];
            const float l2 = ml[((qs * QW + u) * ZI_WAVE + lane) * 2 + 1];
            const float mm = fmaxf(m[u], m2);
            const float mu = (mm == -INFINITY) ? 0.f : mm;
            const float a1 = __builtin_amdgcn_exp2f(m[u] - mu), a2 = __builtin_amdgcn_exp2f(m2 - mu);
            l[u] = l[u] * a1 + l2 * a2;
            m[u] = mm;
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) {
                const pf_f32x4_t v = *reinterpret_cast<const pf_f32x4_t*>(src + (dd * ZI_WAVE + lane) * 4);
                o[u][dd][0] = o[u][dd][0] * a1 + v[0] * a2; o[u][dd][1] = o[u][dd][1] * a1 + v[1] * a2;
                o[u][dd][2] = o[u][dd][2] * a1 + v[2] * a2; o[u][dd][3] = o[u][dd][3] * a1 + v[3] * a2;
            }
        }
    }
#pragma unroll
    for (int u = 0; u < QW; ++u) {
        if (!qvalid[u]) continue;
        if (nc > 1) {
            // one of several cuts of this tile's keys: leave (maximum, sum, unnormalised output) for the merge
            if (nc > max_chunks) {
                if (blockIdx.y == 0)
                    for (int dd = 0; dd < DT; ++dd)
                        for (int x = 0; x < 4; ++x)
                            zi_store(out + (int64_t)(start + off + row[u]) * ldo + (int64_t)h * D + dd * 16 + j * 4 + x, NAN);
                continue;
            }
            const int64_t slot = zi_pf_part_slot(start + off + row[u], nh, h, max_chunks, blockIdx.y);
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) *reinterpret_cast<pf_f32x4_t*>(part_o + slot * D + dd * 16 + j * 4) = o[u][dd];
            if (j == 0) {
                part_ml[slot * 2] = m[u];
                part_ml[slot * 2 + 1] = l[u];
            }
            continue;
        }
        const float inv = 1.f / l[u];
        zi_bf16* orow = out + (int64_t)(start + off + row[u]) * ldo + (int64_t)h * D;
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) {
            uint2 w;
            w.x = zi_pack_bf16x2(o[u][dd][0] * inv, o[u][dd][1] * inv);
            w.y = zi_pack_bf16x2(o[u][dd][2] * inv, o[u][dd][3] * inv);
            *reinterpret_cast<uint2*>(orow + dd * 16 + j * 4) = w;
        }
    }
}

// Merge the cuts of one (query, head): out = sum_c 2^(m_c - M) o_c / sum_c 2^(m_c - M) l_c, in rising order
// of the keys.  One wavefront per (query row of a tile, head); tiles with one cut were written directly.
__global__ void __launch_bounds__(ZI_WAVE)
attention_prefill_merge_kernel(zi_bf16* __restrict__ out, int64_t ldo, const float* __restrict__ part_o,
                               const float* __restrict__ part_ml, const int32_t* __restrict__ tile_entry,
                               const int32_t* __restrict__ tile_off, const int32_t* __restrict__ entry_start,
                               const int32_t* __restrict__ entry_len, const int32_t* __restrict__ entry_past, int nh,
                               int D, int window, int max_chunks, int bm, int chunk_keys) {
    const int tile = blockIdx.x / bm, qi = blockIdx.x % bm, h = blockIdx.y, lane = threadIdx.x;
    const int e = tile_entry[tile], off = tile_off[tile];
    const int start = entry_start[e], len = entry_len[e], past = entry_past[e];
    const int count = (len - off < bm) ? len - off : bm;
    if (qi >= count) return;
    const int nc = zi_pf_cut(past + off, count, window, 0, chunk_keys).nc;
    if (nc == 1 || nc > max_chunks) return;
    const int64_t row = start + off + qi;
    const int64_t slot0 = zi_pf_part_slot(row, nh, h, max_chunks, 0);
    // cut c's (m, l) sit in lane c; a cut none of whose keys this query sees left m = -inf, l = 0
    const float mc = lane < nc ? part_ml[(slot0 + lane) * 2] : -INFINITY;
    const float lc = lane < nc ? part_ml[(slot0 + lane) * 2 + 1] : 0.f;
    const float M = zi_wave_max(mc);
    const float wc = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - M);
    float L = 0.f, acc[2] = {0.f, 0.f};
    for (int c = 0; c < nc; ++c) {
        const float w = __shfl(wc, c, ZI_WAVE);
        L += w * __shfl(lc, c, ZI_WAVE);
#pragma unroll
        for (int v = 0; v < 2; ++v)
            if (lane + v * ZI_WAVE < D) acc[v] += w * part_o[(slot0 + c) * D + lane + v * ZI_WAVE];
    }
    const float inv = 1.f / L;
#pragma unroll
    for (int v = 0; v < 2; ++v)
        if (lane + v * ZI_WAVE < D) zi_store(out + row * ldo + (int64_t)h * D + lane + v * ZI_WAVE, acc[v] * inv);
}

// Floats of workspace a launch over `rows` query rows needs when tiles are cut into up to `max_chunks`.
extern "C" int64_t zi_attention_prefill_workspace(int rows, int nh, int d, int max_chunks) {
    return zi_pf_workspace_floats(rows, nh, d, max_chunks);
}

// Cuts the launch must cover when no query sees more than `keys` keys (position + 1; with a window: the
// window plus one tile and one block, at most).
extern "C" int zi_attention_prefill_chunks(int keys) {
    if (keys < 1) keys = 1;
    return (keys + PF_CHUNK - 1) / PF_CHUNK;
}

// 1 when the shape is this kernel's, else 0.
extern "C" int zi_attention_prefill_supported(int dt, int nh, int nkv, int d, int page_size) {
    if (dt != ZI_BF16 || nkv <= 0 || nh <= 0 || nh % nkv) return 0;
    if (d < 16 || d > 128 || d % 16) return 0;
    return page_size >= 8 && (page_size & (page_size - 1)) == 0;
}

// Which kernel head sizes 64 and 128 take: 1 (the default) loads keys and values straight into LDS, 0 stages
// them through registers like the other head sizes.  For measurements and tests.
static int pf_variant = 1;
extern "C" int zi_attention_prefill_variant(int variant) {
    const int before = pf_variant;
    if (variant == 0 || variant == 1) pf_variant = variant;
    return before;
}

// Queries of a tile: 64, or 128 where the kernel that loads straight into LDS serves (head sizes 64 and 128):
// there a block of keys and values in LDS, and an operand read from it, serves twice the queries.  The caller
// cuts its entries into tiles of this many queries (zi_attention_prefill takes either size for those shapes).
extern "C" int zi_attention_prefill_tile(int dt, int d) {
    return (dt == ZI_BF16 && pf_variant >= 1 && (d == 64 || d == 128)) ? 2 * PF_BM : PF_BM;
}

// Keys one workgroup walks at most: tiles are cut at absolute multiples of this (the shorter of the two cuts).
extern "C" int zi_attention_prefill_chunk_keys() { return PF_CHUNK; }

// The cut for a launch of `groups` tiles x heads none of whose queries sees more than `max_keys` keys (with a
// window: the window plus a tile and a block): the caller sizes max_chunks and the workspace with it and hands
// it to zi_attention_prefill.  Measured at the 1.5B sizes (12 heads), one prompt in one step, cut every 2,048
// against no cut: 16,384 tokens (1,536 groups) 83.7 against 78.0 ms, 8,192 (768) 33.3 against 32.3, 4,096 (384)
// 16.6 against 17.6; at the 32B sizes 16,384 tokens 1,036 against 985 ms.
extern "C" int zi_attention_prefill_chunk_keys_for(int max_keys, int groups) { return zi_pf_chunk_for(max_keys, groups, zi_compute_units()); }

// The smallest tile of queries (every head size takes it).
extern "C" int zi_attention_prefill_tile_min() { return PF_BM; }

// How a launch of `groups` tiles x heads is cut when no query sees more than `max_keys` keys (position + 1) and
// a query sees `window` keys at most (0: all): the keys between cuts go to *chunk_keys, the cuts a tile can
// have are returned; both go to zi_attention_prefill, and the cuts size its workspace.  A windowed tile's keys
// span at most the window, the widest tile and a block, from anywhere in a cut.
extern "C" int zi_attention_prefill_cuts(int max_keys, int window, int groups, int* chunk_keys) {
    if (max_keys < 1) max_keys = 1;
    if (window > 0 && max_keys > window + 2 * PF_BM + PF_BS) max_keys = window + 2 * PF_BM + PF_BS;
    const int chunk = zi_pf_chunk_for(max_keys, groups, zi_compute_units());
    if (window > 0) max_keys += chunk - 1;
    if (chunk_keys) *chunk_keys = chunk;
    return (max_keys + chunk - 1) / chunk;
}

// Tile i covers the queries [tile_off[i], tile_off[i] + tile) of entry tile_entry[i] (fewer at the
// entry's end; `tile` is 64, or 128 for head sizes 64 and 128); entry e brings entry_len[e] tokens that start at row entry_start[e] of q and at
// position entry_past[e] of its sequence, whose block table is row e of block_tables.  `alone` (head sizes 64 and
// 128): workgroups of four wavefronts that walk blocks of 64 keys, two to a compute unit, for launches of many
// tiles; a query's keys are then added in another order, so the result differs by rounding.
extern "C" int zi_attention_prefill(void* out, const void* q, int dt, int num_tiles, int64_t ldq, int64_t ldo,
                                    const void* kcache, const void* vcache, const int32_t* tile_entry,
                                    const int32_t* tile_off, const int32_t* entry_start, const int32_t* entry_len,
                                    const int32_t* entry_past, const int32_t* block_tables, int max_pages,
                                    int num_pages, int nh, int nkv, int d, int page_size, int window, float scale,
                                    int rows, int max_chunks, float* workspace, int64_t workspace_floats, int tile,
                                    int alone, int chunk_keys, hipStream_t stream) {
    ZI_REQUIRE(tile == PF_BM || (tile == 2 * PF_BM && pf_variant >= 1 && (d == 64 || d == 128)),
               "attention_prefill: tiles of %d queries (64, or 128 for head sizes 64 and 128)", tile);
    ZI_REQUIRE(zi_attention_prefill_supported(dt, nh, nkv, d, page_size),
               "attention_prefill: unsupported shape (bfloat16, head_dim a multiple of 16 up to 128, page size a power "
               "of two from 8): dtype %d heads %d kv_heads %d head_dim %d page %d", dt, nh, nkv, d, page_size);
    ZI_REQUIRE(num_tiles >= 0 && max_pages > 0 && num_pages > 0 && window >= 0 && rows >= 0, "attention_prefill: bad sizes");
    ZI_REQUIRE(ldq >= (int64_t)nh * d && ldo >= (int64_t)nh * d && ldq % 8 == 0 && ldo % 4 == 0,
               "attention_prefill: bad row stride");
    ZI_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 && ((uintptr_t)kcache % 16) == 0 &&
                   ((uintptr_t)vcache % 16) == 0,
               "attention_prefill: q, out and the caches must be aligned to 16 bytes");
    ZI_REQUIRE(nh <= 65535, "attention_prefill: too many heads (%d)", nh);
    ZI_REQUIRE(scale > 0.f, "attention_prefill: the scale must be positive, got %g", (double)scale);
    ZI_REQUIRE(chunk_keys == PF_CHUNK || chunk_keys == ZI_PF_CHUNK_LONG, "attention_prefill: tiles are cut every %d or %d keys, not %d",
               PF_CHUNK, ZI_PF_CHUNK_LONG, chunk_keys);
    ZI_REQUIRE(max_chunks >= 1 && max_chunks <= PF_MAXC, "attention_prefill: max_chunks %d outside 1..%d (contexts up to %d keys)",
               max_chunks, PF_MAXC, PF_MAXC * chunk_keys);
    ZI_REQUIRE(max_chunks == 1 || (workspace && ((uintptr_t)workspace % 16) == 0 &&
                                   workspace_floats >= zi_attention_prefill_workspace(rows, nh, d, max_chunks)),
               "attention_prefill: workspace of %lld floats is too small or not aligned", (long long)workspace_floats);
    if (num_tiles == 0) return 0;
    ZI_REQUIRE((int64_t)num_tiles * nh < (1ll << 31) && (int64_t)num_tiles * tile < (1ll << 31), "attention_prefill: too many tiles");
    const dim3 grid(num_tiles * nh, max_chunks);
    int ps_shift = 0;
    while ((1 << ps_shift) < page_size) ++ps_shift;
    float* po = workspace;
    float* pml = workspace ? workspace + (int64_t)rows * nh * max_chunks * d : nullptr;
#define ZI_PF(DD)                                                                                              \
    attention_prefill_kernel<DD><<<grid, PF_WAVES * ZI_WAVE, 0, stream>>>(                                     \
        (zi_bf16*)out, ldo, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache, tile_entry, \
        tile_off, entry_start, entry_len, entry_past, block_tables, max_pages, num_pages, nh, nkv, ps_shift,   \
        window, scale, po, pml, max_chunks, chunk_keys)
#define ZI_PF_DMA(DD, QW, KH)                                                                                  \
    attention_prefill_dma_kernel<DD, QW, KH><<<grid, 4 * KH * ZI_WAVE, 0, stream>>>(                           \
        (zi_bf16*)out, ldo, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache, tile_entry, \
        tile_off, entry_start, entry_len, entry_past, block_tables, max_pages, num_pages, nh, nkv, ps_shift,   \
        window, scale, po, pml, max_chunks, chunk_keys)
    const bool dma = pf_variant >= 1 && (d == 64 || d == 128);
    const bool wide = tile == 2 * PF_BM;
    ZI_REQUIRE(!alone || dma, "attention_prefill: workgroups of four wavefronts are for head sizes 64 and 128");
    if (dma && d == 128 && wide && alone) ZI_PF_DMA(128, 2, 1);
    else if (dma && d == 128 && wide) ZI_PF_DMA(128, 2, 2);
    else if (dma && d == 128 && alone) ZI_PF_DMA(128, 1, 1);
    else if (dma && d == 128) ZI_PF_DMA(128, 1, 2);
    else if (dma && d == 64 && wide && alone) ZI_PF_DMA(64, 2, 1);
    else if (dma && d == 64 && wide) ZI_PF_DMA(64, 2, 2);
    else if (dma && d == 64 && alone) ZI_PF_DMA(64, 1, 1);
    else if (dma && d == 64) ZI_PF_DMA(64, 1, 2);
    else
    switch (d) {
        case 16: ZI_PF(16); break;
        case 32: ZI_PF(32); break;
        case 48: ZI_PF(48); break;
        case 64: ZI_PF(64); break;
        case 80: ZI_PF(80); break;
        case 96: ZI_PF(96); break;
        case 112: ZI_PF(112); break;
        default: ZI_PF(128); break;
    }
#undef ZI_PF
#undef ZI_PF_DMA
    if (max_chunks > 1)
        attention_prefill_merge_kernel<<<dim3(num_tiles * tile, nh), ZI_WAVE, 0, stream>>>(
            (zi_bf16*)out, ldo, po, pml, tile_entry, tile_off, entry_start, entry_len, entry_past, nh, d, window, max_chunks,
            tile, chunk_keys);
    return zi_check_launch("attention_prefill");
}
