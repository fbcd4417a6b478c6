// Paged grouped-query attention for single query tokens, split over the keys, on
// the matrix cores.
//
// One workgroup of four wavefronts per (token, key/value head, chunk of the keys).
// It serves all G = heads / kv_heads query heads of its group from one pass over
// the keys and values, so each cached byte is read once per token: the G heads
// stand in for the 16 "queries" of a v_mfma_f32_16x16x32_bf16 tile (rows beyond G
// are zero).  A token at position p sees keys [lo, p] (lo = 0, or p - window + 1);
// that range, widened down to a multiple of 8, is cut into at most 64 chunks of 256
// keys (512, 1024, ... when there are more than 16384 keys), which depends on the
// token alone, never on the rest of the batch.  Inside a chunk every wavefront takes
// a quarter, in blocks of 64 keys: it loads the block's keys and values straight
// from the cache into matrix-core operands (nothing is shared between wavefronts,
// so nothing goes through LDS), computes the scores transposed, S^T = K . Q^T, so
// that a lane holds the scores of one head, runs the softmax on them in float32,
// and accumulates O^T += V^T . P^T.  The four wavefronts' running (maximum, sum,
// output) are merged through LDS; a token with one chunk is finished there, else
// the chunk leaves a partial and a second kernel merges the chunks in rising order.
// (reference formulas: src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:15-72;
// the scale is applied after the dot product, :44.)
//
// Operand layout: as in the prompt kernel, the keys of a block are assigned to the
// rows of the four score tiles in a permuted order (tile t, row j*4 + e <-> key
// (t/2)*32 + j*8 + (t%2)*4 + e), which makes the eight probabilities a lane holds
// after two tiles the eight consecutive keys that the P.V product wants from it.
// Values are cached transposed ([dim][slot]), so a lane reads 16-byte runs of keys.
//
// bfloat16 only; head_dim a multiple of 16 up to 128; group size up to 16; page size
// a multiple of 8.  Other shapes are the plain kernel's.
#include "zi_common.h"
#include "zi_api.h"
#include "zi_paging.h"

typedef __attribute__((ext_vector_type(8))) __bf16 dec_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float dec_f32x4_t;

#define DEC_MAXC ZI_DEC_MAXC       // most chunks of one token
#define DEC_CHUNK ZI_DEC_CHUNK     // keys of the smallest chunk
#define DEC_WAVES ZI_DEC_WAVES
#define DEC_BLOCK ZI_DEC_BLOCK     // keys a wavefront handles at a time

typedef __attribute__((ext_vector_type(4))) uint32_t dec_u32x4_t;

union dec_pack {
    uint4 u;
    dec_u32x4_t v;
    dec_bf16x8_t b;
    uint16_t h[8];
};

// The cut of a token's keys (DecSplit, dec_split) and every place in the cache come from zi_paging.h.

// The projections of the step's tokens as they leave the matrix product, for the kernel variant that
// rotates and stores them itself (FUSED): row t of `sums` holds the query heads, then the key heads, then
// the value heads, as `splits` float32 partial sums that are added in rising order, then the bias.
// The first `rot` dims of every query and key head turn by the angles of `table` ([token][rot/2][cos,
// sin]); the token's new key and value go to slot slots[t] of the cache.
struct DecProjection {
    const float* sums;
    int splits;
    int64_t split_stride, ldp;
    const void* bias;      // null: none
    int bias_f32;
    const float* table;    // null when rot == 0
    int rot;
    const int32_t* slots;
    int64_t cache_slots;
    int write_kv;
};

template <int D, bool FUSED, int VMODE>
__global__ void __launch_bounds__(DEC_WAVES* ZI_WAVE, 2)
attention_decode_kernel(zi_bf16* __restrict__ out, int64_t ldo, float* __restrict__ part_o,
                        float* __restrict__ part_ml, const zi_bf16* __restrict__ q, int64_t ldq,
                        const zi_bf16* kcache, const zi_bf16* vcache,
                        const int32_t* __restrict__ tok_index, const int32_t* __restrict__ tok_seq,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_tables,
                        int max_pages, int num_pages, int nh, int nkv, int G, int ps, int window, float scale,
                        int max_chunks, int leave_parts, DecProjection pj) {
    static_assert(D % 16 == 0 && D >= 16 && D <= 128, "head_dim must be a multiple of 16 up to 128");
    constexpr int DK = (D + 31) / 32;   // k-steps of the score product
    constexpr int DT = D / 16;          // output tiles of 16 dims
    constexpr bool WHOLE_LINES = D % 64 == 0;   // a key is whole 128-byte lines: see the loads of the keys
    __shared__ float sm[DEC_WAVES][16], sl[DEC_WAVES][16];
    __shared__ dec_f32x4_t so[DEC_WAVES][DT][ZI_WAVE];
    __shared__ uint4 sk[DK][4];        // FUSED: the token's own key, in pieces (k-step, j)
    __shared__ uint16_t sv[D];         // and its value

    // a token's chunks are neighbours in the launch order: those past its count leave at once, beside chunks
    // that stream, and do not gather at the launch's end
    const int x = blockIdx.z, kvh = blockIdx.y, chunk = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int t = tok_index ? tok_index[x] : x;
    const int p = tok_pos[t];
    const DecSplit sp = dec_split(p, window);
    if (sp.count > max_chunks) {
        // The host sized the launch (and the workspace) for fewer keys than this token sees.  Nothing
        // may be written to the workspace then; the token's output is made NaN so that it shows.
        // (With leave_parts the kernel that reads the chunks sees the same count and does that.)
        if (chunk == 0 && !leave_parts)
            for (int i = tid; i < G * D; i += DEC_WAVES * ZI_WAVE)
                zi_store(out + (int64_t)t * ldo + (int64_t)kvh * G * D + i, NAN);
        return;
    }
    if (chunk >= sp.count) return;
    const int32_t* bt = block_tables + (int64_t)(tok_seq ? tok_seq[t] : t) * max_pages;   // no list: token t is of sequence t
    const int ps_shift = (ps & (ps - 1)) == 0 ? __ffs(ps) - 1 : -1;   // no division for the usual page sizes
    const int quarter = sp.len / DEC_WAVES;
    int k_begin, k_end;      // the wavefront's keys; k_end is one past the last
    zi_dec_wave_keys(sp, chunk, wave, p, &k_begin, &k_end);
    const int p8 = p & ~7, pi_last = max_pages - 1;
    // How the values are loaded (VMODE, chosen by the launch: a branch here costs more than it gains).  1: pages of
    // at most 32 tokens, where an instruction's loads cover whole 128-byte lines as they are (sixteen dims' runs of
    // a page's tokens lie side by side): past L2, like the keys.  2: larger pages, where a dim's run of the block's
    // 64 tokens is a line of its own: an instruction takes eight dims' whole lines (lane (r, j): dim r % 8, the
    // eight tokens of piece (r / 8) * 4 + j) and the lanes r and r +- 8 trade halves afterwards, as for the keys;
    // past L2 as well (as halves, non-temporal: 148 against 125 us at page 64).  0: plain loads of halves.
    constexpr bool v_lines = VMODE == 1, v_trade = VMODE == 2;

    // FUSED: eight consecutive columns of the token's projection row (splits added in rising order, then
    // the bias), and the same after the rotation of head column `hc`, dims dim0 .. dim0 + 7.  Four
    // splits' loads are issued at a time (the split index is clamped, what is past the count adds zero).
    const int half = pj.rot / 2;
    auto value8 = [&](int col, float (&v)[8]) {
        const float* p0 = pj.sums + (int64_t)t * pj.ldp + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
        auto four = [&](int s0) {
            float4 a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float* ps2 = p0 + (int64_t)(s0 + u < pj.splits ? s0 + u : s0) * pj.split_stride;
                a[u] = *reinterpret_cast<const float4*>(ps2);
                b[u] = *reinterpret_cast<const float4*>(ps2 + 4);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float keep = s0 + u < pj.splits ? 1.f : 0.f;     // x * 1 is exact; sums are finite
                v[0] += a[u].x * keep; v[1] += a[u].y * keep; v[2] += a[u].z * keep; v[3] += a[u].w * keep;
                v[4] += b[u].x * keep; v[5] += b[u].y * keep; v[6] += b[u].z * keep; v[7] += b[u].w * keep;
            }
        };
        four(0);      // straight-line: the loads of several calls travel together
        for (int s0 = 4; s0 < pj.splits; s0 += 4) four(s0);
        if (pj.bias) {
            if (pj.bias_f32) {
                const float4 a = *reinterpret_cast<const float4*>((const float*)pj.bias + col);
                const float4 b = *reinterpret_cast<const float4*>((const float*)pj.bias + col + 4);
                v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
            } else {
                dec_pack w;
                w.u = *reinterpret_cast<const uint4*>((const zi_bf16*)pj.bias + col);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += __uint_as_float((uint32_t)w.h[e] << 16);
            }
        }
    };
    // one column of the row, the same sum
    auto value1 = [&](int col) {
        const float* p0 = pj.sums + (int64_t)t * pj.ldp + col;
        float v = 0.f;
        auto four = [&](int s0) {
            float a[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) a[u] = p0[(int64_t)(s0 + u < pj.splits ? s0 + u : s0) * pj.split_stride];
#pragma unroll
            for (int u = 0; u < 4; ++u) v += a[u] * (s0 + u < pj.splits ? 1.f : 0.f);
        };
        four(0);
        for (int s0 = 4; s0 < pj.splits; s0 += 4) four(s0);
        if (pj.bias) v += pj.bias_f32 ? ((const float*)pj.bias)[col] : zi_load((const zi_bf16*)pj.bias + col);
        return v;
    };
    auto rotated8 = [&](int hc, int dim0) {
        float a[8];
        value8(hc + dim0, a);
        if (dim0 < pj.rot) {     // rot / 2 is a multiple of 8 (host): the eight dims lie on one side
            const bool first = dim0 < half;
            float b[8];
            value8(hc + (first ? dim0 + half : dim0 - half), b);
            const float4* cs = reinterpret_cast<const float4*>(pj.table + ((int64_t)t * half + (first ? dim0 : dim0 - half)) * 2);
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const float4 w = cs[e2];     // cos, sin of two pairs
                a[2 * e2] = first ? a[2 * e2] * w.x - b[2 * e2] * w.y : a[2 * e2] * w.x + b[2 * e2] * w.y;
                a[2 * e2 + 1] = first ? a[2 * e2 + 1] * w.z - b[2 * e2 + 1] * w.w : a[2 * e2 + 1] * w.z + b[2 * e2 + 1] * w.w;
            }
        }
        dec_pack w;
        w.u.x = zi_pack_bf16x2(a[0], a[1]); w.u.y = zi_pack_bf16x2(a[2], a[3]);
        w.u.z = zi_pack_bf16x2(a[4], a[5]); w.u.w = zi_pack_bf16x2(a[6], a[7]);
        return w;
    };
    // The group's queries as the B operand: lane (r, j) holds head r, dims dk*32 + j*8 ...  FUSED: every
    // wavefront wants the same operand, so each makes the pieces of one k-step and they trade through
    // LDS.  In the workgroup of the last chunk, which holds position p, they make the token's own key
    // (a row of lanes that has no query head, or a second pass) and value the same way.  The wavefront
    // that owns position p stores them to the cache and puts them into its operands; nobody else reads
    // that slot in this kernel.
    const bool last_chunk = FUSED && pj.write_kv && chunk == sp.count - 1;
    const bool owner = last_chunk && p >= k_begin && p < k_begin + quarter;
    // where position p sits in the operands of its block: score tile tt_p, row r_p; value operand b_p,
    // lanes j_p, element e_p
    const int kk_p = (p - k_begin) % DEC_BLOCK;
    const int tt_p = (kk_p / 32) * 2 + (kk_p % 8) / 4, r_p = ((kk_p % 32) / 8) * 4 + kk_p % 4;
    const int b_p = kk_p / 32, j_p = (kk_p % 32) / 8, e_p = kk_p % 8;
    uint4 knew[DK];
    uint32_t vnew[DT / 2 + 1];
    dec_bf16x8_t qop[DK];
    if (FUSED) {
        uint4* sq = reinterpret_cast<uint4*>(&so[0][0][0]);      // [DK][64]; the merge uses `so` much later
        const int key_row = G < 16 ? G : 0;      // the lanes that make the key's pieces
        for (int dk = wave; dk < DK; dk += DEC_WAVES) {
            const bool piece = dk * 32 + j * 8 < D;
            const bool for_key = last_chunk && G < 16 && r == key_row;
            dec_pack w;
            w.u = make_uint4(0, 0, 0, 0);
            if ((r < G || for_key) && piece) w = rotated8(for_key ? (nh + kvh) * D : (kvh * G + r) * D, dk * 32 + j * 8);
            if (for_key) {
                sk[dk][j] = w.u;
                w.u = make_uint4(0, 0, 0, 0);
            }
            sq[dk * ZI_WAVE + lane] = w.u;
            if (last_chunk && G == 16 && r == key_row) {
                dec_pack w2;
                w2.u = make_uint4(0, 0, 0, 0);
                if (piece) w2 = rotated8((nh + kvh) * D, dk * 32 + j * 8);
                sk[dk][j] = w2.u;
            }
        }
        if (last_chunk)
            for (int dim = threadIdx.x; dim < D; dim += DEC_WAVES * ZI_WAVE)
                sv[dim] = zi_float_to_bf16(value1((nh + nkv + kvh) * D + dim));
        __syncthreads();
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            dec_pack w;
            w.u = sq[dk * ZI_WAVE + lane];
            qop[dk] = w.b;
        }
        if (owner) {
            const ZiSlotPlace place = zi_slot_place(pj.slots[t], pj.cache_slots, ps);   // the host checks the range; never write outside the pool
            const bool inside = place.ok;
            const int64_t page = place.page, off = place.off;
#pragma unroll
            for (int dk = 0; dk < DK; ++dk) {
                knew[dk] = sk[dk][j];
                if (inside && r == r_p && dk * 32 + j * 8 < D)
                    *reinterpret_cast<uint4*>(const_cast<zi_bf16*>(kcache) + zi_key_offset(page, kvh, (int)off, nkv, ps, D) + dk * 32 + j * 8) = knew[dk];
            }
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) {
                const int dim = dd * 16 + r;
                const uint32_t hv = sv[dim];
                if (inside && j == j_p)
                    const_cast<zi_bf16*>(vcache)[zi_value_offset(page, kvh, dim, (int)off, nkv, ps, D)].bits = (uint16_t)hv;
                vnew[dd / 2] = (dd & 1) ? (vnew[dd / 2] | (hv << 16)) : hv;
            }
        }
    } else {
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            dec_pack w;
            w.u = make_uint4(0, 0, 0, 0);
            if (r < G && dk * 32 + j * 8 < D)
                w.u = *reinterpret_cast<const uint4*>(q + (int64_t)t * ldq + (int64_t)(kvh * G + r) * D + dk * 32 + j * 8);
            qop[dk] = w.b;
        }
    }
    dec_f32x4_t o[DT];
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) o[dd] = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, lsum = 0.f;   // m is in base-2 units: the maximum of s * scale * log2(e)
    const float scale_log2 = scale * 1.4426950408889634f;

    for (int base = k_begin; base < k_end; base += DEC_BLOCK) {
        // ---- all loads of the block first, in straight-line code: the six table lookups, then keys
        // (4 tiles x DK) and values (DT x 2) from addresses clamped into the sequence and the pool.  What
        // must not count is masked afterwards; with a branch around a load the compiler would wait for it
        // on the spot, one tile after the other.
        dec_pack kop[4][DK], vop[DT][2];
        int kpage[4], kslot[4], vpage[2], vslot[2];
        // Head sizes that are whole 128-byte lines (WHOLE_LINES): a load instruction takes eight keys' lines whole
        // instead of sixteen keys' halves (lane (r, j): row hf * 8 + r % 8 of the tile, piece (r / 8) * 4 + j of
        // line L), and the halves change places between lanes r and r +- 8 afterwards.  Keys and values are read
        // once a step: whole lines can be loaded non-temporally, past L2 (halves cannot: the line's other half
        // would come from memory again).  Decode at the 1.5B sizes, 2,100-token contexts, same box, halves and
        // plain loads against whole lines and non-temporal loads of keys and values: batch 8 5,480 to 5,660 tok/s,
        // batch 64 25.5k to 26.5k, batch 256 41.0k to 42.6k (values alone: 41.9k; keys alone, as halves: slower).
        int kpage2[4][2], kslot2[4][2];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            if constexpr (WHOLE_LINES) {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const ZiTablePlace at = zi_table_place(zi_dec_tile_key(base, tt, hf * 8 + (r & 7)), p, ps, ps_shift, pi_last);
                    kslot2[tt][hf] = at.slot;
                    kpage2[tt][hf] = bt[at.index];
                }
            } else {
                const ZiTablePlace at = zi_table_place(zi_dec_tile_key(base, tt, r), p, ps, ps_shift, pi_last);
                kslot[tt] = at.slot;
                kpage[tt] = bt[at.index];
            }
        }
        if constexpr (v_trade) {      // this lane's eight tokens: piece (r / 8) * 4 + j of the block
            const ZiTablePlace at = zi_table_place(base + ((r >> 3) * 4 + j) * 8, p8, ps, ps_shift, pi_last);
            vslot[0] = at.slot;
            vpage[0] = bt[at.index];
        } else {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const ZiTablePlace at = zi_table_place(zi_dec_value_key0(base, b, j), p8, ps, ps_shift, pi_last);
                vslot[b] = at.slot;
                vpage[b] = bt[at.index];
            }
        }
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            if constexpr (WHOLE_LINES) {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const int page = zi_page_or_zero(kpage2[tt][hf], num_pages);   // a window may have freed it
                    const zi_bf16* kr = kcache + zi_key_offset(page, kvh, kslot2[tt][hf], nkv, ps, D) + ((r >> 3) * 4 + j) * 8;
#pragma unroll
                    for (int L = 0; L < DK / 2; ++L)     // kop[tt][2L + hf] for now: rows hf * 8 .. + 7, all eight pieces of line L
                        kop[tt][2 * L + hf].v = __builtin_nontemporal_load(reinterpret_cast<const dec_u32x4_t*>(kr + L * 64));
                }
            } else {
                const int page = zi_page_or_zero(kpage[tt], num_pages);   // a window may have freed it
                const zi_bf16* kr = kcache + zi_key_offset(page, kvh, kslot[tt], nkv, ps, D);
#pragma unroll
                for (int dk = 0; dk < DK; ++dk)
                    kop[tt][dk].u = *reinterpret_cast<const uint4*>(kr + ((D % 32 == 0 || dk * 32 + j * 8 < D) ? dk * 32 + j * 8 : 0));
            }
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if constexpr (v_trade) {      // vop[dd][b] for now: dims dd * 16 + b * 8 .. + 7, all 64 tokens
                const int page = zi_page_or_zero(vpage[0], num_pages);
                const zi_bf16* vr = vcache + zi_value_offset(page, kvh, b * 8 + (r & 7), vslot[0], nkv, ps, D);
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) vop[dd][b].v = __builtin_nontemporal_load(reinterpret_cast<const dec_u32x4_t*>(vr + (int64_t)dd * 16 * ps));
                continue;
            }
            const int page = zi_page_or_zero(vpage[b], num_pages);
            const zi_bf16* vr = vcache + zi_value_offset(page, kvh, r, vslot[b], nkv, ps, D);
            if constexpr (v_lines) {
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) vop[dd][b].v = __builtin_nontemporal_load(reinterpret_cast<const dec_u32x4_t*>(vr + (int64_t)dd * 16 * ps));
            } else {
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) vop[dd][b].v = *reinterpret_cast<const dec_u32x4_t*>(vr + (int64_t)dd * 16 * ps);
            }
        }
        if constexpr (WHOLE_LINES) {
            // lanes r < 8 hold rows r of both loads' pieces 0..3, lanes r >= 8 rows r - 8 with pieces 4..7: k-step 2L
            // wants row r's pieces 0..3 (lanes >= 8 take them from the second load's lanes r - 8), k-step 2L + 1
            // pieces 4..7 (lanes < 8 take them from the first load's lanes r + 8).  A rotation by eight lanes within
            // every row of sixteen, written to half the lanes.
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int L = 0; L < DK / 2; ++L) {
                    const dec_u32x4_t a = kop[tt][2 * L].v, b = kop[tt][2 * L + 1].v;
                    dec_u32x4_t lo, hi;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        lo[w] = (uint32_t)__builtin_amdgcn_update_dpp((int)a[w], (int)b[w], 0x128, 0xf, 0xc, false);
                        hi[w] = (uint32_t)__builtin_amdgcn_update_dpp((int)b[w], (int)a[w], 0x128, 0xf, 0x3, false);
                    }
                    kop[tt][2 * L].v = lo;
                    kop[tt][2 * L + 1].v = hi;
                }
        }
        if constexpr (v_trade) {
#pragma unroll
            for (int dd = 0; dd < DT; ++dd) {
                const dec_u32x4_t a = vop[dd][0].v, b = vop[dd][1].v;
                dec_u32x4_t lo, hi;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    lo[w] = (uint32_t)__builtin_amdgcn_update_dpp((int)a[w], (int)b[w], 0x128, 0xf, 0xc, false);
                    hi[w] = (uint32_t)__builtin_amdgcn_update_dpp((int)b[w], (int)a[w], 0x128, 0xf, 0x3, false);
                }
                vop[dd][0].v = lo;
                vop[dd][1].v = hi;
            }
        }
        if (D % 32 != 0) {   // the padding of the last k-step must be zero: the query is, but 0 * NaN is not
            const unsigned keep = (DK - 1) * 32 + j * 8 < D ? ~0u : 0u;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                uint4& u = kop[tt][DK - 1].u;
                u.x &= keep; u.y &= keep; u.z &= keep; u.w &= keep;
            }
        }
        // Keys outside [lo, p] get the score -inf below, whatever was loaded for them.  Their values
        // must be zero, since 0 * NaN is NaN: slots outside the range may hold anything.
        if (base < sp.lo || base + DEC_BLOCK > k_end) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int key0 = zi_dec_value_key0(base, b, j);
                unsigned keep[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int ka = key0 + 2 * e, kb2 = ka + 1;
                    keep[e] = ((ka >= sp.lo && ka < k_end) ? 0xffffu : 0u) | ((kb2 >= sp.lo && kb2 < k_end) ? 0xffff0000u : 0u);
                }
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) {
                    uint4& u = vop[dd][b].u;
                    u.x &= keep[0]; u.y &= keep[1]; u.z &= keep[2]; u.w &= keep[3];
                }
            }
        }
        if (FUSED && owner && p < base + DEC_BLOCK) {     // the last block (p >= base: k_end = p + 1)
            if (r == r_p) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int dk = 0; dk < DK; ++dk)
                        if (tt == tt_p) kop[tt][dk].u = knew[dk];
            }
            if (j == j_p) {
                const uint32_t keep = (e_p & 1) ? 0x0000ffffu : 0xffff0000u;
#pragma unroll
                for (int dd = 0; dd < DT; ++dd) {
                    const uint32_t hv = (vnew[dd / 2] >> (16 * (dd & 1))) & 0xffffu, put = (e_p & 1) ? hv << 16 : hv;
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        if (b != b_p) continue;
                        uint4& u = vop[dd][b].u;
                        if (e_p / 2 == 0) u.x = (u.x & keep) | put;
                        if (e_p / 2 == 1) u.y = (u.y & keep) | put;
                        if (e_p / 2 == 2) u.z = (u.z & keep) | put;
                        if (e_p / 2 == 3) u.w = (u.w & keep) | put;
                    }
                }
            }
        }
        // ---- scores of 64 keys for this lane's head
        dec_f32x4_t s[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            s[tt] = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dk = 0; dk < DK; ++dk)
                s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[tt][dk].b, qop[dk], s[tt], 0, 0, 0);
        }
        // softmax in base 2: t = s * scale * log2(e), p = 2^(t - m)
        const bool whole = base >= sp.lo && base + DEC_BLOCK <= k_end;
        float mx = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = zi_dec_score_key(base, tt, j, e);
                const float v = (whole || (key >= sp.lo && key < k_end)) ? s[tt][e] * scale_log2 : -INFINITY;
                s[tt][e] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_use);      // 2^(-inf) = 0 before the first key
        m = m_new;
        float psum = 0.f;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[tt][e] = __builtin_amdgcn_exp2f(s[tt][e] - m_use);   // 0 for keys not seen
                psum += s[tt][e];
            }
        dec_pack pb[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            pb[b].u.x = zi_pack_bf16x2(s[2 * b][0], s[2 * b][1]);
            pb[b].u.y = zi_pack_bf16x2(s[2 * b][2], s[2 * b][3]);
            pb[b].u.z = zi_pack_bf16x2(s[2 * b + 1][0], s[2 * b + 1][1]);
            pb[b].u.w = zi_pack_bf16x2(s[2 * b + 1][2], s[2 * b + 1][3]);
        }
        lsum = lsum * corr + psum;
#pragma unroll
        for (int dd = 0; dd < DT; ++dd) {
            o[dd][0] *= corr; o[dd][1] *= corr; o[dd][2] *= corr; o[dd][3] *= corr;
#pragma unroll
            for (int b = 0; b < 2; ++b)
                o[dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[dd][b].b, pb[b].b, o[dd], 0, 0, 0);
        }
    }
    // ---- merge the four wavefronts: head r's (m, l) and this lane's outputs
    lsum += __shfl_xor(lsum, 16, ZI_WAVE);
    lsum += __shfl_xor(lsum, 32, ZI_WAVE);
    if (j == 0) {
        sm[wave][r] = m;
        sl[wave][r] = lsum;
    }
#pragma unroll
    for (int dd = 0; dd < DT; ++dd) so[wave][dd][lane] = o[dd];
    __syncthreads();
    float M = sm[0][r];
#pragma unroll
    for (int w = 1; w < DEC_WAVES; ++w) M = fmaxf(M, sm[w][r]);
    float a[DEC_WAVES], L = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) {
        a[w] = (sm[w][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sm[w][r] - M);
        L += a[w] * sl[w][r];
    }
    const bool final = sp.count == 1 && !leave_parts;
    const float inv = final ? 1.f / L : 1.f;
    const int64_t slot = zi_dec_part_slot(x, nh, kvh * G + r, chunk);
    for (int dd = wave; dd < DT; dd += DEC_WAVES) {
        dec_f32x4_t acc = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const dec_f32x4_t v = so[w][dd][lane];
            acc[0] += a[w] * v[0]; acc[1] += a[w] * v[1]; acc[2] += a[w] * v[2]; acc[3] += a[w] * v[3];
        }
        if (r >= G) continue;
        if (final) {
            uint2 wv;
            wv.x = zi_pack_bf16x2(acc[0] * inv, acc[1] * inv);
            wv.y = zi_pack_bf16x2(acc[2] * inv, acc[3] * inv);
            *reinterpret_cast<uint2*>(out + (int64_t)t * ldo + (int64_t)(kvh * G + r) * D + dd * 16 + j * 4) = wv;
        } else {
            *reinterpret_cast<dec_f32x4_t*>(part_o + slot * D + dd * 16 + j * 4) = acc;
        }
    }
    if (!final && wave == 0 && j == 0 && r < G) {
        part_ml[slot * 2] = M;
        part_ml[slot * 2 + 1] = L;
    }
}

// Merge the chunks of one (token, head): out = sum_c e^(m_c - M) o_c / sum_c e^(m_c - M) l_c.
__global__ void __launch_bounds__(ZI_WAVE)
attention_decode_merge_kernel(zi_bf16* __restrict__ out, int64_t ldo, const float* __restrict__ part_o,
                              const float* __restrict__ part_ml, const int32_t* __restrict__ tok_index,
                              const int32_t* __restrict__ tok_pos, int nh, int D, int window, int max_chunks) {
    const int x = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int t = tok_index ? tok_index[x] : x;
    const DecSplit sp = dec_split(tok_pos[t], window);
    if (sp.count == 1 || sp.count > max_chunks) return;
    const int64_t slot0 = zi_dec_part_slot(x, nh, h, 0);
    // chunk c's (m, l) sit in lane c
    const float mc = lane < sp.count ? part_ml[(slot0 + lane) * 2] : -INFINITY;
    const float lc = lane < sp.count ? part_ml[(slot0 + lane) * 2 + 1] : 0.f;
    const float M = zi_wave_max(mc);
    const float wc = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - M);   // maxima are in base-2 units
    float L = 0.f, acc[2] = {0.f, 0.f};
    for (int c0 = 0; c0 < sp.count; c0 += 8) {
        float po[8][2];   // eight chunks' loads are issued before the first is used
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int v = 0; v < 2; ++v)
                po[c][v] = (c0 + c < sp.count && lane + v * ZI_WAVE < D)
                               ? part_o[(slot0 + c0 + c) * D + lane + v * ZI_WAVE] : 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float w = __shfl(wc, (c0 + c) & (ZI_WAVE - 1), ZI_WAVE);   // 0 for chunks past the count
            L += w * __shfl(lc, (c0 + c) & (ZI_WAVE - 1), ZI_WAVE);
            acc[0] += w * po[c][0];
            acc[1] += w * po[c][1];
        }
    }
    const float inv = 1.f / L;
#pragma unroll
    for (int v = 0; v < 2; ++v)
        if (lane + v * ZI_WAVE < D) zi_store(out + (int64_t)t * ldo + (int64_t)h * D + lane + v * ZI_WAVE, acc[v] * inv);
}

// The output projection straight from the chunks: sums[s][t][:] = W[:, heads of split s] . merged
// attention of token t for those heads, as float32 partial sums over groups of `hg` heads that the
// next kernel adds in rising order.  One workgroup per (64 rows of W, group of heads): thread (token,
// eight dims) merges the token's chunks for a head as the merge kernel does (maximum first, then the
// weighted sums in rising order; the result is rounded to bfloat16 as if it had been stored), the
// four wavefronts multiply 16 rows each on the matrix cores with the up to 16 tokens as columns.
// The attention kernel must have left every token's chunks in the workspace (leave_parts).  A token
// that sees more chunks than the launch covered gets NaN.
#define DPJ_ROWS 64
template <int D>
__global__ void __launch_bounds__(256)
attention_decode_project_kernel(float* __restrict__ sums, const float* __restrict__ part_o,
                                const float* __restrict__ part_ml, const int32_t* __restrict__ tok_pos, int n, int nh,
                                int window, int max_chunks, const zi_bf16* __restrict__ w, int64_t ldw, int N, int hg) {
    constexpr int DK = (D + 31) / 32;
    constexpr int XS = DK * 32 + 8;     // row stride of the merged head in LDS, in elements (16-byte rows, no bank repeat)
    __shared__ __attribute__((aligned(16))) uint16_t sx[16][XS];
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int r = lane & 15, j = lane >> 4;
    const int split = blockIdx.y, h0 = split * hg, h1 = (h0 + hg < nh) ? h0 + hg : nh;
    const int row = blockIdx.x * DPJ_ROWS + wave * 16 + r;
    const zi_bf16* wr = w + (int64_t)(row < N ? row : N - 1) * ldw;
    // the merging thread's token and dims
    const int mt = tid >> 4, d0 = (tid & 15) * 8;
    dec_f32x4_t acc = dec_f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int h = h0; h < h1; ++h) {
        // ---- the weights of this head's columns first: they do not wait for the merge
        dec_pack a[DK];
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            const bool in = dk * 32 + j * 8 < D;
            a[dk].u = *reinterpret_cast<const uint4*>(wr + (int64_t)h * D + (in ? dk * 32 + j * 8 : 0));
        }
        // ---- merge: eight dims of one token.  The sixteen lanes of a token share its chunks' (maximum,
        // sum): lane q loads those of chunks q, q + 16, ..., and they trade maxima and weights by
        // shuffles, as the merge kernel's lanes do.  These loads and the first eight chunks' outputs
        // travel together.
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
        const int q = tid & 15, mtc = mt < n ? mt : n - 1;
        const int count = dec_split(tok_pos[mtc], window).count;
        const int64_t slot0 = zi_dec_part_slot(mtc, nh, h, 0);
        const float2* ml = reinterpret_cast<const float2*>(part_ml) + slot0;
        const float* po0 = part_o + slot0 * D + (d0 < D ? d0 : 0);
        float2 mlq[DEC_MAXC / 16];
        float4 lo[8], hi[8];
#pragma unroll
        for (int u = 0; u < DEC_MAXC / 16; ++u) mlq[u] = ml[q + 16 * u < count ? q + 16 * u : 0];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int cc = c < count ? c : 0;
            lo[c] = *reinterpret_cast<const float4*>(po0 + (int64_t)cc * D);
            hi[c] = *reinterpret_cast<const float4*>(po0 + (int64_t)cc * D + 4);
        }
        float M = -INFINITY;
#pragma unroll
        for (int u = 0; u < DEC_MAXC / 16; ++u) M = fmaxf(M, q + 16 * u < count ? mlq[u].x : -INFINITY);
#pragma unroll
        for (int off = 1; off < 16; off *= 2) M = fmaxf(M, __shfl_xor(M, off, ZI_WAVE));
        // maxima are in base-2 units; a chunk without keys has maximum -inf and weight 0
        float wq[DEC_MAXC / 16], lq[DEC_MAXC / 16];
#pragma unroll
        for (int u = 0; u < DEC_MAXC / 16; ++u) {
            const bool use = q + 16 * u < count && mlq[u].x != -INFINITY;
            wq[u] = use ? __builtin_amdgcn_exp2f(mlq[u].x - M) : 0.f;
            lq[u] = use ? mlq[u].y : 0.f;
        }
        float L = 0.f;
        const int lane0 = lane & ~15;
#pragma unroll
        for (int u = 0; u < DEC_MAXC / 16; ++u) {
            if (u * 16 >= count) break;      // uniform over the token's lanes
            for (int c0 = u * 16; c0 < u * 16 + 16 && c0 < count; c0 += 8) {
                if (c0 > 0) {
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        const int cc = c0 + c < count ? c0 + c : c0;
                        lo[c] = *reinterpret_cast<const float4*>(po0 + (int64_t)cc * D);
                        hi[c] = *reinterpret_cast<const float4*>(po0 + (int64_t)cc * D + 4);
                    }
                }
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const int src = lane0 + ((c0 + c) & 15);
                    const float wc = __shfl(wq[u], src, ZI_WAVE);     // 0 for chunks past the count
                    L += wc * __shfl(lq[u], src, ZI_WAVE);
                    v[0] += wc * lo[c].x; v[1] += wc * lo[c].y; v[2] += wc * lo[c].z; v[3] += wc * lo[c].w;
                    v[4] += wc * hi[c].x; v[5] += wc * hi[c].y; v[6] += wc * hi[c].z; v[7] += wc * hi[c].w;
                }
            }
        }
        {
            const float inv = count > max_chunks ? NAN : 1.f / L;      // chunks the launch did not cover: it shows
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= inv;
        }
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {     // the padding of the last k-step is zero on both sides
            const unsigned keep = dk * 32 + j * 8 < D ? ~0u : 0u;
            a[dk].u.x &= keep; a[dk].u.y &= keep; a[dk].u.z &= keep; a[dk].u.w &= keep;
        }
        if (h > h0) __syncthreads();        // the last head's operands have been read
        if (d0 < DK * 32) {
            uint4 u;
            u.x = zi_pack_bf16x2(v[0], v[1]); u.y = zi_pack_bf16x2(v[2], v[3]);
            u.z = zi_pack_bf16x2(v[4], v[5]); u.w = zi_pack_bf16x2(v[6], v[7]);
            if (mt >= n || d0 >= D) u = make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4*>(&sx[mt][d0]) = u;
        }
        __syncthreads();
#pragma unroll
        for (int dk = 0; dk < DK; ++dk) {
            dec_pack b;
            b.u = *reinterpret_cast<const uint4*>(&sx[r][dk * 32 + j * 8]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[dk].b, b.b, acc, 0, 0, 0);
        }
    }
    // lane (r, j) holds rows 4j .. 4j+3 of its wavefront's tile for token r
    if (r < n) {
        const int row0 = blockIdx.x * DPJ_ROWS + wave * 16 + j * 4;
        float* dst = sums + ((int64_t)split * n + r) * N + row0;
        if ((N & 3) == 0 && row0 + 3 < N) {
            *reinterpret_cast<dec_f32x4_t*>(dst) = acc;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (row0 + e < N) dst[e] = acc[e];
        }
    }
}

// Floats of workspace the split kernel needs for n tokens.
extern "C" int64_t zi_attention_decode_workspace(int n, int nh, int d) { return zi_dec_workspace_floats(n, nh, d); }

// Chunks the launch must cover when no token sees more than `keys` keys (position + 1, or the window).
extern "C" int zi_attention_decode_chunks(int keys) {
    if (keys < 1) keys = 1;
    // the range is widened down to a multiple of 8: up to 7 more keys.  Past DEC_CHUNK * DEC_MAXC keys
    // the chunks grow and their number drops again, but a token with fewer keys may still need them all.
    if (keys + 7 > DEC_CHUNK * DEC_MAXC) return DEC_MAXC;
    return dec_split(keys - 1 + 7, 0).count;
}

// 1 when the shape is this kernel's, else 0.
extern "C" int zi_attention_decode_supported(int dt, int nh, int nkv, int d, int page_size) {
    if (dt != ZI_BF16 || nkv <= 0 || nh <= 0 || nh % nkv) return 0;
    const int G = nh / nkv;
    return d >= 16 && d <= 128 && d % 16 == 0 && G <= 16 && page_size > 0 && page_size % 8 == 0;
}

// Checks and launches shared by the two entry points; `pj` is null for queries that come rotated in q.
static int dec_launch(const char* who, void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo,
                      const void* kcache, const void* vcache, const int32_t* tok_index, const int32_t* tok_seq,
                      const int32_t* tok_pos, const int32_t* block_tables, int max_pages, int num_pages, int nh, int nkv,
                      int d, int page_size, int window, float scale, int max_chunks, float* workspace,
                      int64_t workspace_floats, const DecProjection* pj, hipStream_t stream) {
    ZI_REQUIRE(zi_attention_decode_supported(dt, nh, nkv, d, page_size),
               "%s: unsupported shape (bfloat16, head_dim a multiple of 16 up to 128, group <= 16, "
               "page size %% 8 == 0): dtype %d heads %d kv_heads %d head_dim %d page %d", who, dt, nh, nkv, d, page_size);
    ZI_REQUIRE(n_idx >= 0 && max_pages > 0 && num_pages > 0 && window >= 0, "%s: bad sizes", who);
    ZI_REQUIRE(max_chunks >= 1 && max_chunks <= DEC_MAXC, "%s: max_chunks %d outside 1..%d", who, max_chunks, DEC_MAXC);
    const int leave_parts = out == nullptr;     // the chunks stay in the workspace for zi_attention_decode_project
    ZI_REQUIRE((leave_parts || (ldo >= (int64_t)nh * d && ldo % 4 == 0)) && (pj || (ldq >= (int64_t)nh * d && ldq % 8 == 0)),
               "%s: bad row stride", who);
    ZI_REQUIRE((pj || ((uintptr_t)q % 16) == 0) && ((uintptr_t)out % 8) == 0 && ((uintptr_t)kcache % 16) == 0 &&
                   ((uintptr_t)vcache % 16) == 0,
               "%s: q, out and the caches must be aligned to 16 bytes", who);
    ZI_REQUIRE(nkv <= 65535 && nh <= 65535, "%s: too many heads", who);
    if (n_idx == 0) return 0;
    ZI_REQUIRE((max_chunks == 1 && !leave_parts) ||
                   (workspace && workspace_floats >= zi_attention_decode_workspace(n_idx, nh, d) &&
                                   ((uintptr_t)workspace % 16) == 0),
               "%s: workspace of %lld floats is too small or not aligned", who, (long long)workspace_floats);
    float* po = workspace;
    float* pml = workspace ? workspace + (int64_t)n_idx * nh * DEC_MAXC * d : nullptr;
    ZI_REQUIRE(n_idx <= 65535, "%s: at most 65535 tokens a launch, got %d", who, n_idx);
    const dim3 grid(max_chunks, nkv, n_idx);
    const int G = nh / nkv;
    const DecProjection none = {};
#define ZI_DEC(DD, VMODE)                                                                                            \
    if (pj)                                                                                                          \
        attention_decode_kernel<DD, true, VMODE><<<grid, DEC_WAVES * ZI_WAVE, 0, stream>>>(                                 \
            (zi_bf16*)out, ldo, po, pml, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache,     \
            tok_index, tok_seq, tok_pos, block_tables, max_pages, num_pages, nh, nkv, G, page_size, window, scale,   \
            max_chunks, leave_parts, *pj);                                                                                      \
    else                                                                                                             \
        attention_decode_kernel<DD, false, VMODE><<<grid, DEC_WAVES * ZI_WAVE, 0, stream>>>(                                \
            (zi_bf16*)out, ldo, po, pml, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache,     \
            tok_index, tok_seq, tok_pos, block_tables, max_pages, num_pages, nh, nkv, G, page_size, window, scale,   \
            max_chunks, leave_parts, none)
    switch (d) {
        case 16: ZI_DEC(16, 0); break;
        case 32: ZI_DEC(32, 0); break;
        case 48: ZI_DEC(48, 0); break;
        case 64:
            if (page_size <= 32) { ZI_DEC(64, 1); } else { ZI_DEC(64, 2); }
            break;
        case 80: ZI_DEC(80, 0); break;
        case 96: ZI_DEC(96, 0); break;
        case 112: ZI_DEC(112, 0); break;
        default:
            if (page_size <= 32) { ZI_DEC(128, 1); } else { ZI_DEC(128, 2); }
            break;
    }
#undef ZI_DEC
    if (max_chunks > 1 && !leave_parts)
        attention_decode_merge_kernel<<<dim3(n_idx, nh), ZI_WAVE, 0, stream>>>((zi_bf16*)out, ldo, po, pml, tok_index,
                                                                              tok_pos, nh, d, window, max_chunks);
    return zi_check_launch(who);
}

extern "C" int zi_attention_decode(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo,
                                   const void* kcache, const void* vcache, const int32_t* tok_index,
                                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables,
                                   int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window,
                                   float scale, int max_chunks, float* workspace, int64_t workspace_floats,
                                   hipStream_t stream) {
    return dec_launch("attention_decode", out, q, dt, n_idx, ldq, ldo, kcache, vcache, tok_index, tok_seq, tok_pos,
                      block_tables, max_pages, num_pages, nh, nkv, d, page_size, window, scale, max_chunks, workspace,
                      workspace_floats, nullptr, stream);
}

// 1 when the fused entry point takes this projection layout, else 0 (then: rotate and store first, and
// call zi_attention_decode).
extern "C" int zi_attention_decode_fused_supported(int dt, int nh, int nkv, int d, int page_size, int rot, int splits,
                                                   int64_t split_stride, int64_t ldp) {
    if (!zi_attention_decode_supported(dt, nh, nkv, d, page_size)) return 0;
    if (rot < 0 || rot > d || rot % 16) return 0;      // rot / 2 a multiple of 8: eight dims on one side
    if (splits < 1 || ldp % 4 || (splits > 1 && split_stride % 4)) return 0;
    return ldp >= (int64_t)(nh + 2 * nkv) * d;
}

// The same attention for tokens whose projections arrive as float32 partial sums (see DecProjection):
// the kernel adds and rotates them itself and writes each token's new key and value to the cache, when
// `write_kv`.  Every token must be the only one of its sequence in the call: a token's keys must not be
// written by another token of the same call.  `table` holds cos and sin per (token, pair), from
// zi_rope_table; `dt` is the type of the caches and of out; `bias` is bfloat16 or float32 (bias_dt).
// `tok_seq` may be null (here and in zi_attention_decode): token t is then of sequence t, row t of
// block_tables.  With out == nullptr the chunks stay unmerged in the workspace for
// zi_attention_decode_project.
extern "C" int zi_attention_decode_fused(void* out, int dt, int n_idx, int64_t ldo, const float* sums, int splits,
                                         int64_t split_stride, int64_t ldp, const void* bias, int bias_dt,
                                         const float* table, int rot, const int32_t* slots, int64_t cache_slots,
                                         int write_kv, void* kcache, void* vcache, const int32_t* tok_index,
                                         const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables,
                                         int max_pages, int num_pages, int nh, int nkv, int d, int page_size,
                                         int window, float scale, int max_chunks, float* workspace,
                                         int64_t workspace_floats, hipStream_t stream) {
    ZI_REQUIRE(zi_attention_decode_fused_supported(dt, nh, nkv, d, page_size, rot, splits, split_stride, ldp),
               "attention_decode_fused: unsupported projection layout (rotary dims %d a multiple of 16 within head_dim %d, "
               "row and split strides multiples of 4: %lld, %lld)", rot, d, (long long)ldp, (long long)split_stride);
    ZI_REQUIRE(sums && ((uintptr_t)sums % 16) == 0, "attention_decode_fused: sums must be aligned to 16 bytes");
    ZI_REQUIRE(rot == 0 || (table && ((uintptr_t)table % 16) == 0), "attention_decode_fused: no angle table, or not aligned");
    ZI_REQUIRE(((uintptr_t)bias % 16) == 0, "attention_decode_fused: bias must be aligned to 16 bytes");
    ZI_REQUIRE(!bias || bias_dt == ZI_BF16 || bias_dt == ZI_F32, "attention_decode_fused: bias must be bfloat16 or float32");
    if (write_kv)
        ZI_REQUIRE(slots && cache_slots > 0 && cache_slots % page_size == 0,
                   "attention_decode_fused: cache of %lld slots is not a whole number of pages of %d",
                   (long long)cache_slots, page_size);
    DecProjection pj;
    pj.sums = sums; pj.splits = splits; pj.split_stride = split_stride; pj.ldp = ldp;
    pj.bias = bias; pj.bias_f32 = bias_dt == ZI_F32;
    pj.table = table; pj.rot = rot; pj.slots = slots; pj.cache_slots = cache_slots; pj.write_kv = write_kv;
    return dec_launch("attention_decode_fused", out, nullptr, dt, n_idx, 0, ldo, kcache, vcache, tok_index, tok_seq,
                      tok_pos, block_tables, max_pages, num_pages, nh, nkv, d, page_size, window, scale, max_chunks,
                      workspace, workspace_floats, &pj, stream);
}

// Heads whose merged attention one workgroup of the projection multiplies (one partial sum for each
// such group): as few as keep the partial sums at 16 or fewer.
extern "C" int zi_attention_decode_project_heads(int nh) { return nh <= 16 ? 1 : (nh + 15) / 16; }

// 1 when zi_attention_decode_project takes the shape, else 0 (then: merge into `out` and multiply).
extern "C" int zi_attention_decode_project_supported(int dt, int n, int nh, int d, int64_t ldw) {
    return dt == ZI_BF16 && n >= 1 && n <= 16 && nh >= 1 && d >= 16 && d <= 128 && d % 16 == 0 && ldw % 8 == 0 &&
           ldw >= (int64_t)nh * d;
}

// The output projection of n <= 16 decoded tokens read from the chunks that zi_attention_decode(_fused)
// left in `workspace` when it was called with out == nullptr for the same n, nh, d, tok_pos, window and
// max_chunks (and without tok_index): sums[s][t][:] = W[:, columns of the heads of group s] . attention
// of token t, float32, s < ceil(nh / zi_attention_decode_project_heads(nh)), rows of `sums` N long.
// W is [N, nh * d] bfloat16 with row stride ldw.
extern "C" int zi_attention_decode_project(float* sums, const float* workspace, int64_t workspace_floats, int n,
                                           const int32_t* tok_pos, int window, int max_chunks, const void* w, int dt,
                                           int64_t ldw, int N, int nh, int d, hipStream_t stream) {
    ZI_REQUIRE(zi_attention_decode_project_supported(dt, n, nh, d, ldw),
               "attention_decode_project: unsupported shape (bfloat16, 1..16 tokens, head_dim a multiple of 16 up to "
               "128, row stride a multiple of 8): dtype %d tokens %d heads %d head_dim %d stride %lld", dt, n, nh, d,
               (long long)ldw);
    ZI_REQUIRE(N >= 1 && window >= 0 && max_chunks >= 1 && max_chunks <= DEC_MAXC, "attention_decode_project: bad sizes");
    ZI_REQUIRE(sums && tok_pos && w && ((uintptr_t)sums % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "attention_decode_project: sums and weights must be aligned to 16 bytes");
    ZI_REQUIRE(workspace && workspace_floats >= zi_attention_decode_workspace(n, nh, d) && ((uintptr_t)workspace % 16) == 0,
               "attention_decode_project: workspace of %lld floats is too small or not aligned", (long long)workspace_floats);
    const float* po = workspace;
    const float* pml = workspace + (int64_t)n * nh * DEC_MAXC * d;
    const int hg = zi_attention_decode_project_heads(nh);
    const dim3 grid((N + DPJ_ROWS - 1) / DPJ_ROWS, (nh + hg - 1) / hg);
    ZI_REQUIRE(grid.y <= 65535, "attention_decode_project: too many heads");
#define ZI_DPJ(DD)                                                                                                    \
    attention_decode_project_kernel<DD><<<grid, 256, 0, stream>>>(sums, po, pml, tok_pos, n, nh, window, max_chunks,   \
                                                                  (const zi_bf16*)w, ldw, N, hg)
    switch (d) {
        case 16: ZI_DPJ(16); break;
        case 32: ZI_DPJ(32); break;
        case 48: ZI_DPJ(48); break;
        case 64: ZI_DPJ(64); break;
        case 80: ZI_DPJ(80); break;
        case 96: ZI_DPJ(96); break;
        case 112: ZI_DPJ(112); break;
        default: ZI_DPJ(128); break;
    }
#undef ZI_DPJ
    return zi_check_launch("attention_decode_project");
}
