// The index arithmetic of the paged cache, shared by the HIP kernels and by a host build.
//
// Everything that turns (sequence, position) into a place in the cache pool, cuts a token's keys into
// chunks, or sizes and indexes a workspace lives here as small inline functions without side effects.
// The kernels call them; csrc/host/paging_model.cpp, compiled with the host compiler alone, calls the same
// functions from loops that mirror the kernels' launches and checks every index against the bounds of
// what it indexes, so that an off-by-one in a block table walk shows on the CPU, without a GPU
// (reference for what the arithmetic must achieve: the cache walk of
// src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:15-72 and its callers :106-162).
//
// Cache layout of one layer: keys [page][kv_head][slot_in_page][head_dim], values transposed
// [page][kv_head][head_dim][slot_in_page].  A token's slot s lives in page s / page_size at offset
// s % page_size; a sequence's logical page i (positions i * page_size ...) is block_table[i], -1 when
// none is held.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define ZI_HD __host__ __device__ __forceinline__
#else
#define ZI_HD inline
#endif

// ---- places in the pool --------------------------------------------------------------------------
ZI_HD int64_t zi_key_offset(int64_t page, int kv_head, int slot_in_page, int nkv, int ps, int d) {
    return ((page * nkv + kv_head) * ps + slot_in_page) * d;          // + dim
}
ZI_HD int64_t zi_value_offset(int64_t page, int kv_head, int dim, int slot_in_page, int nkv, int ps, int d) {
    return ((page * nkv + kv_head) * d + dim) * ps + slot_in_page;
}
// Elements one layer's key (or value) pool holds.
ZI_HD int64_t zi_pool_elements(int64_t num_pages, int nkv, int ps, int d) { return num_pages * nkv * ps * d; }

// Where a token's new key and value go: nothing when the slot is negative (padding) or outside the pool.
struct ZiSlotPlace {
    int ok;
    int64_t page;
    int off;
};
ZI_HD ZiSlotPlace zi_slot_place(int slot, int64_t cache_slots, int ps) {
    ZiSlotPlace s;
    s.ok = slot >= 0 && slot < cache_slots;
    s.page = s.ok ? slot / ps : 0;
    s.off = s.ok ? slot % ps : 0;
    return s;
}

// A page id read from a block table, made safe to address with: ids outside the pool (-1: not held, a
// window has passed it, or the row belongs to no request) read page 0, and what is read is masked.
ZI_HD int zi_page_or_zero(int page_id, int num_pages) { return (unsigned)page_id < (unsigned)num_pages ? page_id : 0; }

// Which entry of a sequence's block table holds key `key`, and where in the page, with the key clamped to
// `last` (so that keys past what the sequence holds address something that exists) and the entry to the
// table's width.  ps_shift = log2(ps) for powers of two, -1 otherwise.
struct ZiTablePlace {
    int index;      // into the block table row
    int slot;       // within the page
};
ZI_HD ZiTablePlace zi_table_place(int key, int last, int ps, int ps_shift, int pi_last) {
    const int kc = key < last ? key : last;
    const int pi = ps_shift >= 0 ? kc >> ps_shift : kc / ps;
    ZiTablePlace t;
    t.slot = kc - pi * ps;
    t.index = pi < pi_last ? pi : pi_last;
    return t;
}

// ---- decode attention: the cut of one token's keys -----------------------------------------------
#define ZI_DEC_MAXC 64       // most chunks of one token
#define ZI_DEC_CHUNK 256     // keys of the smallest chunk
#define ZI_DEC_WAVES 4
#define ZI_DEC_BLOCK 64      // keys a wavefront handles at a time

// A token at position p sees keys [lo, p] (lo = 0, or p - window + 1).  That range, widened down to a
// multiple of 8, is cut into `count` <= 64 chunks of `len` keys (256, or 512, 1024, ... for more than 16,384
// keys); chunk c holds keys [lo_al + c * len, lo_al + (c + 1) * len).
struct DecSplit {
    int lo, lo_al, len, count;
};
ZI_HD DecSplit dec_split(int p, int window) {
    DecSplit s;
    s.lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    s.lo_al = s.lo & ~7;
    const int nk = p - s.lo_al + 1;
    s.len = ZI_DEC_CHUNK;
    while (nk > s.len * ZI_DEC_MAXC) s.len *= 2;
    s.count = (nk + s.len - 1) / s.len;
    return s;
}
// The keys wavefront `wave` of chunk `chunk` walks: [begin, end), in blocks of ZI_DEC_BLOCK from begin.
ZI_HD void zi_dec_wave_keys(const DecSplit& sp, int chunk, int wave, int p, int* begin, int* end) {
    const int quarter = sp.len / ZI_DEC_WAVES;
    *begin = sp.lo_al + chunk * sp.len + wave * quarter;
    *end = (*begin + quarter < p + 1) ? *begin + quarter : p + 1;
}
// The key that row r of score tile tt of the block at `base` holds (the permuted order that makes a lane's
// eight probabilities eight consecutive keys), and the first of the eight keys lane group j reads of the
// block's value half b.
ZI_HD int zi_dec_tile_key(int base, int tt, int r) { return base + (tt / 2) * 32 + (r / 4) * 8 + (tt % 2) * 4 + (r % 4); }
ZI_HD int zi_dec_value_key0(int base, int b, int j) { return base + b * 32 + j * 8; }
// The key whose score is element e of tile tt in lane group j (the same permutation seen from the scores).
ZI_HD int zi_dec_score_key(int base, int tt, int j, int e) { return base + (tt / 2) * 32 + j * 8 + (tt % 2) * 4 + e; }
// Floats of workspace for the chunk partials of n tokens, and the slot of one (token, head, chunk) in it:
// outputs at slot * d, (maximum, sum) at n * nh * 64 * d + slot * 2.
ZI_HD int64_t zi_dec_workspace_floats(int n, int nh, int d) { return (int64_t)n * nh * ZI_DEC_MAXC * (d + 2); }
ZI_HD int64_t zi_dec_part_slot(int token_index, int nh, int head, int chunk) {
    return ((int64_t)token_index * nh + head) * ZI_DEC_MAXC + chunk;
}

// ---- prompt attention: the cut of one tile's keys ---------------------------------------------------
#define ZI_PF_BM 64          // queries of a tile
#define ZI_PF_BS 128         // keys of a block
#define ZI_PF_CHUNK 2048     // keys one workgroup walks at most: the cut of launches over few keys
#define ZI_PF_CHUNK_LONG 16384      // the cut of launches whose queries see more than ZI_PF_LONG_FROM keys and that have
#define ZI_PF_LONG_FROM 6144        // ZI_PF_LONG_GROUPS_PER_CU workgroups (tiles x heads) a compute unit without any cut: those
#define ZI_PF_LONG_GROUPS_PER_CU 3  // fill the chip as they are, and every cut costs a merge (768 on 256 units)
#define ZI_PF_MAXC 64        // most cuts of one tile

// The cut of a launch of `groups` tiles x heads none of whose queries sees more than max_keys keys.
ZI_HD int zi_pf_chunk_for(int max_keys, int groups, int compute_units = 256) {
    return (max_keys > ZI_PF_LONG_FROM && groups >= ZI_PF_LONG_GROUPS_PER_CU * compute_units) ? ZI_PF_CHUNK_LONG : ZI_PF_CHUNK;
}

// A tile of `count` queries whose first sits at position pos0 sees keys [lo_tile, kmax].  Its walk starts at
// kb_first (a multiple of the block) and is cut at absolute multiples of `chunk` into nc cuts, the first
// being cut c0 of the sequence; cut number `cut` (0-based within the tile) walks [kb_begin, khi].
struct PfCut {
    int kmax, lo_tile, kb_first, c0, nc;
    int live;              // this cut exists
    int kb_begin, khi;
};
ZI_HD PfCut zi_pf_cut(int pos0, int count, int window, int cut, int chunk = ZI_PF_CHUNK) {
    PfCut t;
    t.kmax = pos0 + count - 1;
    t.lo_tile = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    t.kb_first = (t.lo_tile / ZI_PF_BS) * ZI_PF_BS;
    t.c0 = t.kb_first / chunk;
    t.nc = t.kmax / chunk - t.c0 + 1;
    const int c = t.c0 + cut;
    t.live = c * chunk <= t.kmax;
    t.kb_begin = (c * chunk > t.kb_first) ? c * chunk : t.kb_first;
    t.khi = ((c + 1) * chunk - 1 < t.kmax) ? (c + 1) * chunk - 1 : t.kmax;
    return t;
}
ZI_HD int64_t zi_pf_workspace_floats(int rows, int nh, int d, int max_chunks) {
    return max_chunks > 1 ? (int64_t)rows * nh * max_chunks * (d + 2) : 0;
}
ZI_HD int64_t zi_pf_part_slot(int64_t row, int nh, int head, int max_chunks, int cut) {
    return (row * nh + head) * max_chunks + cut;
}
