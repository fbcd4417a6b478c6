// A host-side model of how the attention and cache-store kernels walk the paged cache.
//
// Compiled with the host compiler alone (no GPU, no HIP).  For a launch given as the kernels get it (block
// tables, positions, slots, sizes) it runs the same loops over workgroups, wavefronts and lanes as the
// kernels do, with the index arithmetic of zi_paging.h, which the kernels call too, and checks what
// cannot be seen from a result that happens to be right: every index stays inside what it indexes (block
// table rows, the cache pool, the workspace), every key a query may see is read exactly once and from the
// page the sequence holds for it, nothing that is not held is read as if it were, no two writers share a
// place.  Tests feed it block tables from the cache manager under random traffic, with the -1 entries,
// the empty rows and the slot -1 tokens of padded steps (reference for the walk being modelled:
// src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:15-72, :106-162).
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <set>
#include <vector>

#include "../zi_paging.h"

static char pm_error[1024] = "";
extern "C" const char* pm_last_error() { return pm_error; }
static int pm_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(pm_error, sizeof(pm_error), fmt, ap);
    va_end(ap);
    return 1;
}
#define PM_CHECK(cond, ...)                       \
    do {                                          \
        if (!(cond)) return pm_fail(__VA_ARGS__); \
    } while (0)

static int shift_of(int ps) { return (ps & (ps - 1)) == 0 ? __builtin_ctz(ps) : -1; }

// The decode attention launch (attention_decode_kernel, both variants): grid (n_idx, nkv, max_chunks), four
// wavefronts.  `slots` non-null: the variant that also stores each token's new key and value; a token with a
// negative slot there is padding (an entry of no request: an empty block table, a result nobody reads), for
// which only the bounds are checked.
// stats[0] = (token, kv head, key) triples read as visible, stats[1] = workspace slots written,
// stats[2] = tokens that got NaN because the launch covers fewer chunks than they have.
extern "C" int pm_check_decode(int n_idx, const int* tok_index, const int* tok_seq, const int* tok_pos,
                               const int* block_tables, int n_seqs, int max_pages, int num_pages, int nh, int nkv, int d,
                               int ps, int window, int max_chunks, int64_t workspace_floats, int leave_parts,
                               const int* slots, int64_t cache_slots, int64_t* stats) {
    PM_CHECK(nkv > 0 && nh % nkv == 0 && ps > 0 && ps % 8 == 0 && max_pages > 0 && num_pages > 0, "decode: bad sizes");
    const int G = nh / nkv, ps_shift = shift_of(ps), pi_last = max_pages - 1;
    const int64_t pool = zi_pool_elements(num_pages, nkv, ps, d);
    const int64_t ml_base = (int64_t)n_idx * nh * ZI_DEC_MAXC * d;
    std::set<int64_t> written;
    stats[0] = stats[1] = stats[2] = 0;
    for (int x = 0; x < n_idx; ++x) {
        const int t = tok_index ? tok_index[x] : x;
        const int p = tok_pos[t];
        PM_CHECK(p >= 0, "decode: token %d has position %d", t, p);
        const DecSplit sp = dec_split(p, window);
        if (sp.count > max_chunks) {      // the kernel writes NaN and touches nothing else
            ++stats[2];
            continue;
        }
        const int row = tok_seq ? tok_seq[t] : t;
        PM_CHECK(row >= 0 && row < n_seqs, "decode: token %d names block table row %d of %d", t, row, n_seqs);
        const int* bt = block_tables + (int64_t)row * max_pages;
        const int p8 = p & ~7;
        const bool padding = slots && slots[t] < 0;
        for (int kvh = 0; kvh < nkv; ++kvh) {
            std::vector<int> seen(p + 1, 0);
            for (int chunk = 0; chunk < sp.count; ++chunk) {
                for (int wave = 0; wave < ZI_DEC_WAVES; ++wave) {
                    int k_begin, k_end;
                    zi_dec_wave_keys(sp, chunk, wave, p, &k_begin, &k_end);
                    for (int base = k_begin; base < k_end; base += ZI_DEC_BLOCK) {
                        for (int tt = 0; tt < 4; ++tt)
                            for (int r = 0; r < 16; ++r) {
                                const int key = zi_dec_tile_key(base, tt, r);
                                // the lane that holds the score of this key masks by the same key
                                PM_CHECK(zi_dec_score_key(base, tt, r / 4, r % 4) == key,
                                         "decode: tile row %d of tile %d is key %d for the loads and %d for the mask", r, tt,
                                         key, zi_dec_score_key(base, tt, r / 4, r % 4));
                                const ZiTablePlace at = zi_table_place(key, p, ps, ps_shift, pi_last);
                                PM_CHECK(at.index >= 0 && at.index < max_pages && at.slot >= 0 && at.slot < ps,
                                         "decode: key %d of token %d reads block table entry %d (width %d), slot %d", key, t,
                                         at.index, max_pages, at.slot);
                                const int id = bt[at.index], page = zi_page_or_zero(id, num_pages);
                                const int64_t o = zi_key_offset(page, kvh, at.slot, nkv, ps, d);
                                PM_CHECK(o >= 0 && o + d <= pool, "decode: key %d of token %d is read at %lld of %lld", key, t,
                                         (long long)o, (long long)pool);
                                const bool visible = key >= sp.lo && key < k_end && key <= p;
                                if (!visible || padding) continue;
                                PM_CHECK(id >= 0 && id < num_pages, "decode: token %d sees key %d but its page entry is %d", t,
                                         key, id);
                                PM_CHECK(at.index == key / ps && at.slot == key % ps,
                                         "decode: key %d of token %d is read from entry %d slot %d", key, t, at.index, at.slot);
                                ++seen[key];
                            }
                        for (int b = 0; b < 2; ++b)
                            for (int j = 0; j < 4; ++j) {
                                const int key0 = zi_dec_value_key0(base, b, j);
                                const ZiTablePlace at = zi_table_place(key0, p8, ps, ps_shift, pi_last);
                                PM_CHECK(at.index >= 0 && at.index < max_pages && at.slot >= 0 && at.slot + 8 <= ps,
                                         "decode: values of keys %d.. of token %d: entry %d, slots %d..", key0, t, at.index,
                                         at.slot);
                                const int id = bt[at.index], page = zi_page_or_zero(id, num_pages);
                                for (int dim = 0; dim < d; dim += d > 1 ? d - 1 : 1) {      // first and last dim
                                    const int64_t o = zi_value_offset(page, kvh, dim, at.slot, nkv, ps, d);
                                    PM_CHECK(o >= 0 && o + 8 <= pool, "decode: values of key %d of token %d at %lld of %lld",
                                             key0, t, (long long)o, (long long)pool);
                                }
                                bool any = false;
                                for (int e = 0; e < 8; ++e) any = any || (key0 + e >= sp.lo && key0 + e < k_end && key0 + e <= p);
                                if (!any || padding) continue;
                                PM_CHECK(id >= 0 && id < num_pages && at.index == key0 / ps && at.slot == key0 % ps,
                                         "decode: token %d sees keys from %d on but reads their values from entry %d (page %d)",
                                         t, key0, at.index, id);
                            }
                    }
                }
                // what the chunk leaves behind
                if (sp.count > 1 || leave_parts)
                    for (int r = 0; r < G; ++r) {
                        const int64_t slot = zi_dec_part_slot(x, nh, kvh * G + r, chunk);
                        PM_CHECK(slot >= 0 && (slot + 1) * d <= ml_base && ml_base + slot * 2 + 1 < workspace_floats,
                                 "decode: chunk %d of token index %d head %d writes workspace slot %lld (workspace of %lld "
                                 "floats)", chunk, x, kvh * G + r, (long long)slot, (long long)workspace_floats);
                        PM_CHECK(written.insert(slot).second, "decode: workspace slot %lld is written twice", (long long)slot);
                        ++stats[1];
                    }
            }
            for (int key = 0; key <= p && !padding; ++key) {
                const int want = key >= sp.lo ? 1 : 0;
                PM_CHECK(seen[key] == want, "decode: token %d kv head %d reads key %d %d times, %d wanted (position %d, "
                         "window %d)", t, kvh, key, seen[key], want, p, window);
                stats[0] += seen[key];
            }
        }
        if (slots) {
            const ZiSlotPlace place = zi_slot_place(slots[t], cache_slots, ps);
            if (slots[t] >= 0) {
                PM_CHECK(place.ok, "decode: token %d stores to slot %d outside the pool of %lld", t, slots[t],
                         (long long)cache_slots);
                PM_CHECK(bt[p / ps] == place.page && p % ps == place.off,
                         "decode: token %d at position %d stores to page %lld offset %d, its table says page %d offset %d", t, p,
                         (long long)place.page, place.off, bt[p / ps], p % ps);
                for (int kvh = 0; kvh < nkv; ++kvh) {
                    PM_CHECK(zi_key_offset(place.page, kvh, place.off, nkv, ps, d) + d <= pool &&
                                 zi_value_offset(place.page, kvh, d - 1, place.off, nkv, ps, d) < pool,
                             "decode: token %d stores outside the pool", t);
                }
            }
        }
    }
    return 0;
}

// The prompt attention launch (attention_prefill kernels): grid (tiles * nh, cuts), eight wavefronts: four
// groups of tile / 4 queries (tile = 64 or 128 queries), each shared by two wavefronts that take alternate
// halves of every block of 128 keys; or (`alone`) four wavefronts, one a group, and blocks of 64 keys.
// stats[0] = (query, key) pairs covered, stats[1] = workspace slots written, stats[2] = tiles given NaN.
// `entry_real` (or null): the tokens of each entry that are its own; the rest are padding, whose queries'
// results nobody reads and whose keys are nowhere: they are checked for bounds only.
// The keys between the cuts of a tile, as the caller of the kernels chooses them for its launch
// (zi_pf_chunk_for): ZI_PF_CHUNK unless set otherwise.  Returns what it was.
static int pm_pf_chunk = ZI_PF_CHUNK;
extern "C" int pm_set_prefill_chunk(int chunk) {
    const int before = pm_pf_chunk;
    if (chunk == ZI_PF_CHUNK || chunk == ZI_PF_CHUNK_LONG) pm_pf_chunk = chunk;
    return before;
}
extern "C" int pm_prefill_chunk_for(int max_keys, int groups) { return zi_pf_chunk_for(max_keys, groups); }

extern "C" int pm_check_prefill(int num_tiles, const int* tile_entry, const int* tile_off, const int* entry_start,
                                const int* entry_len, const int* entry_past, const int* entry_real, int num_entries,
                                const int* block_tables,
                                int max_pages, int num_pages, int nh, int nkv, int d, int ps, int window, int rows,
                                int max_chunks, int64_t workspace_floats, int tile_queries, int alone, int64_t* stats) {
    PM_CHECK(nkv > 0 && nh % nkv == 0 && ps >= 8 && (ps & (ps - 1)) == 0 && max_pages > 0, "prefill: bad sizes");
    PM_CHECK(tile_queries == ZI_PF_BM || tile_queries == 2 * ZI_PF_BM, "prefill: tiles of %d queries", tile_queries);
    const int BM = tile_queries, QR = tile_queries / 4;
    const int KH = alone ? 1 : 2, BS = 64 * KH;      // wavefronts that share a query group, keys of a block
    const int ps_shift = shift_of(ps), pi_last = max_pages - 1;
    const int64_t pool = zi_pool_elements(num_pages, nkv, ps, d);
    const int64_t ml_base = (int64_t)rows * nh * max_chunks * d;
    PM_CHECK(workspace_floats >= zi_pf_workspace_floats(rows, nh, d, max_chunks), "prefill: workspace of %lld floats, %lld "
             "needed", (long long)workspace_floats, (long long)zi_pf_workspace_floats(rows, nh, d, max_chunks));
    std::set<int64_t> written;
    stats[0] = stats[1] = stats[2] = 0;
    for (int tile = 0; tile < num_tiles; ++tile) {
        const int e = tile_entry[tile], off = tile_off[tile];
        PM_CHECK(e >= 0 && e < num_entries, "prefill: tile %d names entry %d of %d", tile, e, num_entries);
        const int start = entry_start[e], len = entry_len[e], past = entry_past[e];
        PM_CHECK(off >= 0 && off < len && off % BM == 0, "prefill: tile %d starts at %d of %d tokens", tile, off, len);
        const int count = (len - off < BM) ? len - off : BM;
        const int real = entry_real ? entry_real[e] - off : count;      // queries of the tile that are real
        PM_CHECK(start + off + count <= rows, "prefill: tile %d covers rows up to %d of %d", tile, start + off + count, rows);
        const int* bt = block_tables + (int64_t)e * max_pages;
        const int pos0 = past + off;
        const PfCut whole = zi_pf_cut(pos0, count, window, 0, pm_pf_chunk);
        if (whole.nc > max_chunks) {
            ++stats[2];
            continue;
        }
        // pairs[q][key - lo_tile]: times the (query, key) pair was covered
        std::vector<std::vector<int>> pairs(count, std::vector<int>(whole.kmax - whole.lo_tile + 1, 0));
        for (int cut_i = 0; cut_i < whole.nc; ++cut_i) {
            const PfCut cut = zi_pf_cut(pos0, count, window, cut_i, pm_pf_chunk);
            PM_CHECK(cut.live, "prefill: tile %d has %d cuts but cut %d does not exist", tile, whole.nc, cut_i);
            PM_CHECK(cut.kb_begin % ZI_PF_BS == 0 && cut.kb_begin <= cut.khi && cut.khi - cut.kb_begin < pm_pf_chunk,
                     "prefill: cut %d of tile %d walks [%d, %d]", cut_i, tile, cut.kb_begin, cut.khi);
            // the block table entries the workgroup copies to LDS
            const int pi_first = cut.kb_begin >> ps_shift, n_entries = (cut.khi >> ps_shift) - pi_first + 1;
            PM_CHECK(n_entries <= ZI_PF_CHUNK_LONG / 8 + 8, "prefill: %d block table entries for one cut",
                     n_entries);
            for (int kb = cut.kb_begin; kb <= cut.khi; kb += BS) {
                for (int k = 0; k < BS; ++k) {
                    const int key = kb + k, kc = key <= cut.khi ? key : cut.khi;
                    const int idx = (kc >> ps_shift) - pi_first;
                    PM_CHECK(idx >= 0 && idx < n_entries, "prefill: key %d reads staged table entry %d of %d", key, idx,
                             n_entries);
                    const int ti = pi_first + idx < pi_last ? pi_first + idx : pi_last;
                    const int id = bt[ti], page = zi_page_or_zero(id, num_pages);
                    const int64_t o = zi_key_offset(page, 0, kc & (ps - 1), nkv, ps, d);
                    PM_CHECK(o >= 0 && zi_key_offset(page, nkv - 1, kc & (ps - 1), nkv, ps, d) + d <= pool,
                             "prefill: key %d is read outside the pool", key);
                    bool anyone = false;
                    for (int q = 0; q < count && q < real; ++q) {
                        const int qpos = pos0 + q;
                        if (key <= qpos && (window <= 0 || key > qpos - window)) anyone = true;
                    }
                    if (anyone && key <= cut.khi)
                        PM_CHECK(id >= 0 && id < num_pages && ti == key / ps,
                                 "prefill: a query of tile %d sees key %d but its page entry (%d) is %d", tile, key, ti, id);
                }
                // which wavefronts work on which half of the block, and the pairs they cover
                for (int qs = 0; qs < 4; ++qs) {
                    if (qs * QR >= count) continue;
                    const int wave_last = pos0 + ((qs * QR + QR - 1 < count) ? qs * QR + QR - 1 : count - 1);
                    const int wave_lo = (window > 0 && pos0 + qs * QR - window + 1 > 0) ? pos0 + qs * QR - window + 1 : 0;
                    for (int kh = 0; kh < KH; ++kh) {
                        const int kb2 = kb + kh * 64;
                        if (!(kb2 <= wave_last && kb2 + 64 > wave_lo)) continue;
                        for (int r = 0; r < QR && qs * QR + r < count; ++r) {
                            const int q = qs * QR + r, qpos = pos0 + q;
                            for (int k = 0; k < 64; ++k) {
                                const int key = kb2 + k;
                                if (key <= qpos && (window <= 0 || key > qpos - window)) {
                                    PM_CHECK(key >= whole.lo_tile && key <= whole.kmax, "prefill: pair (%d, %d) outside the tile",
                                             qpos, key);
                                    ++pairs[q][key - whole.lo_tile];
                                }
                            }
                        }
                    }
                }
            }
            if (whole.nc > 1)
                for (int q = 0; q < count; ++q)
                    for (int h = 0; h < nh; ++h) {
                        const int64_t slot = zi_pf_part_slot(start + off + q, nh, h, max_chunks, cut_i);
                        PM_CHECK(slot >= 0 && (slot + 1) * d <= ml_base && ml_base + slot * 2 + 1 < workspace_floats,
                                 "prefill: workspace slot %lld outside %lld floats", (long long)slot, (long long)workspace_floats);
                        PM_CHECK(written.insert(slot).second, "prefill: workspace slot %lld is written twice", (long long)slot);
                        ++stats[1];
                    }
        }
        for (int q = 0; q < count; ++q) {
            const int qpos = pos0 + q;
            for (int key = whole.lo_tile; key <= whole.kmax; ++key) {
                const int want = (key <= qpos && (window <= 0 || key > qpos - window)) ? 1 : 0;
                PM_CHECK(pairs[q][key - whole.lo_tile] == want, "prefill: query at %d and key %d are covered %d times, %d wanted",
                         qpos, key, pairs[q][key - whole.lo_tile], want);
                stats[0] += want;
            }
        }
    }
    return 0;
}

// The cache store of the rotary kernels: token t's key and value go to slot slots[t]; negative slots are
// padding.  No place outside the pool, no place written twice.  stats[0] = tokens stored.
extern "C" int pm_check_store(int n, const int* slots, int64_t cache_slots, int num_pages, int nkv, int d, int ps,
                              int64_t* stats) {
    const int64_t pool = zi_pool_elements(num_pages, nkv, ps, d);
    PM_CHECK(cache_slots == (int64_t)num_pages * ps, "store: %lld slots are not %d pages of %d", (long long)cache_slots,
             num_pages, ps);
    std::set<int64_t> keys, values;
    stats[0] = 0;
    for (int t = 0; t < n; ++t) {
        const ZiSlotPlace place = zi_slot_place(slots[t], cache_slots, ps);
        if (slots[t] < 0) {
            PM_CHECK(!place.ok, "store: the negative slot of token %d would be written", t);
            continue;
        }
        PM_CHECK(place.ok, "store: slot %d of token %d lies outside the pool of %lld", slots[t], t, (long long)cache_slots);
        for (int h = 0; h < nkv; ++h) {
            const int64_t ko = zi_key_offset(place.page, h, place.off, nkv, ps, d);
            PM_CHECK(ko >= 0 && ko + d <= pool, "store: key of token %d at %lld of %lld", t, (long long)ko, (long long)pool);
            PM_CHECK(keys.insert(ko).second, "store: two tokens store their key at %lld", (long long)ko);
            for (int dim = 0; dim < d; ++dim) {
                const int64_t vo = zi_value_offset(place.page, h, dim, place.off, nkv, ps, d);
                PM_CHECK(vo >= 0 && vo < pool, "store: value of token %d at %lld of %lld", t, (long long)vo, (long long)pool);
                PM_CHECK(values.insert(vo).second, "store: two tokens store a value at %lld", (long long)vo);
            }
        }
        ++stats[0];
    }
    return 0;
}

// The sizes the kernels' hosts ask for, for the tests to hold against the launches above.
extern "C" int64_t pm_decode_workspace(int n, int nh, int d) { return zi_dec_workspace_floats(n, nh, d); }
extern "C" int64_t pm_prefill_workspace(int rows, int nh, int d, int max_chunks) { return zi_pf_workspace_floats(rows, nh, d, max_chunks); }
extern "C" int pm_decode_chunks(int keys) {
    if (keys < 1) keys = 1;
    if (keys + 7 > ZI_DEC_CHUNK * ZI_DEC_MAXC) return ZI_DEC_MAXC;
    return dec_split(keys - 1 + 7, 0).count;
}
extern "C" int pm_prefill_chunks(int keys) { return ((keys < 1 ? 1 : keys) + pm_pf_chunk - 1) / pm_pf_chunk; }
