// One decoder layer for up to 16 single decoded tokens in ONE launch: a grid of resident workgroups (one a
// compute unit) walks the layer's phases and meets at barriers of its own between them.
//
//   norm -> q/k/v product (+bias, rotation, cache store)  | barrier 1
//   attention over the cached keys, chunk by chunk; the last workgroup to finish a (token, kv head)
//   merges its chunks with the token's own new key and value                         | barrier 2
//   output product + residual add (-> second residual buffer, normed-gain copy, sums of squares) | barrier 3
//   gate/up product + SwiGLU                                                          | barrier 4
//   down product, cut along k; the last workgroup to finish 8 output columns adds the cuts and the residual
//
// Why one launch: at this size a layer is seven dependent launches that move little and wait (a kernel of a
// graph that depends on the one before it takes 2.6 us at least).  Here the weights of the next phase, which
// depend on nothing, are requested BEFORE a workgroup waits at a barrier, so the memory pipe stays full
// while the few kilobytes of activations make their way round.
//
// What is exchanged between workgroups inside the launch (queries, attention chunks, the residual after the
// attention, the activation) is written with write-through stores (system scope) and read with loads of
// agent scope that go past the caches of the reader's XCD, each buffer written once per launch before the
// barrier that precedes its reads: no fence, so no write-back or invalidation of an L2 that is busy
// streaming weights.  Barriers are a two-level tree of counters (groups of 32 workgroups); every wait is
// bounded: after `spin_limit` polls a workgroup sets the abort word and the host's error flag, and every
// workgroup leaves at its next wait.
//
// Matrix products: a unit is 8 weight rows; the 8 wavefronts of a workgroup cut the unit's k range between
// them, in steps of 64: lanes 0-7 of the 16 operand rows hold the 8 rows at k, lanes 8-15 the same rows at
// k + 32, so one load instruction takes 8 rows x 128 bytes (whole cache lines) and two matrix instructions
// (v_mfma_f32_16x16x32_bf16, the up to 16 tokens as the other operand, from LDS) use it; the two halves and
// the 8 wavefronts are added in a fixed order through LDS.  The order of a row's sums depends on the
// matrix's shape and the number of workgroups only.
// (reference for the layer: src/frontend/models/transformer_forward.cpp:63-149; for the parts' formulas see
// norm.hip, rope_kv.hip, attention_decode.hip, gemm_mid.hip, elementwise.hip.)
#include "zi_common.h"
#include "zi_api.h"
#include "zi_paging.h"
#include <mutex>

typedef __attribute__((ext_vector_type(8))) __bf16 dl_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short dl_s16x4_t;
typedef __attribute__((ext_vector_type(4))) float dl_f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned dl_u32x4_t;

#define DL_WAVES 8
#define DL_THREADS (DL_WAVES * ZI_WAVE)
#define DL_UB 4            // units whose wavefront sums lie in LDS before they are added (a turn of the ring)
#define DL_MAX_DPW 10      // most steps of 64 of k one wavefront takes of a unit: k ranges up to 5120
#define DL_MAX_TOKENS 16
#define DL_GROUP 32        // workgroups of one barrier group
#define DL_MAXC 64         // most chunks of one token's keys
#define DL_BARRIERS 4      // per launch

// words of the synchronisation state (each counter or flag that is polled has a 256-byte line of its own)
#define DL_LINE 64
#define DL_W_BASE 0                          // the epoch the launch starts from
#define DL_W_TOP (1 * DL_LINE)
#define DL_W_ABORT (2 * DL_LINE)
#define DL_W_GROUP (8 * DL_LINE)             // 64 lines
#define DL_W_RELEASE (72 * DL_LINE)          // 64 lines
#define DL_W_TASK (136 * DL_LINE)            // one word per (token, kv head): DL_MAX_TOKENS * 256
#define DL_W_UNIT (DL_W_TASK + DL_MAX_TOKENS * 256)      // one word per 8 output columns of the down product
#define DL_SYNC_WORDS (DL_W_UNIT + 4096)

#define DL_ROWS_PLAIN 0
#define DL_ROWS_ROTARY 1
#define DL_ROWS_SWIGLU 2

// Built with -DDL_TIMING, workgroups 0..255 leave the clock (100 MHz) at up to 32 places of a launch in the
// words after the synchronisation state: a probe for whoever tunes the kernel, not part of the product build.
#ifdef DL_TIMING
#define DL_STAMP(i)                                                                                      \
    do {                                                                                                 \
        const int stamp_index = (i);                                                                     \
        if (threadIdx.x == 0 && blockIdx.x < 256 && stamp_index >= 0 && stamp_index < 32)                \
            reinterpret_cast<uint64_t*>(P.sync + DL_SYNC_WORDS)[blockIdx.x * 32 + stamp_index] = wall_clock64(); \
    } while (0)
// the shader clock's count at slot i
#define DL_CYCLES(i)                                                                                     \
    do {                                                                                                 \
        if (threadIdx.x == 0 && blockIdx.x < 256)                                                        \
            reinterpret_cast<uint64_t*>(P.sync + DL_SYNC_WORDS)[blockIdx.x * 32 + (i)] = clock64();      \
    } while (0)
// a stamp by lane 0 of every wavefront, at slot i + wavefront
#define DL_WAVE_STAMP(i, cond)                                                                           \
    do {                                                                                                 \
        if ((threadIdx.x & 63) == 0 && blockIdx.x < 256 && (cond))                                       \
            reinterpret_cast<uint64_t*>(P.sync + DL_SYNC_WORDS)[blockIdx.x * 32 + (i) + (threadIdx.x >> 6)] = wall_clock64(); \
    } while (0)
#else
#define DL_STAMP(i)
#define DL_CYCLES(i)
#define DL_WAVE_STAMP(i, cond)
#endif

union dl_pack {
    dl_u32x4_t u;
    dl_bf16x8_t b;
};

// ---- exchange between workgroups ---------------------------------------------------------------------
__device__ __forceinline__ void dl_put32(void* p, uint32_t v) {
    __hip_atomic_store(reinterpret_cast<uint32_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void dl_putf(float* p, float v) { dl_put32(p, __float_as_uint(v)); }
__device__ __forceinline__ uint32_t dl_get32(const void* p) {
    return __hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t dl_get64(const void* p) {
    return __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float dl_getf(const float* p) { return __uint_as_float(dl_get32(p)); }
__device__ __forceinline__ uint32_t dl_add(uint32_t* p, uint32_t v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// every store this wavefront has issued has been acknowledged
__device__ __forceinline__ void dl_stores_done() { __builtin_amdgcn_s_waitcnt(0); }

__device__ __forceinline__ dl_u32x4_t dl_keep(dl_u32x4_t v, bool keep) { return v & (0u - (unsigned)keep); }

// ---- parameters ------------------------------------------------------------------------------------------
struct DlParams {
    int n, H, I, nh, nkv, d, G, rot, ps, window, max_pages, num_pages;
    int64_t cache_slots;
    float eps1, eps2, w_offset, scale;
    float* resid;                 // [n][H] float32, in and out
    const void *norm1, *norm2;    // gains [H]
    int norm_f32;
    const zi_bf16 *wqkv, *wo, *wgu, *wd;
    int64_t ld_qkv, ld_o, ld_gu, ld_d;
    const void* bias;             // [Qd + 2 KVd] or null
    int bias_f32;
    const float* table;           // [n][rot/2][2] or null
    const int32_t *slots, *pos, *bt;
    zi_bf16 *kcache, *vcache;
    // exchange buffers (inside the workspace)
    zi_bf16 *qbuf, *kvbuf, *attn, *x2, *hbuf;
    float *resid2, *ssq, *part_o, *part_ml, *dsum;
    uint32_t* sync;
    int* err;                     // host memory the device can write: set when a wait ran out
    int nb, max_chunks, S, lds_xs_elems;
    int spin_limit;
};

struct DlRows {
    int mode, d8, rot8, half, qk_heads;
};
__device__ __forceinline__ int dl_row(const DlRows& R, int unit, int r7) {
    if (R.mode == DL_ROWS_SWIGLU) return (unit >> 1) * 16 + (unit & 1) * 4 + (r7 & 3) + (r7 >> 2) * 8;
    if (R.mode == DL_ROWS_ROTARY) {
        const int hh = unit / R.d8, ui = unit - hh * R.d8;
        if (hh < R.qk_heads && ui < R.rot8) return hh * R.d8 * 8 + ui * 4 + (r7 & 3) + (r7 >> 2) * R.half;
    }
    return unit * 8 + r7;
}

// A workgroup's share of one matrix: units unit0 + i * ustride (i < nunits) over the k range of `dsn` steps of
// 64 from step ds0; wavefront w takes the steps w, w + 8, ... of every unit.  What a lane adds to the address
// of a (unit, step), which is the same for every lane of the wavefront, is worked out once: a unit costs a few
// scalar instructions and one load with a 32-bit lane offset per step.
struct DlStream {
    const zi_bf16* w;
    int64_t ldw;
    int N, K;
    DlRows rows;
    int unit0, ustride, nunits;
    int ds0, dsn, dpw;           // wavefront w takes the steps w, w + 8, ... of the range: at most dpw of them
    int ds_tail;                 // the step (of the whole k) that crosses K, or -1
    // per lane: bytes from the first row of a unit at a step to this lane's 16 bytes; `alt` for the units of a
    // rotary stream whose rows are not paired; `tail` at the step that crosses K (clamped into the row)
    uint32_t off, off_alt, off_tail, off_tail_alt;
    uint32_t tail_keep;          // all ones when this lane's 8 values of the step that crosses K lie within K
    int64_t idle_at;             // bytes into the matrix of 16 bytes a wavefront reads when it has nothing to request
};

__device__ __forceinline__ DlStream dl_stream(const zi_bf16* w, int64_t ldw, int N, int K, DlRows rows, int unit0,
                                              int ustride, int nunits, int ds0, int dsn, int r7, int half, int kg) {
    DlStream s;
    s.w = w; s.ldw = ldw; s.N = N; s.K = K; s.rows = rows;
    s.unit0 = unit0; s.ustride = ustride; s.nunits = nunits > 0 ? nunits : 0;
    s.ds0 = ds0; s.dsn = dsn;
    s.dpw = (dsn + DL_WAVES - 1) / DL_WAVES;
    s.ds_tail = (K & 63) ? K >> 6 : -1;
    const int paired = (r7 & 3) + (r7 >> 2) * (rows.mode == DL_ROWS_SWIGLU ? 8 : rows.half);
    const int row_main = rows.mode == DL_ROWS_PLAIN ? r7 : paired;
    const int lane_k = half * 32 + kg * 8;
    int tail_k = (K >> 6) * 64 + lane_k;
    s.tail_keep = tail_k < K ? ~0u : 0u;
    tail_k = (tail_k < K ? tail_k : K - 8) - (K >> 6) * 64;
    s.off = (uint32_t)(row_main * ldw + lane_k) * 2u;
    s.off_alt = (uint32_t)(r7 * ldw + lane_k) * 2u;
    s.off_tail = (uint32_t)(row_main * ldw + tail_k) * 2u;
    s.off_tail_alt = (uint32_t)(r7 * ldw + tail_k) * 2u;
    {
        const int64_t bytes = ((int64_t)(N - 1) * ldw + K) * 2;
        int64_t at = ((int64_t)blockIdx.x * DL_WAVES + (threadIdx.x >> 6)) * 128;
        if (at > bytes - 16) at = (at % (bytes - 15)) & ~(int64_t)15;
        s.idle_at = __builtin_amdgcn_readfirstlane((int)(at >> 4)) * (int64_t)16;
    }
    return s;
}

// The first row of unit `unit` of a stream, and whether its rows follow the plain pattern where the stream's
// other units are paired (a rotary stream's heads beyond the rotated dims, and its value heads).
__device__ __forceinline__ int dl_unit_row(const DlRows& R, int unit, bool* alt) {
    *alt = false;
    if (R.mode == DL_ROWS_SWIGLU) return (unit >> 1) * 16 + (unit & 1) * 4;
    if (R.mode == DL_ROWS_ROTARY) {
        const int hh = unit / R.d8, ui = unit - hh * R.d8;
        if (hh < R.qk_heads && ui < R.rot8) return hh * R.d8 * 8 + ui * 4;
        *alt = true;
    }
    return unit * 8;
}

// The contiguous share of `total` things that workgroup `wg` of `G` takes: [first, first + count).
__device__ __forceinline__ void dl_share(int total, int wg, int G, int* first, int* count) {
    const int lo = (int)(((int64_t)total * wg) / G), hi = (int)(((int64_t)total * (wg + 1)) / G);
    *first = lo;
    *count = hi - lo;
}

// Request this wavefront's steps of unit `ul` of the stream.  `wave` must be known to the compiler as the same
// for every lane (readfirstlane).  A wavefront with fewer steps than the stream's most repeats its last (or the
// range's last), which the cache serves; what it must not count is zeroed where it is used.  A unit past the
// stream's end is requested all the same, as one 16-byte piece that every lane reads: requests made under
// conditions would leave the compiler unable to count how many loads may stay in flight at each use, and it
// would wait for all of them.
template <int DPW>
__device__ __forceinline__ void dl_issue_unit(const DlStream& st, int ul, dl_u32x4_t (&buf)[DPW], int wave) {
    const bool real = ul < st.nunits;
    bool alt;
#ifdef DL_SAME_UNIT      // a probe: every unit reads the stream's first, which the cache then serves
    const int64_t urow = dl_unit_row(st.rows, st.unit0, &alt);
#else
    const int64_t urow = dl_unit_row(st.rows, st.unit0 + (real ? ul : 0) * st.ustride, &alt);
#endif
    const uint32_t off = real ? (alt ? st.off_alt : st.off) : 0u, off_tail = real ? (alt ? st.off_tail_alt : st.off_tail) : 0u;
    // (a unit that is not there: a line of the matrix that is this wavefront's own, or thousands of wavefronts would
    // queue at one memory channel, and the loads behind theirs with them)
    const char* wb = reinterpret_cast<const char*>(st.w) + (real ? (urow * st.ldw + (int64_t)st.ds0 * 64) * 2 : st.idle_at);
    const int last = real ? st.dsn - 1 : 0, tail_at = st.ds_tail - st.ds0, dpw = st.dpw;
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
        // without a condition round the load (see above): a step the stream does not have repeats the last
        int step = wave + 8 * (i < dpw ? i : 0);
        step = step < last ? step : last;
        buf[i] = __builtin_nontemporal_load(
            reinterpret_cast<const dl_u32x4_t*>(wb + (int64_t)step * 128 + (step == tail_at ? off_tail : off)));
    }
}

// The LDS image of the other operand: rows of `kpad` bfloat16 (a multiple of 128), one per token; the 16-byte
// piece c of row t sits at place (c & ~15) | ((c ^ t) & 15).
__device__ __forceinline__ int dl_xs_index(int tok, int k, int kpad) {
    const int c = k >> 3;
    return tok * kpad + (((c & ~15) | ((c ^ tok) & 15)) << 3) + (k & 7);
}

// ---- the barrier ---------------------------------------------------------------------------------------
// Arrivals are counted for ever (modulo 2^32): after barrier `epoch` a group's counter stands at epoch * (its
// size) and the top counter at epoch * ngroups; the last to arrive writes the epoch into every group's flag.
// One thread of a workgroup arrives (every wavefront's stores must have been waited for: dl_stores_done, then
// a workgroup barrier) and later waits; between the two the wavefronts request the loads they want to travel
// meanwhile: memory operations of a wavefront return in order, so the counter's old value would queue behind
// loads requested before it, and requesting loads can itself stall when the memory pipe is full.
__device__ __forceinline__ void dl_arrive(uint32_t* sync, uint32_t epoch, int wg, int G) {
    const int grp = wg / DL_GROUP, ngroups = (G + DL_GROUP - 1) / DL_GROUP;
    const uint32_t gsize = (uint32_t)((grp + 1) * DL_GROUP <= G ? DL_GROUP : G - grp * DL_GROUP);
    const uint32_t old = dl_add(sync + DL_W_GROUP + grp * DL_LINE, 1u);
    if (old + 1u == epoch * gsize) {
        const uint32_t old2 = dl_add(sync + DL_W_TOP, 1u);
        if (old2 + 1u == epoch * (uint32_t)ngroups)
            for (int g = 0; g < ngroups; ++g) dl_put32(sync + DL_W_RELEASE + g * DL_LINE, epoch);
    }
}
// false when the wait ran out or somebody else's did: the caller leaves the kernel
__device__ __forceinline__ bool dl_wait(uint32_t* sync, int* err, int spin_limit, uint32_t epoch, int wg) {
    const uint32_t* flag = sync + DL_W_RELEASE + (wg / DL_GROUP) * DL_LINE;
    int spins = 0;
    while ((int32_t)(dl_get32(flag) - epoch) < 0) {
        if (++spins > spin_limit) {
            dl_put32(sync + DL_W_ABORT, 1u);
            __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return false;
        }
        if ((spins & 255) == 0 && dl_get32(sync + DL_W_ABORT)) return false;
        __builtin_amdgcn_s_sleep(1);
    }
    return true;
}
// A wait ran out: the layer's output is made NaN so that it shows in whatever reads it.
__device__ __forceinline__ void dl_poison(float* resid, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * DL_THREADS + threadIdx.x; i < count; i += (int64_t)gridDim.x * DL_THREADS)
        resid[i] = NAN;
}
// The barrier, with PREFETCH (statements that request loads for later) run by every wavefront while it lasts.
#define DL_BARRIER(EPOCH, PREFETCH)                                                   \
    do {                                                                              \
        dl_stores_done();                                                             \
        __syncthreads();                                                              \
        if (tid == 0) dl_arrive(P.sync, (EPOCH), wg, G);                              \
        { PREFETCH; }                                                                 \
        if (tid == 0) flags[31] = dl_wait(P.sync, P.err, P.spin_limit, (EPOCH), wg);  \
        __syncthreads();                                                              \
        if (!flags[31]) {                                                             \
            dl_poison(P.resid, (int64_t)P.n * P.H);                                   \
            return;                                                                   \
        }                                                                             \
    } while (0)

struct DlAcc {
    dl_f32x4_t a, b;      // the sums of k, and of k + 32
};

// The parameters live in the kernel-argument segment.  Every phase reads the ones it needs from there when it
// starts (DL_PARAMS): held in registers from the kernel's entry on, the sixty of them crowd out the scalars
// of the inner loops, and what is spilled comes back eight registers at a time.
typedef const __attribute__((address_space(4))) DlParams DlParamsK;
__device__ __forceinline__ DlParamsK* dl_fresh(DlParamsK* p) {
    asm volatile("" : "+s"(p));
    return p;
}
#define DL_PARAMS DlParamsK& P = *dl_fresh(Pk)

// four gains from j (a multiple of 4)
__device__ __forceinline__ float4 dl_gain4(const void* w, int f32, float offset, int j) {
    float4 g;
    if (f32) {
        g = *reinterpret_cast<const float4*>((const float*)w + j);
    } else {
        const uint2 raw = *reinterpret_cast<const uint2*>((const zi_bf16*)w + j);
        g = make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                        __uint_as_float(raw.y & 0xffff0000u));
    }
    g.x += offset; g.y += offset; g.z += offset; g.w += offset;
    return g;
}
__device__ __forceinline__ float dl_gain(const void* w, int f32, float offset, int j) {
    return (f32 ? ((const float*)w)[j] : zi_load((const zi_bf16*)w + j)) + offset;
}

// DPW: the most steps of k a wavefront takes of a unit in any of the four products (a template parameter: the
// buffers of a unit are registers).  NBUF units travel or wait in registers at a time.
template <int DPW>
__global__ void __launch_bounds__(DL_THREADS) decode_layer_kernel(DlParams) {
    constexpr int NBUF = DPW <= 4 ? 4 : DPW <= 7 ? 3 : 2;
    constexpr bool BREG = DPW <= 4;      // the other operand of a wavefront's steps stays in registers for a whole product
    extern __shared__ __attribute__((aligned(16))) unsigned char dl_lds[];
    DlParamsK* Pk = (DlParamsK*)__builtin_amdgcn_kernarg_segment_ptr();
    const int G = gridDim.x, wg = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / ZI_WAVE);      // the same for every lane: scalar arithmetic
    const int r = lane & 15, kg = lane >> 4, r7 = r & 7, half = r >> 3;
    // LDS: the other operand (also the attention's merge area) | wavefront sums | added sums | small things
    uint16_t* xs = reinterpret_cast<uint16_t*>(dl_lds);
    float *wsum, *red, *small;
    uint32_t* flags;
    int n;
    uint32_t base;
    {
        DL_PARAMS;
        wsum = reinterpret_cast<float*>(dl_lds + (size_t)P.lds_xs_elems * 2);       // [DL_UB][DL_WAVES][8][16]
        red = wsum + DL_UB * DL_WAVES * 128;                                          // [DL_UB][8][16]
        small = red + DL_UB * 128;                                                    // 256 floats
        flags = reinterpret_cast<uint32_t*>(small + 256);                             // 32 words
        n = P.n;
        base = dl_get32(P.sync + DL_W_BASE);
        DL_STAMP(0);
        DL_CYCLES(30);
    }
    const int tokc = r < n ? r : n - 1;         // the token whose operand row this lane reads

    dl_u32x4_t ring[NBUF][DPW];

    // ---- the weight stream against the LDS operand, unit by unit ----------------------------------------------
    DlAcc acc;
    int scratch_units = 0, scratch_first = 0;      // units whose wavefront sums lie in wsum: [first, first + units)
    // What a lane adds to the address of its operand in the LDS image: the 16-byte pieces (ds & 1) * 8 + kg and + 4
    // of a row's run of 16 pieces, swizzled; the run itself, (ds >> 1) * 256 bytes on, is the same for every lane.
    // A wavefront's steps w, w + 8, ... are all even or all odd, so it needs two of the four.
    uint32_t xsel0 = 0, xsel1 = 0;
    dl_u32x4_t breg[BREG ? DPW : 1][2];
    auto set_operand = [&](const DlStream& st, int kpad) __attribute__((always_inline)) {
        const int odd = wave & 1;
        xsel0 = (uint32_t)(tokc * kpad * 2 + ((((kg + 8 * odd) ^ tokc) & 15) << 4));
        xsel1 = (uint32_t)(tokc * kpad * 2 + ((((kg + 8 * odd + 4) ^ tokc) & 15) << 4));
        if (BREG) {
            const char* xb = reinterpret_cast<const char*>(xs);
#pragma unroll
            for (int i = 0; i < DPW; ++i) {
                int step = wave + 8 * i;
                step = step < st.dsn ? step : 0;
                breg[i][0] = *reinterpret_cast<const dl_u32x4_t*>(xb + xsel0 + (uint32_t)(step >> 1) * 256u);
                breg[i][1] = *reinterpret_cast<const dl_u32x4_t*>(xb + xsel1 + (uint32_t)(step >> 1) * 256u);
            }
        }
    };
    auto process_unit = [&](const DlStream& st, dl_u32x4_t (&buf)[DPW], int ul) __attribute__((always_inline)) {
        const int dsn = st.dsn, tail_at = st.ds_tail - st.ds0, dpw = st.dpw;
        const char* xb = reinterpret_cast<const char*>(xs);
        acc.a = dl_f32x4_t{0.f, 0.f, 0.f, 0.f};
        acc.b = acc.a;
#pragma unroll
        for (int i = 0; i < DPW; ++i) {
            if (i < dpw) {
                const int step = wave + 8 * i;
                dl_pack a, b1, b2;
                a.u = buf[i];
                if (step >= dsn) a.u = dl_u32x4_t{0u, 0u, 0u, 0u};        // a wavefront without a step of its own here
                else if (step == tail_at) a.u &= st.tail_keep;
                if (BREG) {
                    b1.u = breg[i][0];
                    b2.u = breg[i][1];
                } else {
                    const uint32_t run = (uint32_t)((step < dsn ? step : 0) >> 1) * 256u;
                    b1.u = *reinterpret_cast<const dl_u32x4_t*>(xb + xsel0 + run);
                    b2.u = *reinterpret_cast<const dl_u32x4_t*>(xb + xsel1 + run);
                }
                acc.a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b1.b, acc.a, 0, 0, 0);
                acc.b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b2.b, acc.b, 0, 0, 0);
            }
        }
        // rows 0-7 of `a` hold the unit's rows over k, rows 8-15 of `b` the same rows over k + 32
        dl_f32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc.a[e] + __shfl(acc.b[e], (lane + 32) & 63, ZI_WAVE);
        if (kg < 2) {
            float* dst = wsum + (((ul - scratch_first) * DL_WAVES + wave) * 8 + kg * 4) * 16 + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e * 16] = v[e];
        }
        ++scratch_units;
    };
    // add the wavefronts' sums of the units in wsum (rising wavefront order) into red
    auto add_up = [&]() __attribute__((always_inline)) {
        __syncthreads();
        for (int it = tid; it < scratch_units * 128; it += DL_THREADS) {
            const int u = it >> 7, e = it & 127;
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < DL_WAVES; ++w) s += wsum[(u * DL_WAVES + w) * 128 + e];
            red[it] = s;
        }
        __syncthreads();
    };
    // the first NBUF - 1 units of a stream start to travel
    auto prologue = [&](const DlStream& st) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < NBUF - 1; ++b) dl_issue_unit<DPW>(st, b, ring[b], wave);
    };
// A stream whose first NBUF - 1 units have been requested (prologue): NBUF units a turn, each unit's wavefront
// sums are left in LDS while the unit NBUF - 1 further on is requested into the buffer that was worked on last;
// then the turn's sums are added up and EPI(first unit, units) makes of them what the product is for.  The code of
// a turn is short and comes once (what runs once per launch is fetched from memory, not from the instruction
// cache: the flush and the epilogue must not be repeated for every buffer of the ring).
#define DL_UNITS(ST, KPAD, EPI, STAMP0)                                                              \
    do {                                                                                             \
        scratch_first = 0;                                                                           \
        set_operand((ST), (KPAD));                                                                   \
        for (int u0 = 0; u0 < (ST).nunits; u0 += NBUF) {                                             \
            scratch_units = 0;                                                                       \
            _Pragma("unroll") for (int b = 0; b < NBUF; ++b) {                                       \
                DL_STAMP((STAMP0) == 16 && u0 == 0 ? 16 + 2 * b : -1);                               \
                dl_issue_unit<DPW>((ST), u0 + b + NBUF - 1, ring[(b + NBUF - 1) % NBUF], wave);      \
                DL_STAMP((STAMP0) == 16 && u0 == 0 ? 17 + 2 * b : -1);                               \
                if (u0 + b < (ST).nunits) process_unit((ST), ring[b], u0 + b);                       \
            }                                                                                        \
            DL_STAMP((STAMP0) == 16 && u0 == 0 ? 24 : -1);                                           \
            add_up();                                                                                \
            DL_STAMP((STAMP0) == 16 && u0 == 0 ? 25 : -1);                                           \
            EPI(scratch_first, scratch_units);                                                       \
            DL_STAMP((STAMP0) == 16 && u0 == 0 ? 26 : -1);                                           \
            scratch_first += scratch_units;                                                          \
            __syncthreads();                                                                         \
            DL_STAMP((STAMP0) == 16 && u0 == 0 ? 27 : -1);                                           \
        }                                                                                            \
    } while (0)

    // The streams of this workgroup, each made where it is used (scalar arithmetic and five lane offsets).
    auto make_qkv = [&](DlParamsK& P) __attribute__((always_inline)) {
        DlRows rows;
        rows.mode = DL_ROWS_ROTARY; rows.d8 = P.d / 8; rows.rot8 = P.rot / 8; rows.half = P.rot / 2; rows.qk_heads = P.nh + P.nkv;
        const int N1 = (P.nh + 2 * P.nkv) * P.d;
        int first, count;
        dl_share(N1 / 8, wg, G, &first, &count);
        return dl_stream(P.wqkv, P.ld_qkv, N1, P.H, rows, first, 1, count, 0, (P.H + 63) / 64, r7, half, kg);
    };
    auto make_o = [&](DlParamsK& P) __attribute__((always_inline)) {
        DlRows rows;
        rows.mode = DL_ROWS_PLAIN; rows.d8 = 1; rows.rot8 = 0; rows.half = 0; rows.qk_heads = 0;
        int first, count;
        dl_share(P.H / 8, wg, G, &first, &count);
        const int Qd = P.nh * P.d;
        return dl_stream(P.wo, P.ld_o, P.H, Qd, rows, first, 1, count, 0, (Qd + 63) / 64, r7, half, kg);
    };
    auto make_gu = [&](DlParamsK& P) __attribute__((always_inline)) {
        DlRows rows;
        rows.mode = DL_ROWS_SWIGLU; rows.d8 = 1; rows.rot8 = 0; rows.half = 0; rows.qk_heads = 0;
        int first, count;
        dl_share(P.I / 4, wg, G, &first, &count);         // half tiles of 4 gate + 4 up rows
        return dl_stream(P.wgu, P.ld_gu, 2 * P.I, P.H, rows, first, 1, count, 0, (P.H + 63) / 64, r7, half, kg);
    };
    // down: workgroup wg takes cut wg % S of k and the units wg / S, wg / S + G / S, ...
    auto make_d = [&](DlParamsK& P, int* cut_out, int* k0_out, int* klen_out) __attribute__((always_inline)) {
        DlRows rows;
        rows.mode = DL_ROWS_PLAIN; rows.d8 = 1; rows.rot8 = 0; rows.half = 0; rows.qk_heads = 0;
        const int S = P.S, per_cut = G / S, cut = wg % S, lane_unit = wg / S, H = P.H, I = P.I;
        const int ds_total = (I + 63) / 64;
        const int dcut0 = (int)(((int64_t)ds_total * cut) / S), dcut1 = (int)(((int64_t)ds_total * (cut + 1)) / S);
        const int units = (wg < per_cut * S && lane_unit < H / 8) ? (H / 8 - lane_unit + per_cut - 1) / per_cut : 0;
        *cut_out = cut;
        *k0_out = dcut0 * 64;
        *klen_out = (I - dcut0 * 64 < (dcut1 - dcut0) * 64) ? I - dcut0 * 64 : (dcut1 - dcut0) * 64;
        return dl_stream(P.wd, P.ld_d, H, I, rows, lane_unit, per_cut, units, dcut0, dcut1 - dcut0, r7, half, kg);
    };

    // ---- phase 1: x = norm(resid) into LDS, q/k/v ----------------------------------------------------------------
    {
        DL_PARAMS;
        const int H = P.H, nh = P.nh, nkv = P.nkv, d = P.d, rot = P.rot;
        const int Qd = nh * d, KVd = nkv * d;
        const int kpadH = (H + 127) & ~127;
        const DlStream st = make_qkv(P);
        // A wavefront per token.  The row is requested first (up to 8 x 16 bytes a lane stay in registers; longer
        // rows are read again), then the first weights, which take longer and would hold the row up: a
        // wavefront's loads return in the order they were requested.
        {
            const float* resid = P.resid;
            const void* gains = P.norm1;
            const int gf32 = P.norm_f32;
            const float goff = P.w_offset, eps = P.eps1;
            const int t1 = wave < n ? wave : n - 1;
            const float* xr1 = resid + (int64_t)t1 * H;
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = lane * 4 + u * ZI_WAVE * 4;
                v[u] = *reinterpret_cast<const float4*>(xr1 + (j < H ? j : 0));
            }
            prologue(st);
            for (int t = wave; t < n; t += DL_WAVES) {
                const float* xr = resid + (int64_t)t * H;
                if (t != wave) {
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int j = lane * 4 + u * ZI_WAVE * 4;
                        v[u] = *reinterpret_cast<const float4*>(xr + (j < H ? j : 0));
                    }
                }
                float ss = 0.f;
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (lane * 4 + u * ZI_WAVE * 4 < H) ss += v[u].x * v[u].x + v[u].y * v[u].y + v[u].z * v[u].z + v[u].w * v[u].w;
                for (int j = lane * 4 + 8 * ZI_WAVE * 4; j < H; j += ZI_WAVE * 4) {
                    const float4 w = *reinterpret_cast<const float4*>(xr + j);
                    ss += w.x * w.x + w.y * w.y + w.z * w.z + w.w * w.w;
                }
                ss = zi_wave_sum(ss);
                const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int j = lane * 4 + u * ZI_WAVE * 4;
                    if (j >= kpadH) continue;
                    uint2 pk = make_uint2(0u, 0u);
                    if (j < H) {
                        const float4 g = dl_gain4(gains, gf32, goff, j);
                        pk.x = zi_pack_bf16x2(g.x * v[u].x * rstd, g.y * v[u].y * rstd);
                        pk.y = zi_pack_bf16x2(g.z * v[u].z * rstd, g.w * v[u].w * rstd);
                    }
                    *reinterpret_cast<uint2*>(xs + dl_xs_index(t, j, kpadH)) = pk;
                }
                for (int j = lane * 4 + 8 * ZI_WAVE * 4; j < kpadH; j += ZI_WAVE * 4) {
                    uint2 pk = make_uint2(0u, 0u);
                    if (j < H) {
                        const float4 w = *reinterpret_cast<const float4*>(xr + j);
                        const float4 g = dl_gain4(gains, gf32, goff, j);
                        pk.x = zi_pack_bf16x2(g.x * w.x * rstd, g.y * w.y * rstd);
                        pk.y = zi_pack_bf16x2(g.z * w.z * rstd, g.w * w.w * rstd);
                    }
                    *reinterpret_cast<uint2*>(xs + dl_xs_index(t, j, kpadH)) = pk;
                }
            }
        }
        __syncthreads();
        DL_STAMP(1);
        const int d8 = d / 8, half_rot = rot / 2;
        const void* bias = P.bias;
        const int bias_f32 = P.bias_f32, ps = P.ps;
        const float* table = P.table;
        const int32_t* slots = P.slots;
        const int64_t cache_slots = P.cache_slots;
        zi_bf16 *qbuf = P.qbuf, *kvbuf = P.kvbuf, *kcache = P.kcache, *vcache = P.vcache;
        auto epi_qkv = [&](int first_ul, int units) __attribute__((always_inline)) {
            // item: (unit, token, quarter): two neighbouring dims of one head
            for (int it = tid; it < units * 64; it += DL_THREADS) {
                const int u = it >> 6, t = (it >> 2) & 15, q4 = it & 3;
                if (t >= n) continue;
                const int unit = st.unit0 + first_ul + u;
                const int hh = unit / d8, ui = unit - hh * d8;
                const bool rotary = hh < nh + nkv && ui < rot / 8;
                const int ra = rotary ? (q4 >> 1) * 4 + (q4 & 1) * 2 : 2 * q4;
                const float* rr = red + u * 128 + t;
                float v0 = rr[ra * 16], v1 = rr[(ra + 1) * 16];
                const int row0 = dl_row(st.rows, unit, ra);           // the stacked matrix's row: also the bias index
                auto bias_at = [&](int row) {
                    return bias ? (bias_f32 ? ((const float*)bias)[row] : zi_load((const zi_bf16*)bias + row)) : 0.f;
                };
                v0 += bias_at(row0);
                v1 += bias_at(row0 + 1);
                const int dim0 = row0 - hh * d;
                if (rotary) {
                    const int rb = ra ^ 4;                             // the partner rows: the other half
                    const int rowb = dl_row(st.rows, unit, rb);
                    const float b0 = rr[rb * 16] + bias_at(rowb), b1 = rr[(rb + 1) * 16] + bias_at(rowb + 1);
                    const int pair = ui * 4 + (q4 & 1) * 2;            // < rot / 2
                    const float4 cs = *reinterpret_cast<const float4*>(table + ((int64_t)t * half_rot + pair) * 2);
                    if ((q4 >> 1) == 0) {
                        v0 = v0 * cs.x - b0 * cs.y;
                        v1 = v1 * cs.z - b1 * cs.w;
                    } else {
                        v0 = v0 * cs.x + b0 * cs.y;
                        v1 = v1 * cs.z + b1 * cs.w;
                    }
                }
                const uint32_t pk = zi_pack_bf16x2(v0, v1);
                if (hh < nh) {
                    dl_put32(qbuf + (int64_t)t * Qd + hh * d + dim0, pk);
                } else {
                    const bool is_v = hh >= nh + nkv;
                    const int kvh = hh - nh - (is_v ? nkv : 0);
                    dl_put32(kvbuf + (int64_t)t * 2 * KVd + (is_v ? KVd : 0) + kvh * d + dim0, pk);
                    const ZiSlotPlace place = zi_slot_place(slots[t], cache_slots, ps);
                    if (place.ok) {
                        if (!is_v) {
                            *reinterpret_cast<uint32_t*>(kcache + zi_key_offset(place.page, kvh, place.off, nkv, ps, d) + dim0) = pk;
                        } else {
                            vcache[zi_value_offset(place.page, kvh, dim0, place.off, nkv, ps, d)].bits = (uint16_t)(pk & 0xffffu);
                            vcache[zi_value_offset(place.page, kvh, dim0 + 1, place.off, nkv, ps, d)].bits = (uint16_t)(pk >> 16);
                        }
                    }
                }
            }
        };
        DL_UNITS(st, kpadH, epi_qkv, -100);
        DL_STAMP(2);
    }

    // ---- phase 2: attention ----------------------------------------------------------------------------------------------
    // Token t at position p sees the cached keys [lo, p - 1] and its own.  The cached range, widened down to a
    // multiple of 8, is cut into chunks of 128 * nb keys: wavefront w of a chunk's workgroup takes nb blocks of
    // 16 keys.  One task is (token, kv head, chunk); tasks wg, wg + G, ... are this workgroup's.
    {
        DL_PARAMS;
        const int nh = P.nh, nkv = P.nkv, d = P.d, Gh = P.G, nb = P.nb, max_chunks = P.max_chunks, window = P.window;
        const int Qd = nh * d, KVd = nkv * d;
        const int max_pages = P.max_pages, num_pages = P.num_pages;
        const int CK = DL_WAVES * 16 * nb;
        const int ntasks = n * nkv * max_chunks;
        const float scale_log2 = P.scale * 1.4426950408889634f;
        const int ps = P.ps, ps_shift = (ps & (ps - 1)) == 0 ? __ffs(ps) - 1 : -1;
        const int DK = (d + 31) / 32, DT = d / 16;
        const int32_t *pos = P.pos, *bt = P.bt;
        const zi_bf16 *kcache = P.kcache, *vcache = P.vcache, *qbuf = P.qbuf, *kvbuf = P.kvbuf;
        zi_bf16* attn = P.attn;
        float *part_o = P.part_o, *part_ml = P.part_ml;
        uint32_t* task_counters = P.sync + DL_W_TASK;
        // Two sets of registers for a block's keys and values: while one block is worked on the next travels.
        // The first task's first two blocks are requested while the barrier lasts: they were cached by earlier steps.
        dl_u32x4_t kregA[4], kregB[4];
        uint2 vregA[8], vregB[8];
        auto geometry = [&](int task, int* t, int* kvh, int* c, int* p, int* lo, int* lo_al, int* cnt) {
            *c = task % max_chunks;
            const int tk = task / max_chunks;
            *kvh = tk % nkv;
            *t = tk / nkv;
            *p = pos[*t];
            *lo = (window > 0 && *p - window + 1 > 0) ? *p - window + 1 : 0;
            *lo_al = *lo & ~7;
            *cnt = (*p - *lo_al + CK - 1) / CK;
        };
        auto load_block = [&](dl_u32x4_t (&kreg)[4], uint2 (&vreg)[8], int t, int kvh, int kb, int ke) __attribute__((always_inline)) {
            // keys kb .. kb + 15 (clamped to ke - 1), this lane: key kb + r, dims dk*32 + kg*8; values of keys
            // kb + 4 kg .. + 3, dims dd*16 + r
            const int32_t* btr = bt + (int64_t)t * max_pages;
            const int last = ke - 1 > 0 ? ke - 1 : 0;
            const ZiTablePlace ak = zi_table_place(kb + r, last, ps, ps_shift, max_pages - 1);
            const ZiTablePlace av = zi_table_place(kb + 4 * kg, last & ~3, ps, ps_shift, max_pages - 1);
            const int pk = zi_page_or_zero(btr[ak.index], num_pages), pv = zi_page_or_zero(btr[av.index], num_pages);
            const zi_bf16* kr = kcache + zi_key_offset(pk, kvh, ak.slot, nkv, ps, d);
            const zi_bf16* vr = vcache + zi_value_offset(pv, kvh, r, av.slot, nkv, ps, d);
#pragma unroll
            for (int dk = 0; dk < 4; ++dk)
                kreg[dk] = *reinterpret_cast<const dl_u32x4_t*>(kr + ((dk < DK && dk * 32 + kg * 8 < d) ? dk * 32 + kg * 8 : 0));
#pragma unroll
            for (int dd = 0; dd < 8; ++dd) vreg[dd] = *reinterpret_cast<const uint2*>(vr + (int64_t)(dd < DT ? dd : 0) * 16 * ps);
        };
        // request the first two blocks of a task's keys and values, when the task has keys: whether it did
        auto prefetch_task = [&](int task) __attribute__((always_inline)) {
            if (task >= ntasks) return false;
            int t, kvh, c, p, lo, lo_al, cnt;
            geometry(task, &t, &kvh, &c, &p, &lo, &lo_al, &cnt);
            if (c < cnt && cnt <= max_chunks) {
                const int kb = lo_al + c * CK + wave * 16 * nb;
                load_block(kregA, vregA, t, kvh, kb, p);
                load_block(kregB, vregB, t, kvh, kb + 16, p);
                return true;
            }
            return false;
        };
        DL_STAMP(3);
        int fetched = -1;              // the task whose first blocks travel or lie in the registers
        DL_BARRIER(base + 1u, { fetched = prefetch_task(wg) ? wg : -1; });
        DL_STAMP(4);

        float* sm = small;             // [DL_WAVES][16] maxima
        float* sl = small + 128;       // [DL_WAVES][16] sums
        dl_f32x4_t* so = reinterpret_cast<dl_f32x4_t*>(xs);     // [DL_WAVES][8][64]: the operand area is free now
        for (int task = wg; task < ntasks; task += G) {
            int t, kvh, c, p, lo, lo_al, cnt;
            geometry(task, &t, &kvh, &c, &p, &lo, &lo_al, &cnt);
            const bool over = cnt > max_chunks;          // the host sized the launch for fewer keys: NaN shows it
            const bool live = c < cnt && !over;
            if (!live && c != 0) continue;               // chunk 0 always arrives: a token without cached keys has its own
            const int expected = over ? 1 : (cnt > 1 ? cnt : 1);
            if (live) {
                if (fetched != task) prefetch_task(task);            // the task before it had no keys to ask ahead from
                const int wb = lo_al + c * CK + wave * 16 * nb;      // blocks 0 and 1 were requested before
                // the group's queries as the B operand: lane (head r, dims dk*32 + kg*8 ..)
                dl_pack qop[4];
                {
                    uint64_t qa[4], qb[4];
#pragma unroll
                    for (int dk = 0; dk < 4; ++dk) {
                        const bool in = dk < DK && r < Gh && dk * 32 + kg * 8 < d;
                        const zi_bf16* qp = qbuf + (int64_t)t * Qd + (kvh * Gh + (r < Gh ? r : 0)) * d + (in ? dk * 32 + kg * 8 : 0);
                        qa[dk] = dl_get64(qp);
                        qb[dk] = dl_get64(qp + 4);
                    }
#pragma unroll
                    for (int dk = 0; dk < 4; ++dk) {
                        const bool in = dk < DK && r < Gh && dk * 32 + kg * 8 < d;
                        qop[dk].u = dl_keep(dl_u32x4_t{(uint32_t)qa[dk], (uint32_t)(qa[dk] >> 32), (uint32_t)qb[dk],
                                                       (uint32_t)(qb[dk] >> 32)}, in);
                    }
                }
                dl_f32x4_t o[8];
#pragma unroll
                for (int dd = 0; dd < 8; ++dd) o[dd] = dl_f32x4_t{0.f, 0.f, 0.f, 0.f};
                float m = -INFINITY, lsum = 0.f;
                auto block = [&](const dl_u32x4_t (&kreg)[4], const uint2 (&vreg)[8], int kb) __attribute__((always_inline)) {
                    // scores of 16 keys for this lane's head: lane (head r, keys 4 kg .. + 3)
                    dl_f32x4_t s = dl_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int dk = 0; dk < 4; ++dk) {
                        if (dk >= DK) break;
                        dl_pack kk;
                        kk.u = dl_keep(kreg[dk], dk * 32 + kg * 8 < d);
                        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kk.b, qop[dk].b, s, 0, 0, 0);
                    }
                    float mx = -INFINITY;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int key = kb + 4 * kg + e;
                        s[e] = (key >= lo && key < p) ? s[e] * scale_log2 : -INFINITY;
                        mx = fmaxf(mx, s[e]);
                    }
                    mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
                    mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
                    const float m_new = fmaxf(m, mx);
                    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                    const float corr = __builtin_amdgcn_exp2f(m - m_use);
                    m = m_new;
                    float psum = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s[e] = __builtin_amdgcn_exp2f(s[e] - m_use);
                        psum += s[e];
                    }
                    lsum = lsum * corr + psum;
                    // P as the B operand of a 16x16x16 product: lane (head r, keys 4 kg .. + 3), exactly what it holds
                    union { uint2 u; dl_s16x4_t s4; } pb, vb;
                    pb.u.x = zi_pack_bf16x2(s[0], s[1]);
                    pb.u.y = zi_pack_bf16x2(s[2], s[3]);
                    // values of keys outside [lo, p) must be zero: 0 * NaN is NaN
                    uint2 keep;
                    {
                        const int ka = kb + 4 * kg;
                        keep.x = ((ka >= lo && ka < p) ? 0xffffu : 0u) | ((ka + 1 >= lo && ka + 1 < p) ? 0xffff0000u : 0u);
                        keep.y = ((ka + 2 >= lo && ka + 2 < p) ? 0xffffu : 0u) | ((ka + 3 >= lo && ka + 3 < p) ? 0xffff0000u : 0u);
                    }
#pragma unroll
                    for (int dd = 0; dd < 8; ++dd) {
                        if (dd >= DT) break;
                        o[dd][0] *= corr; o[dd][1] *= corr; o[dd][2] *= corr; o[dd][3] *= corr;
                        vb.u.x = vreg[dd].x & keep.x;
                        vb.u.y = vreg[dd].y & keep.y;
                        o[dd] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vb.s4, pb.s4, o[dd], 0, 0, 0);
                    }
                };
                // One block body: set A holds the block at hand, set B the next, which moves into A when the block is
                // done (the copy is also the wait for it), and the block after that is requested into B.
                for (int blk = 0; blk < nb; ++blk) {
                    const int kb = wb + blk * 16;
                    if (kb >= p) break;
                    block(kregA, vregA, kb);
#pragma unroll
                    for (int i = 0; i < 4; ++i) kregA[i] = kregB[i];
#pragma unroll
                    for (int i = 0; i < 8; ++i) vregA[i] = vregB[i];
                    if (blk + 2 < nb) load_block(kregB, vregB, t, kvh, kb + 32, p);
                }
                // the next task's first blocks travel while this one's chunk is merged and written
                fetched = prefetch_task(task + G) ? task + G : -1;
                // the eight wavefronts' (maximum, sum, output) through LDS
                lsum += __shfl_xor(lsum, 16, ZI_WAVE);
                lsum += __shfl_xor(lsum, 32, ZI_WAVE);
                if (kg == 0) {
                    sm[wave * 16 + r] = m;
                    sl[wave * 16 + r] = lsum;
                }
#pragma unroll
                for (int dd = 0; dd < 8; ++dd)
                    if (dd < DT) so[(wave * 8 + dd) * ZI_WAVE + lane] = o[dd];
                __syncthreads();
                float M = sm[r];
#pragma unroll
                for (int w = 1; w < DL_WAVES; ++w) M = fmaxf(M, sm[w * 16 + r]);
                float a[DL_WAVES], L = 0.f;
#pragma unroll
                for (int w = 0; w < DL_WAVES; ++w) {
                    a[w] = (sm[w * 16 + r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sm[w * 16 + r] - M);
                    L += a[w] * sl[w * 16 + r];
                }
                const int64_t slot = ((int64_t)t * nh + kvh * Gh + r) * max_chunks + c;
                for (int dd = wave; dd < DT; dd += DL_WAVES) {
                    dl_f32x4_t v = dl_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w = 0; w < DL_WAVES; ++w) {
                        const dl_f32x4_t x = so[(w * 8 + dd) * ZI_WAVE + lane];
                        v[0] += a[w] * x[0]; v[1] += a[w] * x[1]; v[2] += a[w] * x[2]; v[3] += a[w] * x[3];
                    }
                    if (r < Gh) {
                        float* dst = part_o + slot * d + dd * 16 + kg * 4;
#pragma unroll
                        for (int e = 0; e < 4; ++e) dl_putf(dst + e, v[e]);
                    }
                }
                if (wave == 0 && kg == 0 && r < Gh) {
                    dl_putf(part_ml + slot * 2, M);
                    dl_putf(part_ml + slot * 2 + 1, L);
                }
            }
            // ---- arrival: the last workgroup of (token, kv head) merges
            dl_stores_done();
            __syncthreads();
            if (tid == 0) {
                uint32_t* counter = task_counters + t * nkv + kvh;
                const uint32_t old = dl_add(counter, 1u);
                const bool last = (int)old + 1 == expected;
                if (last) dl_put32(counter, 0u);         // nobody touches it again in this launch
                flags[0] = last;
            }
            __syncthreads();
            if (flags[0]) {
                // Wavefront w merges heads w and w + 8 of the group; lane l holds dims 2 l and 2 l + 1, and chunk l's
                // (maximum, sum).  Everything a head needs is requested at once.
                const int ncs = over ? 0 : cnt;          // chunks to merge
                const int dl2 = 2 * lane < d ? 2 * lane : 0;
                for (int g = wave; g < Gh; g += DL_WAVES) {
                    const int head = kvh * Gh + g;
                    const int64_t slot0 = ((int64_t)t * nh + head) * max_chunks;
                    const uint32_t kk = dl_get32(kvbuf + (int64_t)t * 2 * KVd + kvh * d + dl2);
                    const uint32_t vv = dl_get32(kvbuf + (int64_t)t * 2 * KVd + KVd + kvh * d + dl2);
                    const uint32_t qq = dl_get32(qbuf + (int64_t)t * Qd + head * d + dl2);
                    const uint64_t ml = dl_get64(part_ml + (slot0 + (lane < ncs ? lane : 0)) * 2);
                    uint64_t ov[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) ov[u] = dl_get64(part_o + (slot0 + (u < ncs ? u : 0)) * d + dl2);
                    float dot = 0.f;
                    if (2 * lane < d)
                        dot = __uint_as_float(qq << 16) * __uint_as_float(kk << 16) +
                              __uint_as_float(qq & 0xffff0000u) * __uint_as_float(kk & 0xffff0000u);
                    const float sself = zi_wave_sum(dot) * scale_log2;
                    const float mc = lane < ncs ? __uint_as_float((uint32_t)ml) : -INFINITY;
                    const float lc = lane < ncs ? __uint_as_float((uint32_t)(ml >> 32)) : 0.f;
                    const float M = fmaxf(zi_wave_max(mc), sself);
                    const float wc = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - M);
                    const float ws = __builtin_amdgcn_exp2f(sself - M);
                    // sums in rising chunk order, then the own key
                    float L = 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const float w = __shfl(wc, u, ZI_WAVE);      // 0 for chunks past the count
                        L += w * __shfl(lc, u, ZI_WAVE);
                        a0 += w * __uint_as_float((uint32_t)ov[u]);
                        a1 += w * __uint_as_float((uint32_t)(ov[u] >> 32));
                    }
                    for (int c8 = 8; c8 < ncs; c8 += 8) {
#pragma unroll
                        for (int u = 0; u < 8; ++u) ov[u] = dl_get64(part_o + (slot0 + (c8 + u < ncs ? c8 + u : c8)) * d + dl2);
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const float w = __shfl(wc, (c8 + u) & 63, ZI_WAVE);
                            L += w * __shfl(lc, (c8 + u) & 63, ZI_WAVE);
                            a0 += w * __uint_as_float((uint32_t)ov[u]);
                            a1 += w * __uint_as_float((uint32_t)(ov[u] >> 32));
                        }
                    }
                    L += ws;
                    const float inv = over ? NAN : 1.f / L;
                    a0 = (a0 + ws * __uint_as_float(vv << 16)) * inv;
                    a1 = (a1 + ws * __uint_as_float(vv & 0xffff0000u)) * inv;
                    if (2 * lane < d) dl_put32(attn + (int64_t)t * Qd + head * d + 2 * lane, zi_pack_bf16x2(a0, a1));
                }
            }
            __syncthreads();
        }
        DL_STAMP(5);
    }

    // rows of `klen` values from column k0 of src (what other workgroups wrote) into the LDS image, zeros up to
    // kpad; a thread takes four values of eight rows at a time, all eight loads requested before the first is used
    auto fill_xs = [&](const zi_bf16* src, int64_t ld, int k0, int klen, int kpad) __attribute__((always_inline)) {
        for (int k = tid * 4; k < kpad; k += DL_THREADS * 4) {
            for (int tb = 0; tb < n; tb += 8) {
                uint64_t v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int t = tb + u < n ? tb + u : n - 1;
                    v[u] = dl_get64(src + (int64_t)t * ld + k0 + (k < klen ? k : 0));
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (tb + u < n) *reinterpret_cast<uint64_t*>(xs + dl_xs_index(tb + u, k, kpad)) = k < klen ? v[u] : 0ull;
            }
        }
        __syncthreads();
    };

    // ---- phase 3: output product, residual -------------------------------------------------------------------------------------
    {
        DL_PARAMS;
        const int H = P.H, Qd = P.nh * P.d;
        const int kpadQ = (Qd + 127) & ~127;
        const DlStream st = make_o(P);
        // the weights of the output product travel while the barrier lasts: nothing they need is computed here
        DL_BARRIER(base + 2u, { prologue(st); });
        DL_STAMP(6);
        fill_xs(P.attn, Qd, 0, Qd, kpadQ);
        DL_STAMP(13);
        const float* resid = P.resid;
        float *resid2 = P.resid2, *ssq = P.ssq;
        zi_bf16* x2 = P.x2;
        const void* gains = P.norm2;
        const int gf32 = P.norm_f32;
        const float goff = P.w_offset;
        auto epi_o = [&](int first_ul, int units) __attribute__((always_inline)) {
            for (int it = tid; it < units * 64; it += DL_THREADS) {
                const int u = it >> 6, t = (it >> 2) & 15, q4 = it & 3;
                const int unit = st.unit0 + first_ul + u;
                const int col = unit * 8 + 2 * q4;
                float s2 = 0.f;
                if (t < n) {
                    const float* rr = red + u * 128 + t;
                    const float2 old = *reinterpret_cast<const float2*>(resid + (int64_t)t * H + col);
                    const float v0 = old.x + rr[(2 * q4) * 16], v1 = old.y + rr[(2 * q4 + 1) * 16];
                    dl_putf(resid2 + (int64_t)t * H + col, v0);
                    dl_putf(resid2 + (int64_t)t * H + col + 1, v1);
                    dl_put32(x2 + (int64_t)t * H + col,
                             zi_pack_bf16x2(dl_gain(gains, gf32, goff, col) * v0, dl_gain(gains, gf32, goff, col + 1) * v1));
                    s2 = v0 * v0 + v1 * v1;
                }
                s2 += __shfl_xor(s2, 1, ZI_WAVE);
                s2 += __shfl_xor(s2, 2, ZI_WAVE);
                if (q4 == 0 && t < n) dl_putf(ssq + (int64_t)unit * 16 + t, s2);
            }
        };
        DL_UNITS(st, kpadQ, epi_o, -100);
        DL_STAMP(7);
    }

    // ---- phase 4: gate/up with SwiGLU ---------------------------------------------------------------------------------------------
    {
        DL_PARAMS;
        const int H = P.H, I = P.I;
        const int kpadH = (H + 127) & ~127;
        const DlStream st = make_gu(P);
        // the first units of gate/up travel while the barrier lasts
        DL_BARRIER(base + 3u, { prologue(st); });
        DL_STAMP(8);
        // 1 / rms of every token from the units' sums of squares: thread (token, part) adds the units part,
        // part + 32, ..., eight loads in flight at a time; the 32 parts are then added in rising order
        float* rstd = small + 32;      // [16]
        {
            const float* ssq = P.ssq;
            const float eps = P.eps2;
            const int units_o = H / 8;
            float* parts = red;        // [32][16]
            const int t = tid & 15, part = tid >> 4;
            float s = 0.f;
            for (int u0 = part; u0 < units_o; u0 += 32 * 8) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int u = u0 + 32 * j;
                    v[j] = (u < units_o && t < n) ? dl_getf(ssq + (int64_t)u * 16 + t) : 0.f;
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) s += v[j];
            }
            parts[part * 16 + t] = s;
            __syncthreads();
            if (tid < 16) {
                float a = 0.f;
                for (int q = 0; q < 32; ++q) a += parts[q * 16 + tid];
                rstd[tid] = 1.0f / sqrtf(a / (float)H + eps);
            }
        }
        fill_xs(P.x2, H, 0, H, kpadH);
        DL_STAMP(12);
        zi_bf16* hbuf = P.hbuf;
        auto epi_gu = [&](int first_ul, int units) __attribute__((always_inline)) {
            // item: (unit, token, pair of channels)
            for (int it = tid; it < units * 32; it += DL_THREADS) {
                const int u = it >> 5, t = (it >> 1) & 15, pp = it & 1;
                if (t >= n) continue;
                const int unit = st.unit0 + first_ul + u;
                const float* rr = red + u * 128 + t;
                const float rs = rstd[t];
                float act[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float g = rr[(2 * pp + e) * 16] * rs, up = rr[(4 + 2 * pp + e) * 16] * rs;
                    act[e] = up * (g / (1.f + expf(-g)));
                }
                const int ch = (unit >> 1) * 8 + (unit & 1) * 4 + 2 * pp;
                dl_put32(hbuf + (int64_t)t * I + ch, zi_pack_bf16x2(act[0], act[1]));
            }
        };
        DL_UNITS(st, kpadH, epi_gu, 16);
        DL_STAMP(9);
    }

    // ---- phase 5: down, cut along k; the last cut to arrive at a unit adds them up ---------------------------
    {
        DL_PARAMS;
        const int H = P.H, I = P.I, S = P.S;
        int cut, k0, klen;
        const DlStream st = make_d(P, &cut, &k0, &klen);
        const int kpadD = (st.dsn * 64 + 127) & ~127;
        DL_BARRIER(base + 4u, { prologue(st); });
        DL_STAMP(10);
        if (st.nunits) {
            fill_xs(P.hbuf, I, k0, klen, kpadD);
            DL_STAMP(14);
            float *dsum = P.dsum, *resid = P.resid;
            const float* resid2 = P.resid2;
            uint32_t* unit_counters = P.sync + DL_W_UNIT;
            auto epi_d = [&](int first_ul, int units) __attribute__((always_inline)) {
                for (int it = tid; it < units * 128; it += DL_THREADS) {
                    const int u = it >> 7, row = (it >> 4) & 7, t = it & 15;
                    if (t >= n) continue;
                    const int col = (st.unit0 + (first_ul + u) * st.ustride) * 8 + row;
                    dl_putf(dsum + ((int64_t)cut * n + t) * H + col, red[u * 128 + row * 16 + t]);
                }
                dl_stores_done();
                __syncthreads();
                if (tid < units) {
                    uint32_t* counter = unit_counters + st.unit0 + (first_ul + tid) * st.ustride;
                    const uint32_t old = dl_add(counter, 1u);
                    const bool last = (int)old + 1 == S;
                    if (last) dl_put32(counter, 0u);
                    flags[tid] = last;
                }
                __syncthreads();
                for (int it = tid; it < units * 128; it += DL_THREADS) {
                    const int u = it >> 7, row = (it >> 4) & 7, t = it & 15;
                    if (!flags[u] || t >= n) continue;
                    const int col = (st.unit0 + (first_ul + u) * st.ustride) * 8 + row;
                    const float s = dl_getf(resid2 + (int64_t)t * H + col);
                    float part[16];
#pragma unroll
                    for (int c = 0; c < 16; ++c) part[c] = c < S ? dl_getf(dsum + ((int64_t)c * n + t) * H + col) : 0.f;
                    float total = part[0];
#pragma unroll
                    for (int c = 1; c < 16; ++c) total += part[c];
                    resid[(int64_t)t * H + col] = s + total;
                }
            };
            DL_UNITS(st, kpadD, epi_d, -100);
        }
        DL_STAMP(11);
        DL_CYCLES(31);
        // the next launch starts from the epoch this one ended at (every workgroup read the base long ago: it
        // passed four barriers since)
        if (wg == 0 && tid == 0) dl_put32(P.sync + DL_W_BASE, base + (uint32_t)DL_BARRIERS);
    }
}

// ---- host side ----------------------------------------------------------------------------------------------------------
namespace {
struct DlDevice {
    int cus = 0, lds_max = 0;
    bool ready = false;
};
DlDevice dl_devices[64];
std::mutex dl_mutex;

int dl_device_info(DlDevice* out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return zi_fail("decode_layer: no current device");
    std::lock_guard<std::mutex> lock(dl_mutex);
    DlDevice& D = dl_devices[dev];
    if (!D.ready) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return zi_fail("decode_layer: cannot read the device's properties");
        D.cus = prop.multiProcessorCount;
        D.lds_max = (int)prop.sharedMemPerBlockOptin > 0 ? (int)prop.sharedMemPerBlockOptin : (int)prop.sharedMemPerBlock;
        if (D.lds_max > 160 * 1024) D.lds_max = 160 * 1024;
        const void* kernels[4] = {reinterpret_cast<const void*>(decode_layer_kernel<3>), reinterpret_cast<const void*>(decode_layer_kernel<4>),
                                  reinterpret_cast<const void*>(decode_layer_kernel<7>), reinterpret_cast<const void*>(decode_layer_kernel<10>)};
        for (const void* k : kernels)
            if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, D.lds_max) != hipSuccess)
                return zi_fail("decode_layer: cannot raise the kernel's LDS limit to %d bytes", D.lds_max);
        // every workgroup of the grid must be resident at once: one a compute unit fits, or nothing is launched
        int per_cu[4] = {0, 0, 0, 0};
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[0], decode_layer_kernel<3>, DL_THREADS, D.lds_max) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[1], decode_layer_kernel<4>, DL_THREADS, D.lds_max) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[2], decode_layer_kernel<7>, DL_THREADS, D.lds_max) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[3], decode_layer_kernel<10>, DL_THREADS, D.lds_max) != hipSuccess ||
            per_cu[0] < 1 || per_cu[1] < 1 || per_cu[2] < 1 || per_cu[3] < 1)
            return zi_fail("decode_layer: a workgroup of %d threads with %d bytes of LDS does not fit a compute unit", DL_THREADS, D.lds_max);
        D.ready = true;
    }
    *out = D;
    return 0;
}

struct DlPlan {
    int G, nb, max_chunks, S, xs_elems, lds_bytes;
    int dpw;          // the most steps of k a wavefront takes of a unit, over the four products
    int64_t off_q, off_kv, off_attn, off_resid2, off_x2, off_ssq, off_h, off_po, off_pml, off_dsum, total;
};

int64_t dl_align(int64_t v) { return (v + 255) & ~(int64_t)255; }

// The cut of the down product: cuts of k (a power of two up to 16 that divides into the workgroups) such that the
// most 8-column units x k-steps any workgroup gets is least; the fewest cuts among equals.
int dl_down_cuts(int G, int H, int I) {
    const int units = H / 8, ds_total = (I + 63) / 64;
    int64_t best = -1;
    int best_s = 1;
    for (int s = 1; s <= 16 && s <= G && s <= ds_total; s *= 2) {
        const int per_cut = G / s;
        if (((ds_total + s - 1) / s + DL_WAVES - 1) / DL_WAVES > DL_MAX_DPW && s < 16) continue;     // too long a range for one workgroup
        const int64_t cost = (int64_t)((units + per_cut - 1) / per_cut) * ((ds_total + s - 1) / s + 2);
        if (best < 0 || cost < best) { best = cost; best_s = s; }
    }
    return best_s;
}

int dl_plan(DlPlan* pl, const DlDevice& D, int n, int H, int I, int nh, int nkv, int d, int max_keys, int window) {
    pl->G = D.cus;
    const int Qd = nh * d, KVd = nkv * d;
    int keys = max_keys > 1 ? max_keys - 1 : 0;          // cached keys a token sees at most
    if (window > 0 && keys > window - 1) keys = window - 1;
    keys += 7;                                           // the range is widened down to a multiple of 8
    // blocks of 16 keys a wavefront: as few as keep the tasks to one round of the workgroups and the chunks to DL_MAXC
    int nb = (int)(((int64_t)n * nkv * keys + (int64_t)128 * pl->G - 1) / ((int64_t)128 * pl->G));
    const int nb_min = (keys + 128 * DL_MAXC - 1) / (128 * DL_MAXC);
    if (nb < nb_min) nb = nb_min;
    if (nb < 1) nb = 1;
    pl->nb = nb;
    pl->max_chunks = (keys + 128 * nb - 1) / (128 * nb);
    if (pl->max_chunks < 1) pl->max_chunks = 1;
    pl->S = dl_down_cuts(pl->G, H, I);
    const int ds_total = (I + 63) / 64;
    const int cut_len = ((ds_total + pl->S - 1) / pl->S) * 64;
    {
        const int steps_h = (H + 63) / 64, steps_q = (Qd + 63) / 64, steps_d = (ds_total + pl->S - 1) / pl->S;
        int most = steps_h > steps_q ? steps_h : steps_q;
        if (steps_d > most) most = steps_d;
        pl->dpw = (most + DL_WAVES - 1) / DL_WAVES;
    }
    int kmax = H > Qd ? H : Qd;
    if (cut_len > kmax) kmax = cut_len;
    const int kpad = (kmax + 127) & ~127;
    int xs_elems = n * kpad;
    const int merge_bytes = DL_WAVES * 8 * ZI_WAVE * 16;      // the attention's merge area
    const int weights_bytes = (16 * DL_MAXC + 16) * 4;
    if (xs_elems * 2 < merge_bytes) xs_elems = merge_bytes / 2;
    if (xs_elems * 2 < weights_bytes) xs_elems = weights_bytes / 2;
    pl->xs_elems = (xs_elems + 7) & ~7;
    pl->lds_bytes = pl->xs_elems * 2 + (DL_UB * DL_WAVES * 128 + DL_UB * 128 + 256 + 32) * 4;
    int64_t off = 0;
    pl->off_q = off; off = dl_align(off + (int64_t)n * Qd * 2);
    pl->off_kv = off; off = dl_align(off + (int64_t)n * 2 * KVd * 2);
    pl->off_attn = off; off = dl_align(off + (int64_t)n * Qd * 2);
    pl->off_resid2 = off; off = dl_align(off + (int64_t)n * H * 4);
    pl->off_x2 = off; off = dl_align(off + (int64_t)n * H * 2);
    pl->off_ssq = off; off = dl_align(off + (int64_t)(H / 8) * 16 * 4);
    pl->off_h = off; off = dl_align(off + (int64_t)n * I * 2);
    pl->off_po = off; off = dl_align(off + (int64_t)n * nh * pl->max_chunks * d * 4);
    pl->off_pml = off; off = dl_align(off + (int64_t)n * nh * pl->max_chunks * 2 * 4);
    pl->off_dsum = off; off = dl_align(off + (int64_t)pl->S * n * H * 4);
    pl->total = off;
    return 0;
}

const char* dl_unsupported(int dt, int n, int H, int I, int nh, int nkv, int d, int rot, int ps) {
    if (dt != ZI_BF16) return "bfloat16 only";
    if (n < 1 || n > DL_MAX_TOKENS) return "1..16 tokens";
    if (nkv <= 0 || nh <= 0 || nh % nkv || nh / nkv > 16) return "heads a multiple of the key/value heads, groups of up to 16";
    if (nkv > 256) return "at most 256 key/value heads";
    if (d < 16 || d > 128 || d % 16) return "head_dim a multiple of 16 up to 128";
    if (rot < 0 || rot > d || rot % 16) return "rotary dims a multiple of 16 within head_dim";
    if (H % 8 || I % 8 || H < 8 || I < 8) return "hidden and intermediate sizes multiples of 8";
    if (H / 8 > 4096) return "hidden size up to 32768";
    if (ps <= 0 || ps % 8) return "page size a multiple of 8";
    return nullptr;
}
}  // namespace

// Words of the synchronisation state; the caller allocates them on the device, zeroed once, and keeps them for
// every call (all layers share them; they must be zeroed again after a call reported a wait that ran out).
extern "C" int zi_decode_layer_sync_words() {
#ifdef DL_TIMING
    return DL_SYNC_WORDS + 256 * 32 * 2;
#else
    return DL_SYNC_WORDS;
#endif
}

// Clock stamps a workgroup leaves per launch after the synchronisation words (a -DDL_TIMING build), else 0.
extern "C" int zi_decode_layer_stamps() {
#ifdef DL_TIMING
    return 32;
#else
    return 0;
#endif
}

// 1 when zi_decode_layer takes the shape on the current device, else 0.
extern "C" int zi_decode_layer_supported(int dt, int n, int H, int I, int nh, int nkv, int d, int rot, int page_size,
                                         int max_keys, int window) {
    if (dl_unsupported(dt, n, H, I, nh, nkv, d, rot, page_size)) return 0;
    DlDevice D;
    if (dl_device_info(&D) != 0) return 0;
    DlPlan pl;
    dl_plan(&pl, D, n, H, I, nh, nkv, d, max_keys, window);
    return pl.lds_bytes <= D.lds_max && pl.max_chunks <= DL_MAXC && pl.dpw <= DL_MAX_DPW;
}

// Bytes of workspace a call with these sizes needs.
extern "C" int64_t zi_decode_layer_workspace(int n, int H, int I, int nh, int nkv, int d, int max_keys, int window) {
    DlDevice D;
    if (dl_device_info(&D) != 0) return -1;
    DlPlan pl;
    dl_plan(&pl, D, n, H, I, nh, nkv, d, max_keys, window);
    return pl.total;
}

// One pre-norm decoder layer for n <= 16 tokens that are each the only one of their sequence in the step
// (token t is of sequence t, row t of block_tables): resid [n][H] float32 is read and replaced by
//   r2 = resid + Wo . attention(rotate(Wqkv . norm1(resid) + bias));  resid = r2 + Wd . swiglu(Wgu . norm2(r2))
// with the token's new key and value stored at slot slots[t] of the cache.  wgu holds gate and up rows
// alternating in blocks of 8.  `sync` are zi_decode_layer_sync_words() zeroed words that every call shares;
// `err` is host memory that the device can write (pinned): it is set to 1 when a wait inside the kernel ran
// out, and the caller must then treat the step as failed and zero `sync`.  `max_keys` bounds position + 1 of
// every token.
extern "C" int zi_decode_layer(float* resid, int n, int H, int I, const void* norm1, const void* norm2, int norm_dt,
                               float eps1, float eps2, int add_one, const void* wqkv, int64_t ld_qkv, const void* bias,
                               int bias_dt, const void* wo, int64_t ld_o, const void* wgu, int64_t ld_gu, const void* wd,
                               int64_t ld_d, int dt, const float* table, int rot, const int32_t* slots,
                               int64_t cache_slots, void* kcache, void* vcache, const int32_t* tok_pos,
                               const int32_t* block_tables, int max_pages, int num_pages, int nh, int nkv, int d,
                               int page_size, int window, float scale, int max_keys, void* workspace,
                               int64_t workspace_bytes, uint32_t* sync, int* err, int spin_limit, hipStream_t stream) {
    const char* why = dl_unsupported(dt, n, H, I, nh, nkv, d, rot, page_size);
    ZI_REQUIRE(!why, "decode_layer: unsupported shape (%s): tokens %d hidden %d intermediate %d heads %d kv_heads %d "
               "head_dim %d rotary %d page %d", why ? why : "", n, H, I, nh, nkv, d, rot, page_size);
    ZI_REQUIRE(resid && norm1 && norm2 && wqkv && wo && wgu && wd && slots && kcache && vcache && tok_pos && block_tables &&
                   workspace && sync && err, "decode_layer: null argument");
    ZI_REQUIRE(norm_dt == ZI_BF16 || norm_dt == ZI_F32, "decode_layer: gains must be bfloat16 or float32");
    ZI_REQUIRE(!bias || bias_dt == ZI_BF16 || bias_dt == ZI_F32, "decode_layer: bias must be bfloat16 or float32");
    ZI_REQUIRE(rot == 0 || table, "decode_layer: no angle table");
    ZI_REQUIRE(eps1 > 0.f && eps2 > 0.f, "decode_layer: eps must be positive");
    ZI_REQUIRE(max_pages > 0 && num_pages > 0 && window >= 0 && max_keys >= 1 && spin_limit > 0, "decode_layer: bad sizes");
    ZI_REQUIRE(cache_slots > 0 && cache_slots % page_size == 0, "decode_layer: cache of %lld slots is not a whole number of pages of %d",
               (long long)cache_slots, page_size);
    const int Qd = nh * d, KVd = nkv * d;
    ZI_REQUIRE(ld_qkv >= H && ld_o >= Qd && ld_gu >= H && ld_d >= I && ld_qkv % 8 == 0 && ld_o % 8 == 0 && ld_gu % 8 == 0 &&
                   ld_d % 8 == 0, "decode_layer: bad row strides");
    ZI_REQUIRE(((uintptr_t)resid % 16) == 0 && ((uintptr_t)wqkv % 16) == 0 && ((uintptr_t)wo % 16) == 0 && ((uintptr_t)wgu % 16) == 0 &&
                   ((uintptr_t)wd % 16) == 0 && ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0 &&
                   ((uintptr_t)workspace % 256) == 0 && ((uintptr_t)table % 16) == 0 && ((uintptr_t)sync % 256) == 0,
               "decode_layer: operands must be aligned to 16 bytes, workspace and sync to 256");
    DlDevice D;
    if (dl_device_info(&D) != 0) return 1;
    DlPlan pl;
    dl_plan(&pl, D, n, H, I, nh, nkv, d, max_keys, window);
    ZI_REQUIRE(pl.lds_bytes <= D.lds_max, "decode_layer: %d bytes of LDS needed, %d there are", pl.lds_bytes, D.lds_max);
    ZI_REQUIRE(pl.max_chunks <= DL_MAXC, "decode_layer: too many keys");
    ZI_REQUIRE(pl.dpw <= DL_MAX_DPW, "decode_layer: rows of more than %d values", DL_MAX_DPW * DL_WAVES * 64);
    ZI_REQUIRE(workspace_bytes >= pl.total, "decode_layer: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
               (long long)pl.total);
    DlParams P;
    P.n = n; P.H = H; P.I = I; P.nh = nh; P.nkv = nkv; P.d = d; P.G = nh / nkv; P.rot = rot; P.ps = page_size;
    P.window = window; P.max_pages = max_pages; P.num_pages = num_pages; P.cache_slots = cache_slots;
    P.eps1 = eps1; P.eps2 = eps2; P.w_offset = add_one ? 1.f : 0.f; P.scale = scale;
    P.resid = resid; P.norm1 = norm1; P.norm2 = norm2; P.norm_f32 = norm_dt == ZI_F32;
    P.wqkv = (const zi_bf16*)wqkv; P.wo = (const zi_bf16*)wo; P.wgu = (const zi_bf16*)wgu; P.wd = (const zi_bf16*)wd;
    P.ld_qkv = ld_qkv; P.ld_o = ld_o; P.ld_gu = ld_gu; P.ld_d = ld_d;
    P.bias = bias; P.bias_f32 = bias_dt == ZI_F32;
    P.table = table; P.slots = slots; P.pos = tok_pos; P.bt = block_tables;
    P.kcache = (zi_bf16*)kcache; P.vcache = (zi_bf16*)vcache;
    unsigned char* ws = (unsigned char*)workspace;
    P.qbuf = (zi_bf16*)(ws + pl.off_q); P.kvbuf = (zi_bf16*)(ws + pl.off_kv); P.attn = (zi_bf16*)(ws + pl.off_attn);
    P.resid2 = (float*)(ws + pl.off_resid2); P.x2 = (zi_bf16*)(ws + pl.off_x2); P.ssq = (float*)(ws + pl.off_ssq);
    P.hbuf = (zi_bf16*)(ws + pl.off_h); P.part_o = (float*)(ws + pl.off_po); P.part_ml = (float*)(ws + pl.off_pml);
    P.dsum = (float*)(ws + pl.off_dsum);
    P.sync = sync; P.err = err;
    P.nb = pl.nb; P.max_chunks = pl.max_chunks; P.S = pl.S; P.lds_xs_elems = pl.xs_elems; P.spin_limit = spin_limit;
    if (pl.dpw <= 3) decode_layer_kernel<3><<<pl.G, DL_THREADS, pl.lds_bytes, stream>>>(P);
    else if (pl.dpw <= 4) decode_layer_kernel<4><<<pl.G, DL_THREADS, pl.lds_bytes, stream>>>(P);
    else if (pl.dpw <= 7) decode_layer_kernel<7><<<pl.G, DL_THREADS, pl.lds_bytes, stream>>>(P);
    else decode_layer_kernel<10><<<pl.G, DL_THREADS, pl.lds_bytes, stream>>>(P);
    return zi_check_launch("decode_layer");
}
