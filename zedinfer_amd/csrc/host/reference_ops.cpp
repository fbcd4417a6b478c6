// Plain C++ references of the operators that the HIP kernels compute, for the host compiler.
//
// One function an operator, loops over whole arrays, float32 in and out with sums in double, no tiling, no
// vector types, nothing shared with the kernels' sources (the places of the paged cache are written out
// here once more, on purpose).  The tests compile this file with g++ and hold it against the plain Python
// implementation on the CPU, and the kernels against it on the GPU.  The formulas are the reference
// engine's (cited at each function; paths relative to its checkout), which keeps a CPU implementation
// beside every device operator in the same way (src/backend/ops/*/cpu/).
//
// Layout of the paged cache, as the kernels have it: keys [page][kv_head][slot][dim], values transposed
// [page][kv_head][dim][slot]; a token's place is given as a global slot number page * page_size + offset;
// a sequence's pages are a row of `block_tables` ([sequences][max_pages], -1 where it holds none).
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <algorithm>
#include <limits>
#include <vector>

namespace {

char ref_error[512] = "";

int ref_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ref_error, sizeof(ref_error), fmt, ap);
    va_end(ap);
    return 1;
}

#define REF_REQUIRE(cond, ...) \
    do {                       \
        if (!(cond)) return ref_fail(__VA_ARGS__); \
    } while (0)

int64_t key_place(int64_t page, int kv_head, int slot, int dim, int nkv, int ps, int d) {
    return ((page * nkv + kv_head) * ps + slot) * d + dim;
}

int64_t value_place(int64_t page, int kv_head, int slot, int dim, int nkv, int ps, int d) {
    return ((page * nkv + kv_head) * d + dim) * ps + slot;
}

}  // namespace

extern "C" const char* ref_last_error() { return ref_error; }

// out[i, :] = table[ids[i], :], no scaling; an id outside the table gives a row of NaN (the engine's choice:
// it shows instead of reading foreign memory).  (src/backend/ops/embedding/cpu/embedding_cpu.cpp:10-23)
extern "C" int ref_embedding(float* out, const float* table, const int* ids, int n, int vocab, int width) {
    REF_REQUIRE(out && table && ids && n >= 0 && vocab > 0 && width > 0, "embedding: bad arguments");
    for (int i = 0; i < n; ++i)
        for (int c = 0; c < width; ++c)
            out[(int64_t)i * width + c] = (ids[i] >= 0 && ids[i] < vocab) ? table[(int64_t)ids[i] * width + c]
                                                                         : std::numeric_limits<float>::quiet_NaN();
    return 0;
}

// y = w * x / sqrt(mean(x^2) + eps): eps inside the root, the weight as it is (add_one: 1 + w, for families
// that store the gain that way).  (src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:17-29)
extern "C" int ref_rms_norm(float* out, const float* x, const float* w, int n, int width, float eps, int add_one) {
    REF_REQUIRE(out && x && w && n >= 0 && width > 0 && eps > 0.f, "rms_norm: bad arguments");
    for (int i = 0; i < n; ++i) {
        const float* row = x + (int64_t)i * width;
        double ss = 0.0;
        for (int c = 0; c < width; ++c) ss += (double)row[c] * (double)row[c];
        const double inv = 1.0 / std::sqrt(ss / width + (double)eps);
        for (int c = 0; c < width; ++c)
            out[(int64_t)i * width + c] = (float)(((add_one ? 1.0 : 0.0) + (double)w[c]) * ((double)row[c] * inv));
    }
    return 0;
}

// The residual sum and the norm after it: resid += delta (in place, float32: the residual stream is kept in
// 32 bits), out = rms_norm(resid).  (src/frontend/models/transformer_forward.cpp:113-118: add, then norm)
extern "C" int ref_add_rms_norm(float* resid, const float* delta, float* out, const float* w, int n, int width, float eps,
                                int add_one) {
    REF_REQUIRE(resid && delta, "add_rms_norm: bad arguments");
    for (int64_t i = 0; i < (int64_t)n * width; ++i) resid[i] = resid[i] + delta[i];
    return ref_rms_norm(out, resid, w, n, width, eps, add_one);
}

// out[M, N] = x[M, K] . w[N, K]^T + bias[N]  (src/backend/ops/linear/op.cpp:57-58;
// src/backend/ops/linear/cpu/linear_cpu.cpp:26-85)
extern "C" int ref_linear(float* out, const float* x, const float* w, const float* bias, int M, int N, int K) {
    REF_REQUIRE(out && x && w && M >= 0 && N > 0 && K > 0, "linear: bad arguments");
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double s = 0.0;
            for (int k = 0; k < K; ++k) s += (double)x[(int64_t)m * K + k] * (double)w[(int64_t)n * K + k];
            out[(int64_t)m * N + n] = (float)(s + (bias ? (double)bias[n] : 0.0));
        }
    return 0;
}

// Rotation of the first rotary_dim dims of every head of x [n, heads, d], in place, by the tokens' absolute
// positions: the dims are paired (k, k + rotary_dim / 2), the pair's angle is pos / theta^(2k / rotary_dim),
//   x[k] <- a cos - b sin,  x[k + rotary_dim / 2] <- b cos + a sin   (a, b the old values).
// (src/backend/ops/rope/cpu/rope_cpu.cpp:33, :47-52, :62-65)
extern "C" int ref_rope_neox(float* x, const int* pos, int n, int heads, int d, int rotary_dim, double theta) {
    REF_REQUIRE(x && pos && n >= 0 && heads > 0 && d > 0, "rope: bad arguments");
    REF_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0 && theta > 0.0, "rope: rotary_dim %d of %d",
                rotary_dim, d);
    const int half = rotary_dim / 2;
    for (int i = 0; i < n; ++i)
        for (int h = 0; h < heads; ++h) {
            float* v = x + ((int64_t)i * heads + h) * d;
            for (int k = 0; k < half; ++k) {
                const double angle = (double)pos[i] / std::pow(theta, 2.0 * k / rotary_dim);
                const double c = std::cos(angle), s = std::sin(angle), a = v[k], b = v[k + half];
                v[k] = (float)(a * c - b * s);
                v[k + half] = (float)(b * c + a * s);
            }
        }
    return 0;
}

// The new tokens' keys [n, nkv, d] (rotated already) and values go to their slots of the paged cache; a
// token with slot -1 is stored nowhere (padding).  (The reference scatters by slot the same way,
// src/backend/ops/kv_scatter/nvidia/paged_kv_scatter.cu, called at src/frontend/models/transformer_forward.cpp:103;
// its cache keeps the values untransposed.)
extern "C" int ref_kv_store(float* kcache, float* vcache, const float* k, const float* v, const int* slots, int n, int nkv,
                            int d, int ps, int num_pages) {
    REF_REQUIRE(kcache && vcache && k && v && slots && nkv > 0 && d > 0 && ps > 0 && num_pages > 0, "kv_store: bad arguments");
    for (int i = 0; i < n; ++i) {
        if (slots[i] < 0) continue;
        const int64_t page = slots[i] / ps;
        const int off = slots[i] % ps;
        REF_REQUIRE(page < num_pages, "kv_store: token %d goes to slot %d, the pool has %d pages of %d", i, slots[i],
                    num_pages, ps);
        for (int h = 0; h < nkv; ++h)
            for (int c = 0; c < d; ++c) {
                kcache[key_place(page, h, off, c, nkv, ps, d)] = k[((int64_t)i * nkv + h) * d + c];
                vcache[value_place(page, h, off, c, nkv, ps, d)] = v[((int64_t)i * nkv + h) * d + c];
            }
    }
    return 0;
}

// Causal grouped-query attention of n query tokens over the paged cache.  Token i belongs to sequence
// tok_seq[i] and stands at position p = tok_pos[i]; its head h (key/value head h / (nh / nkv)) sees the
// keys at positions [max(0, p - window + 1), p] (window 0: all of [0, p]) of that sequence, key j in slot
// j % ps of page block_tables[seq][j / ps]:  s_j = (q . k_j) * scale (the scale after the dot product),
// softmax with the maximum taken off, out = sum_j P_j v_j.  The same function stands beside the prompt
// kernels and the decode kernels: they differ in how they walk, not in what they compute.
// (src/backend/ops/self_attention/cpu/paged_attention_cpu.cpp:106-162; grouping :111, bound :116, scale :135)
extern "C" int ref_paged_attention(float* out, const float* q, const float* kcache, const float* vcache,
                                   const int* block_tables, int max_pages, const int* tok_seq, const int* tok_pos, int n,
                                   int nh, int nkv, int d, int ps, int num_pages, int window, float scale) {
    REF_REQUIRE(out && q && kcache && vcache && block_tables && tok_seq && tok_pos, "attention: null argument");
    REF_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0 && d > 0 && ps > 0 && max_pages > 0 && window >= 0,
                "attention: heads %d / %d, head_dim %d, page size %d", nh, nkv, d, ps);
    const int group = nh / nkv;
    std::vector<double> score, acc(d);
    for (int i = 0; i < n; ++i) {
        const int p = tok_pos[i];
        REF_REQUIRE(p >= 0 && p / ps < max_pages, "attention: token %d at position %d, tables of %d pages", i, p, max_pages);
        const int* table = block_tables + (int64_t)tok_seq[i] * max_pages;
        const int lo = window > 0 ? std::max(0, p - window + 1) : 0;
        for (int h = 0; h < nh; ++h) {
            const int g = h / group;
            const float* qv = q + ((int64_t)i * nh + h) * d;
            score.assign(p - lo + 1, 0.0);
            double top = -std::numeric_limits<double>::infinity();
            for (int j = lo; j <= p; ++j) {
                const int page = table[j / ps];
                REF_REQUIRE(page >= 0 && page < num_pages, "attention: token %d needs key %d, page %d of the table is %d", i, j,
                            j / ps, page);
                double s = 0.0;
                for (int c = 0; c < d; ++c) s += (double)qv[c] * (double)kcache[key_place(page, g, j % ps, c, nkv, ps, d)];
                score[j - lo] = s * (double)scale;
                top = std::max(top, score[j - lo]);
            }
            double sum = 0.0;
            std::fill(acc.begin(), acc.end(), 0.0);
            for (int j = lo; j <= p; ++j) {
                const double w = std::exp(score[j - lo] - top);
                sum += w;
                const int page = table[j / ps];
                for (int c = 0; c < d; ++c) acc[c] += w * (double)vcache[value_place(page, g, j % ps, c, nkv, ps, d)];
            }
            for (int c = 0; c < d; ++c) out[((int64_t)i * nh + h) * d + c] = (float)(acc[c] / sum);
        }
    }
    return 0;
}

// out = up * gate / (1 + exp(-gate))  (src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23)
extern "C" int ref_swiglu(float* out, const float* gate, const float* up, int64_t count) {
    REF_REQUIRE(out && gate && up && count >= 0, "swiglu: bad arguments");
    for (int64_t i = 0; i < count; ++i) out[i] = (float)((double)up[i] * ((double)gate[i] / (1.0 + std::exp(-(double)gate[i]))));
    return 0;
}

// The highest logit of every row, the lowest index among equals; NaN never wins.
// (src/backend/ops/argmax/cpu/argmax_cpu.cpp:11-55, ties :17-19)
extern "C" int ref_argmax(int* out, const float* logits, int rows, int vocab) {
    REF_REQUIRE(out && logits && rows >= 0 && vocab > 0, "argmax: bad arguments");
    for (int r = 0; r < rows; ++r) {
        int best = 0;
        float top = -std::numeric_limits<float>::infinity();
        bool any = false;
        for (int i = 0; i < vocab; ++i) {
            const float v = logits[(int64_t)r * vocab + i];
            if (v > top || (!any && v == top)) {
                top = v;
                best = i;
                any = true;
            }
        }
        out[r] = best;
    }
    return 0;
}

// One token a row by temperature / top-k / top-p / repetition-penalty sampling from the uniform draw u of the
// row: penalty on the raw logits of the listed recent tokens (l > 0 ? l / p : l * p, once per listing),
// division by the temperature, softmax, order by falling probability (equal ones by rising id), keep the
// first top_k (0: all), then the smallest prefix whose sum reaches top_p, renormalise, take the first entry
// whose running sum exceeds u (the last one if none does).  A row with temperature <= 0 takes the argmax
// of its raw logits.  Probabilities are float32, as the sampler's that this follows.
// (src/frontend/sampler/sampler.cpp:195-265 truncatedDist and sampleFromDist, :410-490 the steps)
extern "C" int ref_sample(int* out, const float* logits, int rows, int vocab, const float* temperature, const int* top_k,
                          const float* top_p, const float* penalty, const float* uniform, const int* recent,
                          const int* recent_len, int max_recent) {
    REF_REQUIRE(out && logits && temperature && top_k && top_p && penalty && uniform && rows >= 0 && vocab > 0,
                "sample: bad arguments");
    std::vector<float> l(vocab), prob(vocab);
    std::vector<int> order(vocab);
    for (int r = 0; r < rows; ++r) {
        const float* row = logits + (int64_t)r * vocab;
        if (!(temperature[r] > 0.f)) {
            if (ref_argmax(out + r, row, 1, vocab)) return 1;
            continue;
        }
        for (int i = 0; i < vocab; ++i) l[i] = row[i];
        if (recent && recent_len && penalty[r] != 1.f)
            for (int k = 0; k < recent_len[r] && k < max_recent; ++k) {
                const int t = recent[(int64_t)r * max_recent + k];
                if (t >= 0 && t < vocab) l[t] = l[t] > 0.f ? l[t] / penalty[r] : l[t] * penalty[r];
            }
        float top = -std::numeric_limits<float>::infinity();
        for (int i = 0; i < vocab; ++i) {
            l[i] = l[i] / temperature[r];
            top = std::max(top, l[i]);
        }
        double sum = 0.0;
        for (int i = 0; i < vocab; ++i) {
            prob[i] = std::exp(l[i] - top);
            sum += prob[i];
        }
        for (int i = 0; i < vocab; ++i) {
            prob[i] = (float)(prob[i] / sum);
            order[i] = i;
        }
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return prob[a] > prob[b]; });
        int keep = (top_k[r] > 0 && top_k[r] < vocab) ? top_k[r] : vocab;
        if (top_p[r] < 1.f) {
            double run = 0.0;
            for (int i = 0; i < keep; ++i) {
                run += prob[order[i]];
                if (run >= (double)top_p[r]) {
                    keep = i + 1;
                    break;
                }
            }
        }
        double kept = 0.0;
        for (int i = 0; i < keep; ++i) kept += prob[order[i]];
        double run = 0.0;
        int chosen = order[keep - 1];
        for (int i = 0; i < keep; ++i) {
            run += prob[order[i]] / kept;
            if (run > (double)uniform[r]) {
                chosen = order[i];
                break;
            }
        }
        out[r] = chosen;
    }
    return 0;
}
