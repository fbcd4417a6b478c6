// The library matrix product for many rows: out = x . weight^T (+ bias) through hipBLASLt, called from
// this library so that every launch of a step is a call into it (nothing of a step goes through another
// host layer), and so that the algorithm is chosen by measurement where the caller asks for it.
// (reference: the engine sends products of this kind to its vendor library the same way,
// src/backend/ops/linear/nvidia/linear_cublas.cu:134-231.)
//
// All matrices are row-major: x [M, K] (row stride ldx), weight [N, K] (ldw), bfloat16.  In the
// library's column-major terms a row-major matrix is its own transpose, so
//   straight:    out [M, N] row-major (ldo) = column-major [N, M]:  A = weight (transposed), B = x
//   transposed:  out [N, M] row-major (ldo) = column-major [M, N]:  A = x (transposed),      B = weight
// both with k = K, accumulated in float32; the output is bfloat16 or float32.  The bias (bfloat16 [N],
// straight only) is added by the library's epilogue along the rows of its column-major result.
//
// One plan per shape (sizes, strides, output type, with or without bias, which way round) holds the
// library's descriptors and the algorithm: the first of the library's own proposals until
// zi_gemm_lt_tune has timed a number of them on the caller's operands and kept the fastest.  Plans, and
// with them the choices, belong to the process (every engine in it gets the same bits for a shape) and live
// until it ends.  The calls are serialised by a mutex; the handle belongs to one device, the
// one that was current at the first call.
#include "zi_common.h"
#include "zi_api.h"
#include <hipblaslt/hipblaslt.h>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace {

struct LtPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    std::vector<hipblasLtMatmulHeuristicResult_t> proposals;
    int chosen = 0;          // index into proposals
    int used = 0;            // a product of this shape has run outside of tuning
    int tuned = 0;
    float tuned_us = 0.f;
};

//                     M,       N,       K,       ldx,     ldw,     ldo,     out_dt, bias, transposed
using LtKey = std::tuple<int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int, int>;

std::mutex lt_mutex;
hipblasLtHandle_t lt_handle = nullptr;
int lt_device = -1;
std::map<LtKey, LtPlan> lt_plans;
const int LT_PROPOSALS = 32;

const char* lt_status(hipblasStatus_t s) {
    switch (s) {
        case HIPBLAS_STATUS_SUCCESS: return "success";
        case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
        case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
        case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
        case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
        case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
        case HIPBLAS_STATUS_ARCH_MISMATCH: return "architecture mismatch";
        default: return "error";
    }
}

#define LT_CHECK(call, what)                                                             \
    do {                                                                                 \
        hipblasStatus_t lt_s = (call);                                                   \
        if (lt_s != HIPBLAS_STATUS_SUCCESS) return zi_fail("gemm_lt: %s: %s (%d)", what, lt_status(lt_s), (int)lt_s); \
    } while (0)

int lt_ready() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return zi_fail("gemm_lt: no current device");
    if (lt_handle == nullptr) {
        LT_CHECK(hipblasLtCreate(&lt_handle), "creating the handle");
        lt_device = dev;
    }
    ZI_REQUIRE(dev == lt_device, "gemm_lt: made for device %d, called on device %d", lt_device, dev);
    return 0;
}

// The plan of a shape, made at its first use.  The caller holds the mutex.
int lt_plan(const LtKey& key, uint64_t workspace_bytes, LtPlan** out) {
    auto it = lt_plans.find(key);
    if (it != lt_plans.end()) {
        *out = &it->second;
        return 0;
    }
    const auto [M, N, K, ldx, ldw, ldo, out_dt, bias, transposed] = key;
    LtPlan p;
    const hipDataType tin = HIP_R_16BF, tout = out_dt == ZI_F32 ? HIP_R_32F : HIP_R_16BF;
    LT_CHECK(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "matmul descriptor");
    const int32_t opa = HIPBLAS_OP_T, opb = HIPBLAS_OP_N;
    LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opa, sizeof(opa)), "transa");
    LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opb, sizeof(opb)), "transb");
    if (bias) {
        const uint32_t ep = HIPBLASLT_EPILOGUE_BIAS;
        const int32_t bt = HIP_R_16BF;
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep)), "epilogue");
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)), "bias type");
    }
    // column-major: A is [K, m] with ld, B is [K, n], C is [m, n]
    const int64_t m = transposed ? M : N, n = transposed ? N : M;
    const int64_t lda = transposed ? ldx : ldw, ldb = transposed ? ldw : ldx;
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.a, tin, K, m, lda), "layout of A");
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.b, tin, K, n, ldb), "layout of B");
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.c, tout, m, n, ldo), "layout of C");
    hipblasLtMatmulPreference_t pref = nullptr;
    LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref), "preference");
    LT_CHECK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                                   sizeof(workspace_bytes)), "workspace preference");
    p.proposals.resize(LT_PROPOSALS);
    int got = 0;
    const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(lt_handle, p.desc, p.a, p.b, p.c, p.c, pref, LT_PROPOSALS,
                                                              p.proposals.data(), &got);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (s != HIPBLAS_STATUS_SUCCESS || got <= 0)
        return zi_fail("gemm_lt: the library proposes no algorithm for M=%lld N=%lld K=%lld (%s)", (long long)M,
                       (long long)N, (long long)K, lt_status(s));
    p.proposals.resize(got);
    *out = &(lt_plans[key] = p);
    return 0;
}

int lt_run(LtPlan* p, int which, void* out, const void* x, const void* weight, const void* bias, int transposed,
           void* workspace, uint64_t workspace_bytes, hipStream_t stream) {
    const hipblasLtMatmulHeuristicResult_t& h = p->proposals[which];
    ZI_REQUIRE(h.workspaceSize <= workspace_bytes, "gemm_lt: the algorithm wants %zu bytes of workspace, %llu are given",
               h.workspaceSize, (unsigned long long)workspace_bytes);
    if (bias)
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)), "bias pointer");
    const float alpha = 1.f, beta = 0.f;
    const void* A = transposed ? x : weight;
    const void* B = transposed ? weight : x;
    LT_CHECK(hipblasLtMatmul(lt_handle, p->desc, &alpha, A, p->a, B, p->b, &beta, out, p->c, out, p->c, &h.algo, workspace,
                             workspace_bytes, stream), "matmul");
    return 0;
}

int lt_check(const void* out, int out_dt, const void* x, const void* weight, const void* bias, int transposed, int64_t M,
             int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldo) {
    ZI_REQUIRE(out && x && weight, "gemm_lt: null operand");
    ZI_REQUIRE(out_dt == ZI_F32 || out_dt == ZI_BF16, "gemm_lt: unknown output type %d", out_dt);
    ZI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_lt: empty product %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
    ZI_REQUIRE(ldx >= K && ldw >= K && ldo >= (transposed ? M : N), "gemm_lt: a row stride is shorter than its row");
    ZI_REQUIRE(!(transposed && bias), "gemm_lt: no bias with the transposed result");
    return 0;
}

}  // namespace

// out = x . weight^T (+ bias), or its transpose; `workspace` is device memory of workspace_bytes that the
// algorithm may use (the same size at every call of a shape: it is part of what the library proposes for).
extern "C" int zi_gemm_lt(void* out, int out_dt, const void* x, const void* weight, const void* bias, int transposed,
                          int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* workspace,
                          int64_t workspace_bytes, hipStream_t stream) {
    if (lt_check(out, out_dt, x, weight, bias, transposed, M, N, K, ldx, ldw, ldo)) return 1;
    std::lock_guard<std::mutex> hold(lt_mutex);
    if (lt_ready()) return 1;
    LtPlan* p = nullptr;
    if (lt_plan(LtKey{M, N, K, ldx, ldw, ldo, out_dt, bias != nullptr, transposed != 0}, (uint64_t)workspace_bytes, &p)) return 1;
    p->used = 1;
    return lt_run(p, p->chosen, out, x, weight, bias, transposed, workspace, (uint64_t)workspace_bytes, stream);
}

// Time up to `candidates` of the library's proposals for this product on the given operands (`rounds` runs each
// after one that does not count; `out` is overwritten) and keep the fastest for every later call of the shape
// (the first proposal, unless another is at least 3 % faster).
// Waits for the stream.  A shape is tuned once: later calls return what the first found, and a shape that
// zi_gemm_lt has already served keeps the algorithm it was served with.
// chosen / proposed / microseconds may be null.
extern "C" int zi_gemm_lt_tune(void* out, int out_dt, const void* x, const void* weight, const void* bias, int transposed,
                               int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* workspace,
                               int64_t workspace_bytes, int candidates, int rounds, int* chosen, int* proposed,
                               float* microseconds, hipStream_t stream) {
    if (lt_check(out, out_dt, x, weight, bias, transposed, M, N, K, ldx, ldw, ldo)) return 1;
    ZI_REQUIRE(candidates > 0 && rounds > 0, "gemm_lt_tune: candidates and rounds must be positive");
    std::lock_guard<std::mutex> hold(lt_mutex);
    if (lt_ready()) return 1;
    LtPlan* p = nullptr;
    if (lt_plan(LtKey{M, N, K, ldx, ldw, ldo, out_dt, bias != nullptr, transposed != 0}, (uint64_t)workspace_bytes, &p)) return 1;
    if (!p->tuned && p->used) {
        // products of this shape have run with the first proposal: it stays, so that no engine of the process
        // sees its rounding change in the middle of its life
        p->tuned = 1;
    }
    if (!p->tuned) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return zi_fail("gemm_lt_tune: no events");
        const int n = candidates < (int)p->proposals.size() ? candidates : (int)p->proposals.size();
        float best = 0.f, first = 0.f;
        int best_i = -1, failed = 0;
        for (int i = 0; i < n && !failed; ++i) {
            if (p->proposals[i].workspaceSize > (uint64_t)workspace_bytes) continue;
            if (lt_run(p, i, out, x, weight, bias, transposed, workspace, (uint64_t)workspace_bytes, stream)) continue;   // not runnable: skip
            failed |= hipEventRecord(e0, stream) != hipSuccess;
            for (int r = 0; r < rounds && !failed; ++r)
                failed |= lt_run(p, i, out, x, weight, bias, transposed, workspace, (uint64_t)workspace_bytes, stream);
            failed |= hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess;
            float ms = 0.f;
            failed |= hipEventElapsedTime(&ms, e0, e1) != hipSuccess;
            if (!failed && i == 0) first = ms;
            if (!failed && (best_i < 0 || ms < best)) {
                best = ms;
                best_i = i;
            }
        }
        // the library's own first proposal stays unless another beats it by 3 %: differences below that are
        // the clock's, and a choice that flips from run to run changes the rounding for nothing
        if (!failed && best_i > 0 && first > 0.f && best > 0.97f * first) {
            best = first;
            best_i = 0;
        }
        hipEventDestroy(e0);
        hipEventDestroy(e1);
        if (failed || best_i < 0) return zi_fail("gemm_lt_tune: timing failed for M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
        p->chosen = best_i;
        p->tuned = 1;
        p->tuned_us = best * 1000.f / rounds;
    }
    if (chosen) *chosen = p->chosen;
    if (proposed) *proposed = (int)p->proposals.size();
    if (microseconds) *microseconds = p->tuned_us;
    return 0;
}

// Fix the algorithm of a shape by its place among the library's proposals (what zi_gemm_lt_tune reported in an
// earlier run), without timing anything.
extern "C" int zi_gemm_lt_choose(int out_dt, int with_bias, int transposed, int64_t M, int64_t N, int64_t K, int64_t ldx,
                                 int64_t ldw, int64_t ldo, int64_t workspace_bytes, int which) {
    std::lock_guard<std::mutex> hold(lt_mutex);
    if (lt_ready()) return 1;
    LtPlan* p = nullptr;
    if (lt_plan(LtKey{M, N, K, ldx, ldw, ldo, out_dt, with_bias != 0, transposed != 0}, (uint64_t)workspace_bytes, &p)) return 1;
    ZI_REQUIRE(which >= 0 && which < (int)p->proposals.size(), "gemm_lt_choose: proposal %d of %d", which, (int)p->proposals.size());
    ZI_REQUIRE(p->proposals[which].workspaceSize <= (uint64_t)workspace_bytes, "gemm_lt_choose: proposal %d wants more workspace", which);
    p->chosen = which;
    p->tuned = 1;
    return 0;
}
