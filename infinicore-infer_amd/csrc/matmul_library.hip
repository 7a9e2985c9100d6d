// The library matrix product for many rows, called without a framework in between:
// C[M, N] = alpha * A[M, K] W[N, K]^T through hipBLASLt.  A product's descriptors and the
// algorithm chosen for it are kept per shape, so a call costs a table lookup and one
// hipblasLtMatmul.  ic_matmul_tune times the algorithms the library proposes for a shape on
// the device and keeps the fastest.  Host code only: there is no kernel in this file.
//
// hipBLASLt is column-major.  Row-major C[M, N] = A W^T is column-major C^T[N, M] =
// (W as [K, N])^T (A as [K, M]): its matrix "A" is W with transposition, its "B" is A.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

#define IC_ERR_LIBRARY (-3)        // the library refused a call
#define IC_ERR_NO_ALGORITHM (-4)   // the library proposes no algorithm for this product

namespace {

struct Key {
    int a_dtype, c_dtype, M, N, K, lda, ldw, ldc;
    bool operator==(const Key& o) const {
        return a_dtype == o.a_dtype && c_dtype == o.c_dtype && M == o.M && N == o.N && K == o.K && lda == o.lda &&
               ldw == o.ldw && ldc == o.ldc;
    }
};
struct KeyHash {
    size_t operator()(const Key& k) const {
        size_t h = 1469598103934665603ull;
        const int v[8] = {k.a_dtype, k.c_dtype, k.M, k.N, k.K, k.lda, k.ldw, k.ldc};
        for (int x : v) h = (h ^ (size_t)(unsigned)x) * 1099511628211ull;
        return h;
    }
};
struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t lw = nullptr, la = nullptr, lc = nullptr;
    std::vector<hipblasLtMatmulHeuristicResult_t> candidates;   // [0] is the library's first choice
    int chosen = 0;
    bool all_listed = false;                                     // every algorithm of the library was appended
    bool timed = false;                                          // `chosen` comes from timing on the device
};

std::mutex g_mu;
hipblasLtHandle_t g_handle = nullptr;
std::unordered_map<Key, Plan, KeyHash> g_plans;

hipDataType lt_type(int dtype) { return dtype == IC_BF16 ? HIP_R_16BF : HIP_R_32F; }

// A product that was not timed itself takes the algorithm that timing chose for the same matrices at the
// nearest row count within an eighth of its own, if the library accepts it for this shape: the steps of a
// running batch have token counts near the budget that was timed, seldom exactly it.
void borrow_from_neighbour(const Key& key, Plan& p, size_t workspace_bytes) {
    const Plan* from = nullptr;
    int dist = 0;
    for (const auto& kv : g_plans) {
        const Key& o = kv.first;
        if (!kv.second.timed || kv.second.chosen == 0) continue;
        if (o.a_dtype != key.a_dtype || o.c_dtype != key.c_dtype || o.N != key.N || o.K != key.K || o.lda != key.lda ||
            o.ldw != key.ldw || o.ldc != key.ldc)
            continue;
        const int d = o.M > key.M ? o.M - key.M : key.M - o.M;
        if (8 * d > o.M) continue;
        if (!from || d < dist) { from = &kv.second; dist = d; }
    }
    if (!from) return;
    hipblasLtMatmulHeuristicResult_t r = from->candidates[from->chosen];
    const float one = 1.f, zero = 0.f;
    size_t need = 0;
    if (hipblaslt_ext::matmulIsAlgoSupported(g_handle, p.desc, &one, p.lw, p.la, &zero, p.lc, p.lc, r.algo, need) !=
            HIPBLAS_STATUS_SUCCESS || need > workspace_bytes)
        return;
    r.workspaceSize = need;
    r.state = HIPBLAS_STATUS_SUCCESS;
    p.candidates.push_back(r);
    p.chosen = (int)p.candidates.size() - 1;
}

// Finds or makes the plan of a product.  Called with g_mu held.
int plan_for(const Key& key, size_t workspace_bytes, Plan** out) {
    auto it = g_plans.find(key);
    if (it != g_plans.end()) { *out = &it->second; return IC_OK; }
    if (!g_handle && hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) return IC_ERR_LIBRARY;
    Plan p;
    const hipblasOperation_t tw = HIPBLAS_OP_T, ta = HIPBLAS_OP_N;
    bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &tw, sizeof(tw)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &ta, sizeof(ta)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.lw, lt_type(key.a_dtype), key.K, key.N, key.ldw) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.la, lt_type(key.a_dtype), key.K, key.M, key.lda) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.lc, lt_type(key.c_dtype), key.N, key.M, key.ldc) == HIPBLAS_STATUS_SUCCESS;
    hipblasLtMatmulPreference_t pref = nullptr;
    ok = ok && hipblasLtMatmulPreferenceCreate(&pref) == HIPBLAS_STATUS_SUCCESS;
    const uint64_t ws = workspace_bytes;
    ok = ok && hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)) == HIPBLAS_STATUS_SUCCESS;
    int found = 0;
    if (ok) {
        p.candidates.resize(16);
        ok = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.lw, p.la, p.lc, p.lc, pref, (int)p.candidates.size(),
                                             p.candidates.data(), &found) == HIPBLAS_STATUS_SUCCESS;
    }
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (ok) {
        std::vector<hipblasLtMatmulHeuristicResult_t> usable;
        for (int i = 0; i < found; ++i)
            if (p.candidates[i].state == HIPBLAS_STATUS_SUCCESS && p.candidates[i].workspaceSize <= workspace_bytes)
                usable.push_back(p.candidates[i]);
        p.candidates.swap(usable);
    }
    if (!ok || p.candidates.empty()) {
        if (p.lw) hipblasLtMatrixLayoutDestroy(p.lw);
        if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
        if (p.lc) hipblasLtMatrixLayoutDestroy(p.lc);
        if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
        return ok ? IC_ERR_NO_ALGORITHM : IC_ERR_LIBRARY;
    }
    borrow_from_neighbour(key, p, workspace_bytes);
    *out = &g_plans.emplace(key, std::move(p)).first->second;
    return IC_OK;
}

int run(Plan& p, int which, const void* A, const void* W, void* C, float alpha, void* workspace, size_t workspace_bytes,
        hipStream_t stream) {
    const float beta = 0.f;
    const hipblasLtMatmulHeuristicResult_t& r = p.candidates[which];
    const hipblasStatus_t st = hipblasLtMatmul(g_handle, p.desc, &alpha, W, p.lw, A, p.la, &beta, C, p.lc, C, p.lc, &r.algo,
                                               workspace, workspace_bytes, stream);
    return st == HIPBLAS_STATUS_SUCCESS ? IC_OK : IC_ERR_LIBRARY;
}

bool args_ok(const void* A, int a_dtype, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc) {
    const bool types = (a_dtype == IC_BF16 && (c_dtype == IC_BF16 || c_dtype == IC_F32)) || (a_dtype == IC_F32 && c_dtype == IC_F32);
    return types && A && W && C && M > 0 && N > 0 && K > 0 && lda >= K && ldw >= K && ldc >= N;
}

}  // namespace

// 1 when the direct path takes these types (bfloat16 operands with a bfloat16 or float32 result; all float32).
IC_EXPORT int ic_matmul_supported(int a_dtype, int c_dtype) {
    return (a_dtype == IC_BF16 && (c_dtype == IC_BF16 || c_dtype == IC_F32)) || (a_dtype == IC_F32 && c_dtype == IC_F32);
}

// C[M, N] = alpha * A[M, K] W[N, K]^T (W has A's type).  workspace: device memory the library may use.
IC_EXPORT int ic_matmul(const void* A, int a_dtype, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                        int ldw, int ldc, float alpha, void* workspace, long long workspace_bytes, hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (!args_ok(A, a_dtype, W, C, c_dtype, M, N, K, lda, ldw, ldc) || workspace_bytes < 0) return IC_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_mu);
    Plan* p = nullptr;
    const int st = plan_for(Key{a_dtype, c_dtype, M, N, K, lda, ldw, ldc}, (size_t)workspace_bytes, &p);
    if (st) return st;
    return run(*p, p->chosen, A, W, C, alpha, workspace, (size_t)workspace_bytes, stream);
}

// Times every algorithm the library proposes for this product (reps launches each, after one to warm up) on
// `stream` and keeps the fastest, if it beats the library's first choice by 3 %, for later ic_matmul calls of the
// same shape, and of shapes first seen later that differ only by a row count within an eighth of this one.
// Synchronises the stream.
// flush (may be nullptr): device memory, larger than the chip's caches, that is overwritten before every timed
// launch, so that the operands come from memory as a model's weights do and not from the last launch's cache lines.
// Returns the number of algorithms tried (>= 1) or an error code (< 0).
IC_EXPORT int ic_matmul_tune(const void* A, int a_dtype, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldw, int ldc, void* workspace, long long workspace_bytes, void* flush, long long flush_bytes,
                             int reps, hipStream_t stream) {
    if (!args_ok(A, a_dtype, W, C, c_dtype, M, N, K, lda, ldw, ldc) || workspace_bytes < 0 || reps < 1 || flush_bytes < 0) return IC_ERR_ARG;
    if (!flush) flush_bytes = 0;
    std::lock_guard<std::mutex> lock(g_mu);
    Plan* p = nullptr;
    const int st = plan_for(Key{a_dtype, c_dtype, M, N, K, lda, ldw, ldc}, (size_t)workspace_bytes, &p);
    if (st) return st;
    if (!p->all_listed) {
        // beside what the heuristic proposes, every algorithm the library has for these types that takes this shape
        p->all_listed = true;
        std::vector<hipblasLtMatmulHeuristicResult_t> all;
        const hipDataType ta = lt_type(a_dtype), tc = lt_type(c_dtype);
        if (hipblaslt_ext::getAllAlgos(g_handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, ta, ta, tc,
                                       tc, HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
            const float one = 1.f, zero = 0.f;
            for (auto& r : all) {
                size_t need = 0;
                if (hipblaslt_ext::matmulIsAlgoSupported(g_handle, p->desc, &one, p->lw, p->la, &zero, p->lc, p->lc, r.algo,
                                                         need) != HIPBLAS_STATUS_SUCCESS || need > (size_t)workspace_bytes)
                    continue;
                r.workspaceSize = need;
                r.state = HIPBLAS_STATUS_SUCCESS;
                p->candidates.push_back(r);
            }
        }
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return IC_ERR_LIBRARY;
    if (hipEventCreate(&e1) != hipSuccess) { hipEventDestroy(e0); return IC_ERR_LIBRARY; }
    auto time_one = [&](int i, int n) -> float {            // ms per launch, < 0: failed
        if (run(*p, i, A, W, C, 1.0f, workspace, (size_t)workspace_bytes, stream) != IC_OK) return -1.f;
        float total = 0.f;
        for (int r = 0; r < n; ++r) {
            if (flush_bytes > 0 && hipMemsetAsync(flush, r & 1, (size_t)flush_bytes, stream) != hipSuccess) return -1.f;
            hipEventRecord(e0, stream);
            const bool ok = run(*p, i, A, W, C, 1.0f, workspace, (size_t)workspace_bytes, stream) == IC_OK;
            hipEventRecord(e1, stream);
            float ms = 0.f;
            if (hipEventSynchronize(e1) != hipSuccess || !ok || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.f;
            total += ms;
        }
        return total / n;
    };
    // first round: one timed launch each; second round: the eight best and the first choice, reps launches each
    std::vector<std::pair<float, int>> quick;
    for (int i = 0; i < (int)p->candidates.size(); ++i) {
        const float ms = time_one(i, 1);
        if (ms >= 0.f) quick.push_back({ms, i});
    }
    std::sort(quick.begin(), quick.end());
    std::vector<int> finalists = {0};
    for (size_t k = 0; k < quick.size() && finalists.size() < 9; ++k)
        if (quick[k].second != 0) finalists.push_back(quick[k].second);
    float best = -1.f, first = -1.f;
    int best_i = 0, tried = (int)quick.size();
    for (int i : finalists) {
        const float ms = time_one(i, reps);
        if (ms < 0.f) continue;
        if (i == 0) first = ms;
        if (best < 0.f || ms < best) { best = ms; best_i = i; }
    }
    if (best < 0.f) tried = 0;
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    if (tried == 0) return IC_ERR_LIBRARY;
    // the library's own first choice stays unless another is clearly (3 %) faster: timing noise must not pick
    p->chosen = (first > 0.f && best > 0.97f * first) ? 0 : best_i;
    p->timed = true;
    return tried;
}
