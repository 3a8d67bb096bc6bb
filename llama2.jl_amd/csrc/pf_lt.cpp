// Plain products of the batched prompt pass through hipBLASLt (ROCm's GEMM library):
//   D[M][N] (fp32) = X[M][K] (bf16) * W[N][K]^T (bf16)  (+ D),  fp32 sums
// which is matmul! (reference src/matmul.jl:3-23) for M activation vectors at once on weights expanded to bf16.
// Used for the products without arithmetic behind them (q | k | v, and wo and w2 with their residual add as
// beta = 1); w1 | w3 with SwiGLU and the attention stay with this library's own kernels (k_prefill.hip).
//
// The library is opened at run time (dlopen), so that this one does not need it to load: where it is missing, or any
// of its calls fails at set-up, pf_lt_open returns nullptr with the reason and the prompt pass runs its own product
// kernels throughout.
#include <dlfcn.h>
#include <stdlib.h>
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <map>
#include <string>
#include <tuple>
#include <vector>

#include "l2h_internal.h"

namespace {
struct LtApi {
    void *so = nullptr;
#define LT_FN(name) decltype(&hipblasLt##name) name = nullptr
    LT_FN(Create);
    LT_FN(Destroy);
    LT_FN(MatmulDescCreate);
    LT_FN(MatmulDescDestroy);
    LT_FN(MatmulDescSetAttribute);
    LT_FN(MatrixLayoutCreate);
    LT_FN(MatrixLayoutDestroy);
    LT_FN(MatmulPreferenceCreate);
    LT_FN(MatmulPreferenceDestroy);
    LT_FN(MatmulPreferenceSetAttribute);
    LT_FN(MatmulAlgoGetHeuristic);
    LT_FN(Matmul);
#undef LT_FN
};

struct LtPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t lw = nullptr, lx = nullptr, ld = nullptr;
    hipblasLtMatmulAlgo_t algo{};
};
}  // namespace

struct PfLt {
    LtApi api;
    hipblasLtHandle_t handle = nullptr;
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    std::map<std::tuple<int, int64_t, int64_t, int64_t, bool>, LtPlan> plans;
};

static const size_t PF_LT_WORKSPACE = (size_t)64 << 20;
static const int PF_LT_CANDIDATES = 4;  // heuristic results timed once per shape (the first is not always the fastest)

void pf_lt_close(PfLt *lt) {
    if (!lt) return;
    for (auto &kv : lt->plans) {
        LtPlan &p = kv.second;
        if (p.lw) lt->api.MatrixLayoutDestroy(p.lw);
        if (p.lx) lt->api.MatrixLayoutDestroy(p.lx);
        if (p.ld) lt->api.MatrixLayoutDestroy(p.ld);
        if (p.desc) lt->api.MatmulDescDestroy(p.desc);
    }
    if (lt->handle) lt->api.Destroy(lt->handle);
    if (lt->workspace) (void)hipFree(lt->workspace);
    if (lt->api.so) dlclose(lt->api.so);
    delete lt;
}

PfLt *pf_lt_open(std::string *why) {
    auto fail = [&](PfLt *lt, const std::string &m) -> PfLt * {
        if (why) *why = m;
        pf_lt_close(lt);
        return nullptr;
    };
    PfLt *lt = new PfLt();
    LtApi &a = lt->api;
    // L2H_HIPBLASLT names the shared object to open instead of the system's (another build of the library; a name that
    // does not exist leaves the own product kernels in charge, which is how the fallback is tested)
    const char *named = getenv("L2H_HIPBLASLT");
    if (named && *named) {
        a.so = dlopen(named, RTLD_NOW | RTLD_LOCAL);
    } else {
        a.so = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
        if (!a.so) a.so = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
    }
    if (!a.so) {
        const char *e = dlerror();
        return fail(lt, std::string("hipBLASLt not found: ") + (e ? e : ""));
    }
#define LT_SYM(name)                                                                   \
    do {                                                                               \
        a.name = (decltype(a.name))dlsym(a.so, "hipblasLt" #name);                     \
        if (!a.name) return fail(lt, "hipBLASLt lacks hipblasLt" #name);               \
    } while (0)
    LT_SYM(Create);
    LT_SYM(Destroy);
    LT_SYM(MatmulDescCreate);
    LT_SYM(MatmulDescDestroy);
    LT_SYM(MatmulDescSetAttribute);
    LT_SYM(MatrixLayoutCreate);
    LT_SYM(MatrixLayoutDestroy);
    LT_SYM(MatmulPreferenceCreate);
    LT_SYM(MatmulPreferenceDestroy);
    LT_SYM(MatmulPreferenceSetAttribute);
    LT_SYM(MatmulAlgoGetHeuristic);
    LT_SYM(Matmul);
#undef LT_SYM
    if (a.Create(&lt->handle) != HIPBLAS_STATUS_SUCCESS) {
        lt->handle = nullptr;
        return fail(lt, "hipblasLtCreate failed");
    }
    if (hipMalloc(&lt->workspace, PF_LT_WORKSPACE) != hipSuccess) {
        lt->workspace = nullptr;
        return fail(lt, "no memory for the hipBLASLt workspace");
    }
    lt->workspace_bytes = PF_LT_WORKSPACE;
    return lt;
}

// In the library's column-major terms: D^T (N x M, leading dimension ldd) = op_T(W as K x N) * (X as K x M) + beta D^T.
static bool pf_lt_plan(PfLt *lt, hipStream_t s, LtPlan &p, const uint16_t *W, const uint16_t *X, int M, int64_t N, int64_t K,
                       int64_t ldd, bool accumulate, std::string *err) {
    LtApi &a = lt->api;
    auto bad = [&](const char *m) {
        if (err) *err = m;
        return false;
    };
    if (a.MatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return bad("hipblasLtMatmulDescCreate");
    const hipblasOperation_t tw = HIPBLAS_OP_T, tx = HIPBLAS_OP_N;
    if (a.MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &tw, sizeof(tw)) != HIPBLAS_STATUS_SUCCESS ||
        a.MatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tx, sizeof(tx)) != HIPBLAS_STATUS_SUCCESS)
        return bad("hipblasLtMatmulDescSetAttribute");
    if (a.MatrixLayoutCreate(&p.lw, HIP_R_16BF, (uint64_t)K, (uint64_t)N, K) != HIPBLAS_STATUS_SUCCESS ||
        a.MatrixLayoutCreate(&p.lx, HIP_R_16BF, (uint64_t)K, (uint64_t)M, K) != HIPBLAS_STATUS_SUCCESS ||
        a.MatrixLayoutCreate(&p.ld, HIP_R_32F, (uint64_t)N, (uint64_t)M, ldd) != HIPBLAS_STATUS_SUCCESS)
        return bad("hipblasLtMatrixLayoutCreate");
    hipblasLtMatmulPreference_t pref = nullptr;
    if (a.MatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return bad("hipblasLtMatmulPreferenceCreate");
    uint64_t wsz = lt->workspace_bytes;
    hipblasLtMatmulHeuristicResult_t res[PF_LT_CANDIDATES];
    int got = 0;
    // (L2H_PF_LT_CANDIDATES: how many of the library's proposals to consider, 1 .. 4; 0 = none, which is how the path
    // "the library is there but has nothing for this product" is tested)
    int want = PF_LT_CANDIDATES;
    if (const char *e = getenv("L2H_PF_LT_CANDIDATES")) want = std::max(0, std::min(PF_LT_CANDIDATES, atoi(e)));
    const bool pref_ok = a.MatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &wsz, sizeof(wsz)) == HIPBLAS_STATUS_SUCCESS;
    const hipblasStatus_t st =
        pref_ok && want > 0 ? a.MatmulAlgoGetHeuristic(lt->handle, p.desc, p.lw, p.lx, p.ld, p.ld, pref, want, res, &got)
                            : HIPBLAS_STATUS_INTERNAL_ERROR;
    a.MatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || got < 1) return bad("hipBLASLt has no algorithm for this product");
    p.algo = res[0].algo;
    // Large products: time the candidates once on the real operands and a scratch result.
    if (got > 1 && M >= 128) {
        float *scratch = nullptr;
        if (hipMalloc(&scratch, (size_t)M * (size_t)ldd * sizeof(float)) == hipSuccess) {
            hipEvent_t e0 = nullptr, e1 = nullptr;
            if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess &&
                hipMemsetAsync(scratch, 0, (size_t)M * (size_t)ldd * sizeof(float), s) == hipSuccess) {
                const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
                // every candidate twice in turn (two runs to warm up, then five timed ones); a candidate's time is the
                // shorter of its two: a single short measurement now and then picks a tile that is 10 % slower
                float t_of[PF_LT_CANDIDATES];
                for (int c = 0; c < PF_LT_CANDIDATES; c++) t_of[c] = 0.0f;
                for (int round = 0; round < 2; round++)
                    for (int c = 0; c < got; c++) {
                        if (res[c].state != HIPBLAS_STATUS_SUCCESS || res[c].workspaceSize > lt->workspace_bytes) continue;
                        bool ok = true;
                        float ms = 0.0f;
                        for (int it = 0; it < 7 && ok; it++) {
                            if (it == 2) ok = hipEventRecord(e0, s) == hipSuccess;
                            ok = ok && a.Matmul(lt->handle, p.desc, &alpha, W, p.lw, X, p.lx, &beta, scratch, p.ld, scratch, p.ld,
                                                &res[c].algo, lt->workspace, lt->workspace_bytes, s) == HIPBLAS_STATUS_SUCCESS;
                        }
                        ok = ok && hipEventRecord(e1, s) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
                             hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
                        if (ok && (t_of[c] == 0.0f || ms < t_of[c])) t_of[c] = ms;
                    }
                float best = 0.0f;
                for (int c = 0; c < got; c++)
                    if (t_of[c] > 0.0f && (best == 0.0f || t_of[c] < best)) {
                        best = t_of[c];
                        p.algo = res[c].algo;
                    }
            }
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            (void)hipStreamSynchronize(s);
            (void)hipFree(scratch);
        }
        (void)hipGetLastError();
    }
    return true;
}

// D == nullptr: only finds (and keeps) the algorithm for the shape, so that a library that has none is noticed before
// anything has been computed with it
hipError_t pf_lt_gemm(PfLt *lt, hipStream_t s, const uint16_t *W, const uint16_t *X, float *D, int M, int64_t N, int64_t K,
                      int64_t ldd, bool accumulate, std::string *err) {
    if (!lt || M < 1 || N < 1 || K < 1 || ldd < N) return hipErrorInvalidValue;
    const auto key = std::make_tuple(M, N, K, ldd, accumulate);
    auto it = lt->plans.find(key);
    if (it == lt->plans.end()) {
        LtPlan p;
        if (!pf_lt_plan(lt, s, p, W, X, M, N, K, ldd, accumulate, err)) {
            if (p.lw) lt->api.MatrixLayoutDestroy(p.lw);
            if (p.lx) lt->api.MatrixLayoutDestroy(p.lx);
            if (p.ld) lt->api.MatrixLayoutDestroy(p.ld);
            if (p.desc) lt->api.MatmulDescDestroy(p.desc);
            return hipErrorNotSupported;
        }
        it = lt->plans.emplace(key, p).first;
    }
    if (!D) return hipSuccess;
    const LtPlan &p = it->second;
    const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
    const hipblasStatus_t st = lt->api.Matmul(lt->handle, p.desc, &alpha, W, p.lw, X, p.lx, &beta, D, p.ld, D, p.ld, &p.algo,
                                              lt->workspace, lt->workspace_bytes, s);
    if (st != HIPBLAS_STATUS_SUCCESS) {
        if (err) *err = "hipblasLtMatmul failed (status " + std::to_string((int)st) + ")";
        return hipErrorUnknown;
    }
    return hipSuccess;
}
