// Plain matrix products of many rows, handed to the vendor library (hipBLASLt) without a detour through
// another framework's dispatcher: out[M, N] = a[M, K] . w[N, K]^T, bfloat16 in, bfloat16 or float out, 32-bit sums.
// (The reference hands its projections to cuBLAS the same way, src/minillm/cuda/matrix.cpp:11-37.)
//
// Row-major out[M, N] is the column-major N x M matrix w^T(as stored: K x N, ld K)^T . a(as stored: K x M,
// ld K).  The library's choice of algorithm for a shape is looked up once and kept; the caller brings the
// workspace (the same for every call, so that calls on one stream may follow each other without clearing it).
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {
struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};
hipblasLtHandle_t g_handle = nullptr;
std::map<std::tuple<int, int, int, size_t, int>, Plan> g_plans;
std::mutex g_mutex;

int make_plan(int M, int N, int K, size_t workspace_bytes, int out_float, Plan& p) {
    if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return -10;
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) != HIPBLAS_STATUS_SUCCESS)
        return -11;
    if (hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, K) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, K) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.c, out_float ? HIP_R_32F : HIP_R_16BF, N, M, N) != HIPBLAS_STATUS_SUCCESS)
        return -12;
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return -13;
    const uint64_t ws = workspace_bytes;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
    // the library's candidates in the order of its own estimate; the first whose scratch memory fits
    constexpr int CANDIDATES = 8;
    hipblasLtMatmulHeuristicResult_t results[CANDIDATES];
    int found = 0;
    const hipblasStatus_t st =
        hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, CANDIDATES, results, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || found < 1) return -14;
    int pick = -1;
    for (int i = 0; i < found && pick < 0; ++i)
        if (results[i].state == HIPBLAS_STATUS_SUCCESS && results[i].workspaceSize <= workspace_bytes) pick = i;
    if (pick < 0) return -15;
    p.algo = results[pick].algo;
    p.workspace = results[pick].workspaceSize;
    return 0;
}
}  // namespace

// Returns 0, or a negative number that names the library call that failed (-1: bad sizes, -2: no handle,
// -10 .. -15: setting up the product, -20: the product itself).
extern "C" int mlr_library_gemm(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                                void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return -1;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_handle == nullptr && hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) return -2;
    const auto key = std::make_tuple(M, N, K, workspace_bytes, out_float ? 1 : 0);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        Plan p;
        const int rc = make_plan(M, N, K, workspace_bytes, out_float, p);
        if (rc != 0) return rc;
        it = g_plans.emplace(key, p).first;
    }
    const Plan& p = it->second;
    const float one = 1.0f, zero = 0.0f;
    const hipblasStatus_t st = hipblasLtMatmul(g_handle, p.desc, &one, w, p.a, a, p.b, &zero, out, p.c, out, p.c,
                                               &p.algo, workspace, p.workspace, stream);
    return st == HIPBLAS_STATUS_SUCCESS ? 0 : -20;
}
