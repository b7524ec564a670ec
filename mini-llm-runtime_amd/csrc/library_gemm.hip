// Plain matrix products of many rows, handed to the vendor library (hipBLASLt) without a detour through
// another framework's dispatcher: out[M, N] = a[M, K] . w[N, K]^T, bfloat16 in, bfloat16 or float out, 32-bit sums.
// (The reference hands its projections to cuBLAS the same way, src/minillm/cuda/matrix.cpp:11-37.)
//
// Row-major out[M, N] is the column-major N x M matrix w^T(as stored: K x N, ld K)^T . a(as stored: K x M,
// ld K).  The algorithm for a shape is chosen once and kept: the library lists its candidates in the order of
// its own estimate (up to 32 are asked for), and the first call of a shape runs each of them on the caller's
// operands and keeps the fastest (the estimate is off by up to 2x at a few hundred rows and by 5-10 % on some
// large shapes; among 32 candidates instead of 8 the 0.6B sizes' products of 128 rows find one that is 15 %
// faster, for a quarter of a second more of timing in a server's first minute); only
// row counts that are likely to come again are timed, see below.  While the stream
// is being captured nothing can be timed; a shape that is first met there keeps the library's first candidate
// for good, so that a captured step and a later eager step of the same shape never use different algorithms
// (the engine runs every shape eagerly before it captures it).  The caller brings the workspace (the same for every
// call, so that calls on one stream may follow each other without clearing it).
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
    bool timed = false;  // the algorithm was chosen by measurement
    hipblasLtMatmulHeuristicResult_t candidates[32];
    int found = 0;
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
    constexpr int CANDIDATES = sizeof(p.candidates) / sizeof(p.candidates[0]);
    hipblasLtMatmulHeuristicResult_t results[CANDIDATES];
    int found = 0;
    const hipblasStatus_t st =
        hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, CANDIDATES, results, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || found < 1) return -14;
    for (int i = 0; i < found; ++i)
        if (results[i].state == HIPBLAS_STATUS_SUCCESS && results[i].workspaceSize <= workspace_bytes)
            p.candidates[p.found++] = results[i];
    if (p.found < 1) return -15;
    p.algo = p.candidates[0].algo;
    p.workspace = p.candidates[0].workspaceSize;
    return 0;
}

int g_tuning = 1;

// Runs every candidate on the caller's operands (each writes the same product into `out`) and keeps the
// fastest.  A candidate that fails is passed over.
void choose_by_time(Plan& p, const void* a, const void* w, void* out, void* workspace, size_t workspace_bytes,
                    hipStream_t stream) {
    p.timed = true;
    if (p.found < 2) return;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) {
        if (t0) (void)hipEventDestroy(t0);
        return;
    }
    const float one = 1.0f, zero = 0.0f;
    float best = 0.0f;
    int pick = -1;
    for (int i = 0; i < p.found; ++i) {
        const hipblasLtMatmulHeuristicResult_t& c = p.candidates[i];
        float fastest = 0.0f;
        bool ok = true;
        // One untimed run, then the fastest of three, each on cold caches (the workspace, which holds nothing
        // between calls, is overwritten first: 128 MB push the operands out of the L2 and most of the
        // last-level cache): in a model a weight is never in a cache when its product starts, and a
        // candidate that wins on cached operands can lose by a tenth there.
        for (int run = 0; run < 4 && ok; ++run) {
            if (run > 0 && workspace_bytes > 0 &&
                hipMemsetAsync(workspace, 0, workspace_bytes, stream) != hipSuccess)
                ok = false;
            if (ok && hipEventRecord(t0, stream) != hipSuccess) ok = false;
            if (ok && hipblasLtMatmul(g_handle, p.desc, &one, w, p.a, a, p.b, &zero, out, p.c, out, p.c, &c.algo,
                                      workspace, c.workspaceSize, stream) != HIPBLAS_STATUS_SUCCESS)
                ok = false;
            float ms = 0.0f;
            if (ok && (hipEventRecord(t1, stream) != hipSuccess || hipEventSynchronize(t1) != hipSuccess ||
                       hipEventElapsedTime(&ms, t0, t1) != hipSuccess))
                ok = false;
            if (ok && run > 0 && (fastest == 0.0f || ms < fastest)) fastest = ms;
        }
        if (ok && (pick < 0 || fastest < best)) {
            best = fastest;
            pick = i;
        }
    }
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    (void)hipGetLastError();
    if (pick >= 0) {
        p.algo = p.candidates[pick].algo;
        p.workspace = p.candidates[pick].workspaceSize;
    }
}
}  // namespace

// Whether the first call of a shape times the library's candidates (1, the default) or takes the first (0).
extern "C" void mlr_library_gemm_tuning(int on) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_tuning = on;
}

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
    Plan& p = it->second;
    // Row counts that come again (few rows: decoding batches are filled up to a few sizes; multiples of 64:
    // prompt portions) are worth the 8 x 4 launches; a mixed step's odd row count may never return.
    if (!p.timed && g_tuning && (M <= 64 || M % 64 == 0)) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone)
            choose_by_time(p, a, w, out, workspace, workspace_bytes, stream);
        else
            p.timed = true;        // chosen: the first candidate, which the graph now holds
    }
    const float one = 1.0f, zero = 0.0f;
    const hipblasStatus_t st = hipblasLtMatmul(g_handle, p.desc, &one, w, p.a, a, p.b, &zero, out, p.c, out, p.c,
                                               &p.algo, workspace, p.workspace, stream);
    return st == HIPBLAS_STATUS_SUCCESS ? 0 : -20;
}
