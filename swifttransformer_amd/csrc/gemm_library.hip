// Products through hipBLASLt (bfloat16, and float with true 32-bit multiply-adds).
//
// The reference runs every product of the model through cuBLAS
// (src/csrc/util/cublas_wrapper.cc:29, cublasGemmStridedBatchedEx); the AMD counterpart of
// that library stands here for the shapes where it beats the hand-written kernels: more
// than 12 rows, or very large weight matrices at any row count (st_gemm decides).  Bias, ReLU and
// the residual sum still ride in the product (the library's epilogue and its beta*C term),
// so the residual stream is summed in float exactly as in the other kernels.
//
// y[M,N] = x[M,K] W[N,K]^T, all row-major.  Read column-major, y is an N x M matrix
// = op(A) op(B) with A = W (K x N, transposed) and B = x (K x M).
#include "common.h"
#include "api.h"

#include <hipblaslt/hipblaslt.h>
#include <map>
#include <mutex>
#include <tuple>

namespace st {

namespace {

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr, d = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool usable = false;
    bool tuned = false;      // chosen by timing the candidates rather than by the library's order
};

using PlanKey = std::tuple<int, int, int, int, int, int, int, int>;   // M N K relu bias residual out_f32 dtype

struct Library {
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    std::map<PlanKey, Plan> plans;
    std::mutex mutex;
    bool failed = false;
    bool tuning = false;     // products issued now have their candidates timed (st_gemm_library_tuning)
    void* flush = nullptr;   // overwritten between timed runs so that they meet their weights in memory
};

Library& library() {
    static Library lib;
    return lib;
}

constexpr size_t kWorkspaceBytes = 64u << 20;
bool g_allow_workspace = false;
constexpr size_t kMaxPlans = 4096;     // beyond this many shapes the table starts over
constexpr size_t kFlushBytes = 384u << 20;   // more than the 256 MB memory-side cache

void free_plan(Plan& p) {
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    for (hipblasLtMatrixLayout_t l : {p.a, p.b, p.c, p.d})
        if (l) hipblasLtMatrixLayoutDestroy(l);
    p = Plan();
}

bool ok(hipblasStatus_t s) { return s == HIPBLAS_STATUS_SUCCESS; }

// one-time set-up; on failure the library is marked unusable and the caller's own kernels run
bool ensure_library(Library& lib) {
    if (lib.failed) return false;
    if (lib.handle) return true;
    if (!ok(hipblasLtCreate(&lib.handle)) ||
        hipMalloc(&lib.workspace, kWorkspaceBytes) != hipSuccess) {
        lib.failed = true;
        return false;
    }
    lib.workspace_bytes = kWorkspaceBytes;
    return true;
}

// What a timing run of the candidates needs: the caller's operands (read only) and its stream.
struct TuneArgs {
    const void* x; const void* w; const float* bias; const float* residual; hipStream_t stream;
};

// Times the library's candidate kernels for a plan on the caller's operands (into a scratch
// result) and returns the index of the fastest.  Only called outside stream capture.
// In the step these products meet their weights in memory, not in a cache (a model's weights
// are many times the 256 MB memory-side cache), so between two timed runs a buffer larger
// than that cache is overwritten: run back to back, the candidates would race on cached
// weights, and the winner of that race is not the fastest in the step.
int pick_fastest(Library& lib, Plan& p, const hipblasLtMatmulHeuristicResult_t* found, int n_found, int fallback,
                 int M, int N, int K, bool bias, bool residual, bool out_f32, int dtype, const TuneArgs& t) {
    constexpr int kRuns = 5;
    const size_t out_bytes = (size_t)M * N * ((out_f32 || dtype == kF32) ? 4 : 2);
    void* scratch = nullptr;
    void* flush = lib.flush;
    if (hipMalloc(&scratch, out_bytes) != hipSuccess) return fallback;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        hipFree(scratch);
        return fallback;
    }
    if (bias) {
        const void* bp = t.bias;
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp));
    }
    const float alpha = 1.f, beta = residual ? 1.f : 0.f;
    const void* c = residual ? (const void*)t.residual : (const void*)scratch;
    int best = fallback;
    float best_ms = 1e30f;
    for (int i = 0; i < n_found; ++i) {
        // Candidates that keep partial results in a workspace stay out: these plans are for
        // recorded steps, and what the library does to such a workspace between launches (a
        // clearing memset node would be one thing) is not this file's to know.  Of ~150
        // candidates seen for a model's shapes six wanted one; leaving them out costs <2 %.
        if (found[i].workspaceSize > 0) continue;
        bool good = true;
        float total = 0.f;
        for (int rep = 0; rep <= kRuns && good; ++rep) {         // the first run is not counted
            if (flush) hipMemsetAsync(flush, rep, kFlushBytes, t.stream);
            hipEventRecord(e0, t.stream);
            good = ok(hipblasLtMatmul(lib.handle, p.desc, &alpha, t.w, p.a, t.x, p.b, &beta, c, p.c, scratch, p.d,
                                      &found[i].algo, lib.workspace, found[i].workspaceSize, t.stream));
            hipEventRecord(e1, t.stream);
            float ms = 0.f;
            if (hipEventSynchronize(e1) != hipSuccess) { good = false; break; }
            hipEventElapsedTime(&ms, e0, e1);
            if (rep > 0) total += ms;
        }
        if (!good) continue;
        if (total < best_ms) { best_ms = total; best = i; }
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(scratch);
    return best;
}

Plan make_plan(Library& lib, int M, int N, int K, bool relu, bool bias, bool residual, bool out_f32, int dtype,
               bool tune, const TuneArgs& tune_args) {
    Plan p;
    const hipDataType in_t = dtype == kF32 ? HIP_R_32F : HIP_R_16BF;
    const hipDataType out_t = (out_f32 || dtype == kF32) ? HIP_R_32F : HIP_R_16BF;
    // HIPBLAS_COMPUTE_32F: float accumulation, and for float operands plain 32-bit multiply-adds
    // (the reduced-precision float mode is a different compute type and is never asked for)
    if (!ok(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F))) return p;
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta));
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb));
    hipblasLtEpilogue_t ep = HIPBLASLT_EPILOGUE_DEFAULT;
    if (bias && relu) ep = HIPBLASLT_EPILOGUE_RELU_BIAS;
    else if (bias) ep = HIPBLASLT_EPILOGUE_BIAS;
    else if (relu) ep = HIPBLASLT_EPILOGUE_RELU;
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep));
    if (bias) {
        const int32_t bias_t = HIP_R_32F;
        if (!ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_t,
                                                sizeof(bias_t))))
            return p;
    }
    if (!ok(hipblasLtMatrixLayoutCreate(&p.a, in_t, K, N, K)) ||      // W as K x N, ld K
        !ok(hipblasLtMatrixLayoutCreate(&p.b, in_t, K, M, K)) ||      // x as K x M, ld K
        !ok(hipblasLtMatrixLayoutCreate(&p.c, out_t, N, M, N)) ||
        !ok(hipblasLtMatrixLayoutCreate(&p.d, out_t, N, M, N)))
        return p;
    hipblasLtMatmulPreference_t pref = nullptr;
    if (!ok(hipblasLtMatmulPreferenceCreate(&pref))) return p;
    // Only kernels that need no workspace are asked for: any product may end up in a recorded
    // step (a plan made outside a recording is used inside one later), and what the library does
    // to a workspace between launches (a clearing memset node would be one thing) is not this
    // file's to know.  g_allow_workspace lifts that for measurements.
    const size_t max_workspace = g_allow_workspace ? lib.workspace_bytes : 0;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                          &max_workspace, sizeof(max_workspace));
    constexpr int kCandidates = 32;
    hipblasLtMatmulHeuristicResult_t found[kCandidates];
    int n_found = 0;
    const int want = tune ? kCandidates : 1;
    const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(lib.handle, p.desc, p.a, p.b, p.c, p.d,
                                                              pref, want, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    (void)residual;
    if (!ok(s) || n_found < 1) return p;
    int best = -1;
    for (int i = 0; i < n_found && best < 0; ++i)
        if (found[i].workspaceSize <= lib.workspace_bytes) best = i;
    if (best < 0) return p;
    if (tune) {                                      // the fall-back too, if there is one without
        for (int i = 0; i < n_found; ++i)
            if (found[i].workspaceSize == 0) { best = i; break; }
    }
    if (tune && n_found > 1) best = pick_fastest(lib, p, found, n_found, best, M, N, K, bias, residual, out_f32, dtype, tune_args);
    p.algo = found[best].algo;
    p.workspace = found[best].workspaceSize;
    p.usable = true;
    p.tuned = tune;
    return p;
}

}  // namespace

// Runs the product in the library if it has a kernel for it; *handled says whether it did.
// Combinations the library's epilogue does not express in this engine's order (ReLU before
// the residual sum, a residual into a bfloat16 result) are left to the caller's kernels.
int gemm_library(void* out, const void* x, const void* w, const float* bias, const float* residual,
                 int M, int N, int K, int relu, int out_f32, int dtype, hipStream_t stream, bool* handled) {
    *handled = false;
    if (relu != 0 && relu != 1) return 0;            // `relu` is the activation's number: none or ReLU here
    if ((relu && residual) || (residual && !out_f32 && dtype != kF32)) return 0;
    if (K % 8 != 0 || N % 8 != 0) return 0;
    Library& lib = library();
    std::lock_guard<std::mutex> guard(lib.mutex);
    if (!ensure_library(lib)) return 0;
    const PlanKey key(M, N, K, relu ? 1 : 0, bias ? 1 : 0, residual ? 1 : 0, out_f32 ? 1 : 0, dtype);
    auto it = lib.plans.find(key);
    if (it == lib.plans.end() && lib.plans.size() >= kMaxPlans) {
        // a server that has seen this many row counts keeps only those it meets from now on;
        // products already queued hold their kernels' arguments themselves
        for (auto& kv : lib.plans) free_plan(kv.second);
        lib.plans.clear();
        it = lib.plans.end();
    }
    // The few row counts of recorded decode steps come back at every step: while such a step is
    // being prepared (st_gemm_library_tuning) the library's candidates are timed for its
    // products, once (of 32 candidates on weights from memory: batch 32 10,700 -> 11,500
    // tokens/s, batch 64 15,000 -> 15,700, batch 256 20,800 -> 21,700).  Prompt-sized products
    // gain nothing over the library's first suggestion (the fastest of 48 for each of a layer's
    // four products at 2,048 rows), and timing costs ~20 ms a shape, too much for row counts
    // that come and go.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
    const bool tune = lib.tuning && !capturing;
    if (it != lib.plans.end() && tune && it->second.usable && !it->second.tuned) {
        free_plan(it->second);                       // made in passing before: chosen properly now
        lib.plans.erase(it);
        it = lib.plans.end();
    }
    if (it == lib.plans.end()) {
        const TuneArgs targs{x, w, bias, residual, stream};
        it = lib.plans.emplace(key, make_plan(lib, M, N, K, relu, bias != nullptr, residual != nullptr,
                                              out_f32 != 0, dtype, tune, targs)).first;
    }
    Plan& p = it->second;
    if (!p.usable) return 0;
    if (bias) {
        const void* bp = bias;
        if (!ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp))))
            return 0;
    }
    const float alpha = 1.f, beta = residual ? 1.f : 0.f;
    const void* c = residual ? (const void*)residual : (const void*)out;
    const hipblasStatus_t s = hipblasLtMatmul(lib.handle, p.desc, &alpha, w, p.a, x, p.b, &beta, c, p.c,
                                              out, p.d, &p.algo, lib.workspace, p.workspace, stream);
    ST_CHECK(ok(s), "gemm: hipblasLtMatmul failed with status %d (M=%d N=%d K=%d)", (int)s, M, N, K);
    *handled = true;
    return 0;
}

}  // namespace st

// Creates the library handle and its workspace now rather than inside the first product,
// which may be issued while a stream is being captured (no allocation is allowed there).
// Returns 1 if the library is usable.
// on != 0: from now on every library product issued outside stream capture has its candidate
// kernels timed on its own operands, once per shape, and keeps the fastest; on == 0: back to
// the library's first suggestion for shapes not met yet.  Meant to bracket the preparation of
// a step that will be replayed many times.
extern "C" int st_gemm_library_tuning(int on) {
    st::Library& lib = st::library();
    std::lock_guard<std::mutex> guard(lib.mutex);
    if (!st::ensure_library(lib)) return 0;
    lib.tuning = on != 0;
    if (lib.tuning && !lib.flush) {
        if (hipMalloc(&lib.flush, st::kFlushBytes) != hipSuccess) {
            (void)hipGetLastError();                 // no room: the candidates race on warm weights
            lib.flush = nullptr;
        }
    } else if (!lib.tuning && lib.flush) {
        hipFree(lib.flush);
        lib.flush = nullptr;
    }
    return 1;
}

// on != 0: plans made from now on may use the library's kernels that need a workspace (for
// measurements; such plans must not be used in recorded steps).
extern "C" int st_gemm_library_allow_workspace(int on) {
    st::Library& lib = st::library();
    std::lock_guard<std::mutex> guard(lib.mutex);
    st::g_allow_workspace = on != 0;
    return 0;
}

extern "C" int st_gemm_library_init() {
    st::Library& lib = st::library();
    std::lock_guard<std::mutex> guard(lib.mutex);
    return st::ensure_library(lib) ? 1 : 0;
}
