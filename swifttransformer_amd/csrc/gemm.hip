// Matrix products y = x * W^T (+ bias) (activation) (+ residual) for activations
// x[M,K] and weights W[N,K] stored [out, in] as in the weight files.
//
// The reference calls cuBLAS for its five products (QKV src/csrc/layer/attention.cc:102-111,
// out :255-264, FC1/FC2 src/csrc/layer/ffn.cc:71-80, :96-105, LM head
// src/csrc/model/gpt/gpt.cc:192-201) and runs bias, activation and residual as
// separate kernels (src/csrc/kernel/addbias.cu:23, :72,
// src/csrc/kernel/fused_addbias_activ.cu:26-45).  Here they are the epilogue of
// the product.  Accumulation is always in float; with float operands every
// multiply-add is a true 32-bit FMA.
#include "common.h"
#include "api.h"
#include "gemm_extras.h"
#include "activation.h"

#include <atomic>

namespace st {

static std::atomic<uint64_t> g_path_counts[kNumGemmPaths];
void count_gemm_path(int path) {
    if (path >= 0 && path < kNumGemmPaths) g_path_counts[path].fetch_add(1, std::memory_order_relaxed);
}

// ---------------------------------------------------------------- generic tiled
// 64x64 output tile per workgroup, 16-deep K steps through LDS, 4x4 outputs per
// thread.  Any M, N, K; any alignment.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, const TI* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int act, const StGemmExtras ex) {
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float xs[BK][BM + 4];
    __shared__ float ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tr = tid / 16, tc = tid % 16;   // thread's 4x4 block: rows tr*4.., cols tc*4..
    float acc[4][4] = {};
    // loading: thread loads 4 consecutive k of one row: row = tid / 4, k = (tid % 4) * 4
    const int lr = tid / 4, lk = (tid % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int mr = m0 + lr, nr = n0 + lr;
            xs[lk + i][lr] = (mr < M && k < K) ? Elem<TI>::load(x + (int64_t)mr * K + k) : 0.f;
            ws[lk + i][lr] = (nr < N && k < K) ? Elem<TI>::load(w + (int64_t)nr * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = xs[k][tr * 4 + i]; b[i] = ws[k][tc * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tr * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tc * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[n];
            v = apply_activation(act, v);
            if (residual) v += residual[(int64_t)m * N + n];
            Elem<TO>::store(out + (int64_t)m * N + n, v);
            if (ex.k_cache && n >= ex.q_size) {
                int which;
                const int64_t dst = kv_scatter_offset(ex, m, n, &which);
                if (dst >= 0) Elem<TO>::store((TO*)(which ? ex.v_cache : ex.k_cache) + dst, v);
            }
        }
    }
}

template <typename TI, typename TO>
static int launch_tiled(void* out, const void* x, const void* w, const float* bias,
                        const float* residual, int M, int N, int K, int act,
                        const StGemmExtras& ex, hipStream_t stream) {
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    gemm_tiled_kernel<TI, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TI*)x, (const TI*)w, bias,
                                                       residual, M, N, K, act, ex);
    ST_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

int gemm_bf16_fast(void* out, const void* x, const void* w, const float* bias, const float* residual,
                   int M, int N, int K, int act, int out_f32, const StGemmExtras& ex,
                   hipStream_t stream, bool* handled);
bool gemm_bf16_can_fuse_norm(int M, int N, int K);
bool gemm_bf16_can_fuse_merge(int M, int N, int K, int splits, int heads, int head_dim);
bool gemm_wide_offered(int M, int N, int K);
int gemm_wide_groups();
int gemm_wide(float* out, const bf16_t* x, const bf16_t* w, const float* bias, int M, int N, int K,
              const StGemmExtras& ex, hipStream_t stream);
int gemm_library(void* out, const void* x, const void* w, const float* bias, const float* residual,
                 int M, int N, int K, int act, int out_f32, int dtype, hipStream_t stream, bool* handled);

// Float products always go to the library when it has a kernel (the float kernel here is the
// plain tiled one).  For bfloat16:
// from this many rows on the vendor library's kernels are faster than the hand-written ones
// (measured on 2048..8192-wide products: 30 us against 67 us for a layer's four products at
// 24 rows, 220 us against 390 us at 2048; in a recorded decode step of a 24-layer model of
// width 2048, with the library's kernels chosen by timing: 13 rows 6,630 against 6,440
// tokens/s, 16 rows 7,680 against 7,240); up to 12 rows the resident-slab kernel with its
// fused norm and cache write wins (12 rows 6,030 against 6,000, 8 rows 4,850 against 4,730).
// A product that takes the norm as its prologue is the resident kernel's at any row count it
// accepts (up to 16): the caller decides that (at width 2048 it pays up to 16 rows).
constexpr int kLibraryMinRows = 13;
static std::atomic<int> g_library_min_rows{kLibraryMinRows};
// With fewer rows the library still wins on large, deep matrices (decode of the 30B shape at
// batch 8: 456 against 408 tokens/s), while on 2048-deep ones its launches cost more inside a
// recorded step than its kernels save (3,935 against 4,214 tokens/s; the 50272 x 2048 head
// takes 50 us there against 44 us here).  The limits between them were fitted in recorded decode
// steps at the layer sizes of OPT-2.7B, 6.7B and 13B (24 Mi weights, 2,560 deep against 40 Mi
// and 4,096: batch 8 at the 2.7B sizes 2,515 against 2,356 tokens/s, at the 13B sizes 909
// against 884, the same at the 6.7B sizes).
constexpr int64_t kLibraryMinWeights = 24ll << 20;
constexpr int kLibraryMinDepth = 2560;
static std::atomic<int64_t> g_library_min_weights{kLibraryMinWeights};
static std::atomic<int> g_library_min_depth{kLibraryMinDepth};

}  // namespace st

using namespace st;

// dtype: storage type of x and W.  out_f32 != 0: the result is stored as float
// (residual stream, logits) whatever `dtype` is.  algo: 0 = best available,
// 1 = the generic tiled kernel (the plain one that the others are checked against),
// 2 = the vendor library (an error if it has no kernel for the shape),
// 3 = the hand-written matrix-core kernels whatever the number of rows.
// extras: optional fused work (see gemm_extras.h), or null.
extern "C" int st_gemm(void* out, const void* x, const void* w, const float* bias,
                       const float* residual, int M, int N, int K, int activation, int dtype,
                       int out_f32, int algo, const StGemmExtras* extras, hipStream_t stream) {
    ST_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    ST_CHECK(activation_known(activation), "gemm: activation %d has no kernel (0 none, 1 ReLU, 2 SiLU, "
             "3 GELU in its tanh form)", activation);
    const int act = activation;
    StGemmExtras ex = {};
    if (extras) ex = *extras;
    ST_CHECK(out && w && (x || ex.ln_x || ex.mg_o), "gemm: null operand");
    if (ex.k_cache) {
        ST_CHECK(ex.v_cache && ex.token_item && ex.positions && ex.block_table, "gemm: K/V scatter lacks an operand");
        ST_CHECK(ex.head_dim > 0 && ex.kv_size % ex.head_dim == 0 && ex.q_size >= 0 &&
                 ex.q_size + 2 * ex.kv_size == N && ex.page_size > 0 && ex.max_pages > 0 && ex.head_dim % 4 == 0,
                 "gemm: K/V scatter sizes do not match the product (N=%d q=%d kv=%d)", N, ex.q_size, ex.kv_size);
        ST_CHECK(!out_f32 || dtype == kF32, "gemm: K/V scatter stores the storage type");
        ST_CHECK(!act && !residual, "gemm: K/V scatter goes with a plain product");
    }
    if (M == 0) return 0;
    // the persistent kernel for a few rows and a very wide matrix: float results of a plain product
    const bool wide_can = dtype == kBF16 && out_f32 && !residual && act == 0 && !ex.k_cache && !ex.mg_o &&
                          (algo == 0 || algo == 3) && K % 8 == 0 && gemm_wide_offered(M, N, K) &&
                          ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                            reinterpret_cast<uintptr_t>(ex.ln_x) | reinterpret_cast<uintptr_t>(ex.ln_gamma) |
                            reinterpret_cast<uintptr_t>(ex.ln_beta) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (ex.ln_x) {
        ST_CHECK(dtype == kBF16 && algo == 0 && (wide_can || (!ex.ln_rows && gemm_bf16_can_fuse_norm(M, N, K))),
                 "gemm: no kernel fuses the norm%s for M=%d N=%d K=%d dtype=%d", ex.ln_rows ? " of picked rows" : "",
                 M, N, K, dtype);
        ST_CHECK(ex.ln_eps > 0.f, "gemm: norm eps must be positive");
    }
    ST_CHECK(!ex.ln_rows || ex.ln_x, "gemm: a row index without a norm prologue");
    ST_CHECK(!ex.best_ids || wide_can, "gemm: no kernel finds the rows' best outputs for M=%d N=%d K=%d dtype=%d "
             "(float results of a plain bfloat16 product of few rows with a very wide matrix only)", M, N, K, dtype);
    // (with neither fusion asked for, the rule below still sends large deep matrices to the library)
    if (wide_can && (ex.ln_x || ex.best_ids || (M < g_library_min_rows &&
            !((int64_t)N * K >= g_library_min_weights && K >= g_library_min_depth)))) {
        const int rc = gemm_wide((float*)out, (const bf16_t*)x, (const bf16_t*)w, bias, M, N, K, ex, stream);
        if (rc == 0) count_gemm_path(kPathWide);
        return rc;
    }
    if (ex.mg_o) {
        ST_CHECK(ex.mg_lse && !ex.ln_x && dtype == kBF16 && algo == 0 &&
                 gemm_bf16_can_fuse_merge(M, N, K, ex.mg_splits, ex.mg_heads, ex.mg_head_dim),
                 "gemm: no kernel merges %d splits of %d heads for M=%d N=%d K=%d dtype=%d", ex.mg_splits,
                 ex.mg_heads, M, N, K, dtype);
    }
    // The library's epilogues serve no function but ReLU: another one is applied in place by the
    // elementwise kernel after the library's product (a product with a residual sum cannot be
    // split like that and stays with the kernels here).
    const bool in_epilogue = activation_in_library(act);
    const bool library_can = in_epilogue || !residual;
    ST_CHECK(algo != 2 || library_can, "gemm: the library path has no activation %d before a residual sum", act);
    const bool to_library = algo == 2 || (algo == 0 && !ex.ln_x && !ex.mg_o && library_can &&
        (dtype == kF32 || M >= g_library_min_rows ||
         ((int64_t)N * K >= g_library_min_weights && K >= g_library_min_depth)));
    if (to_library && (dtype == kF32 || dtype == kBF16)) {
        bool handled = false;
        int rc = gemm_library(out, x, w, bias, residual, M, N, K, in_epilogue ? act : 0, out_f32, dtype, stream, &handled);
        if (rc != 0) return rc;
        ST_CHECK(handled || algo != 2, "gemm: the library has no kernel for M=%d N=%d K=%d", M, N, K);
        if (handled) {
            count_gemm_path(kPathLibrary);
            if (!in_epilogue) {
                rc = st_activation_multiply(out, N, out, N, nullptr, 0, M, N, act,
                                            (out_f32 || dtype == kF32) ? kF32 : kBF16, stream);
                if (rc != 0) return rc;
            }
            if (!ex.k_cache) return 0;
            const size_t es = dtype == kF32 ? 4 : 2;
            const char* o = (const char*)out;
            return st_kv_write(ex.k_cache, ex.v_cache, ex.page_stride, o + es * ex.q_size,
                               o + es * (ex.q_size + ex.kv_size), N, ex.token_item, ex.positions,
                               ex.block_table, ex.max_pages, ex.page_size, M,
                               ex.kv_size / ex.head_dim, ex.head_dim, dtype, stream);
        }
    }
    if (dtype == kF32) {
        count_gemm_path(kPathGenericF32);
        return launch_tiled<float, float>(out, x, w, bias, residual, M, N, K, act, ex, stream);
    } else if (dtype == kBF16) {
        if (algo == 0 || algo == 3) {
            bool handled = false;
            int rc = gemm_bf16_fast(out, x, w, bias, residual, M, N, K, act, out_f32, ex, stream, &handled);
            if (rc != 0 || handled) return rc;
            ST_CHECK(!ex.ln_x && !ex.mg_o, "gemm: the prologue could not be fused");
        }
        count_gemm_path(kPathGenericBf16);
        if (out_f32) return launch_tiled<bf16_t, float>(out, x, w, bias, residual, M, N, K, act, ex, stream);
        return launch_tiled<bf16_t, bf16_t>(out, x, w, bias, residual, M, N, K, act, ex, stream);
    }
    ST_CHECK(false, "gemm: unknown dtype %d", dtype);
    return 0;
}

// The rule by which bfloat16 products go to the vendor library: from `min_rows` rows on, and below
// that for matrices of at least `min_weights` elements that are at least `min_depth` deep.  -1
// leaves a setting as it is, -2 puts the fitted default back.  For measurements and tests: the rule
// is read when a product is issued, so a step recorded earlier keeps the kernels it was recorded
// with until it is recorded again.
extern "C" int st_gemm_library_rule(int min_rows, int64_t min_weights, int min_depth) {
    if (min_rows >= 0) g_library_min_rows = min_rows;
    else if (min_rows == -2) g_library_min_rows = kLibraryMinRows;
    if (min_weights >= 0) g_library_min_weights = min_weights;
    else if (min_weights == -2) g_library_min_weights = kLibraryMinWeights;
    if (min_depth >= 0) g_library_min_depth = min_depth;
    else if (min_depth == -2) g_library_min_depth = kLibraryMinDepth;
    return 0;
}

// Calls of st_gemm per kernel family since the last reset (order of st::GemmPath); returns the
// number of families.  `out` may be null.
extern "C" int st_gemm_path_counts(uint64_t* out, int reset) {
    for (int i = 0; i < kNumGemmPaths; ++i) {
        const uint64_t v = reset ? g_path_counts[i].exchange(0) : g_path_counts[i].load();
        if (out) out[i] = v;
    }
    return kNumGemmPaths;
}

// Whether st_gemm (algo 0) can take a split attention output (partials and log-sum-exps) as its input.
extern "C" int st_gemm_can_fuse_merge(int M, int N, int K, int splits, int heads, int head_dim, int dtype) {
    return dtype == kBF16 && gemm_bf16_can_fuse_merge(M, N, K, splits, heads, head_dim) ? 1 : 0;
}

// Whether st_gemm (algo 0) can take its input through a fused LayerNorm for this shape.
extern "C" int st_gemm_can_fuse_norm(int M, int N, int K, int dtype) {
    return dtype == kBF16 && gemm_bf16_can_fuse_norm(M, N, K) ? 1 : 0;
}

// Whether st_gemm (algo 0) runs a float-result product of this shape in the persistent kernel for
// very wide matrices, which takes the norm of picked rows as its prologue and finds the rows' best
// outputs; and how many workgroups that kernel runs (16 scratch entries each for the best outputs).
extern "C" int st_gemm_wide_offered(int M, int N, int K, int dtype) {
    return dtype == kBF16 && K % 8 == 0 && gemm_wide_offered(M, N, K) ? 1 : 0;
}
extern "C" int st_gemm_wide_groups() { return gemm_wide_groups(); }
