// Matrix products y = x * W^T (+ bias) (ReLU) (+ residual) for activations
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

namespace st {

// ---------------------------------------------------------------- generic tiled
// 64x64 output tile per workgroup, 16-deep K steps through LDS, 4x4 outputs per
// thread.  Any M, N, K; any alignment.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, const TI* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int relu) {
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
            if (relu) v = fmaxf(v, 0.f);
            if (residual) v += residual[(int64_t)m * N + n];
            Elem<TO>::store(out + (int64_t)m * N + n, v);
        }
    }
}

template <typename TI, typename TO>
static int launch_tiled(void* out, const void* x, const void* w, const float* bias,
                        const float* residual, int M, int N, int K, int relu, hipStream_t stream) {
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    gemm_tiled_kernel<TI, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TI*)x, (const TI*)w, bias,
                                                       residual, M, N, K, relu);
    ST_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

int gemm_bf16_fast(void* out, const void* x, const void* w, const float* bias, const float* residual,
                   int M, int N, int K, int relu, int out_f32, hipStream_t stream, bool* handled);

}  // namespace st

using namespace st;

// dtype: storage type of x and W.  out_f32 != 0: the result is stored as float
// (residual stream, logits) whatever `dtype` is.  algo: 0 = best available,
// 1 = the generic tiled kernel (the plain one that the others are checked against).
extern "C" int st_gemm(void* out, const void* x, const void* w, const float* bias,
                       const float* residual, int M, int N, int K, int relu, int dtype,
                       int out_f32, int algo, hipStream_t stream) {
    ST_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    ST_CHECK(out && x && w, "gemm: null operand");
    if (M == 0) return 0;
    if (dtype == kF32) {
        return launch_tiled<float, float>(out, x, w, bias, residual, M, N, K, relu, stream);
    } else if (dtype == kBF16) {
        if (algo == 0) {
            bool handled = false;
            int rc = gemm_bf16_fast(out, x, w, bias, residual, M, N, K, relu, out_f32, stream, &handled);
            if (rc != 0 || handled) return rc;
        }
        if (out_f32) return launch_tiled<bf16_t, float>(out, x, w, bias, residual, M, N, K, relu, stream);
        return launch_tiled<bf16_t, bf16_t>(out, x, w, bias, residual, M, N, K, relu, stream);
    }
    ST_CHECK(false, "gemm: unknown dtype %d", dtype);
    return 0;
}
