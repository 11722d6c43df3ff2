// bfloat16 matrix products on the matrix cores: y = x * W^T (+bias)(ReLU)(+residual),
// x[M,K], W[N,K] both contiguous along K, float accumulation.
//
// Two kernels, both with W as the MFMA "A" operand (rows = output features n) and x
// as the "B" operand (columns = tokens m), so that a lane ends up with four
// consecutive n of one token and stores them as one vector:
//   * skinny (M <= 64, decoding): v_mfma_f32_16x16x32_bf16, operands straight from
//     global memory (W is read exactly once, x comes from cache); a workgroup owns 16
//     or 32 output features, its 4..16 waves split K and sum through LDS, so that a
//     weight matrix of a few MB still has thousands of waves loading at once;
//   * tiled (any M): 128x128 tiles through LDS, v_mfma_f32_32x32x16_bf16.
// The lane -> k assignment inside one MFMA is the same for both operands, so the sum
// over k does not depend on which k values a lane holds.
//
// Reference: cuBLAS calls with half accumulation (src/csrc/util/cublas_wrapper.h:141-144)
// followed by separate bias/activation/residual kernels (src/csrc/layer/ffn.cc:85-92,
// src/csrc/kernel/addbias.cu:23-37).
#include "common.h"
#include "api.h"

namespace st {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ inline bf16x8 load8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8 zero8() {
    return __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
}

// epilogue for 4 consecutive n (n0..n0+3) of token m
template <bool OUT_F32>
__device__ inline void store4(void* out, const float* bias, const float* residual, int relu,
                              int m, int n0, int N, floatx4 v) {
    float r[4] = {v[0], v[1], v[2], v[3]};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int n = n0 + i;
        if (n < N) {
            if (bias) r[i] += bias[n];
            if (relu) r[i] = fmaxf(r[i], 0.f);
            if (residual) r[i] += residual[(int64_t)m * N + n];
        }
    }
    if (n0 + 3 < N && (N & 3) == 0) {
        if (OUT_F32) {
            *reinterpret_cast<float4*>((float*)out + (int64_t)m * N + n0) = make_float4(r[0], r[1], r[2], r[3]);
        } else {
            uint2 p;
            p.x = (uint32_t)float_to_bf16(r[0]) | ((uint32_t)float_to_bf16(r[1]) << 16);
            p.y = (uint32_t)float_to_bf16(r[2]) | ((uint32_t)float_to_bf16(r[3]) << 16);
            *reinterpret_cast<uint2*>((bf16_t*)out + (int64_t)m * N + n0) = p;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + i;
            if (n < N) {
                if (OUT_F32) ((float*)out)[(int64_t)m * N + n] = r[i];
                else ((bf16_t*)out)[(int64_t)m * N + n].bits = float_to_bf16(r[i]);
            }
        }
    }
}

// ------------------------------------------------------------------------ skinny
// One workgroup owns 16*NT output features and all of K; its WAVES waves split K and
// add their partial tiles through LDS (a tree, no traffic between workgroups: their
// L2s are not shared across the chip's XCDs).  grid = ceil(N / (16*NT)).
// K % 8 == 0; kw (k per wave) % 64 == 0.
template <int MT, int NT, int WAVES, bool OUT_F32>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    void* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int relu, int kw) {
    extern __shared__ floatx4 red[];                 // [WAVES/2][MT*NT][64]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, r16 = lane & 15;
    const int n_base = blockIdx.x * (16 * NT);
    const int k_begin = wave * kw;
    const int k_end = min(K, k_begin + kw);
    const bf16_t* wrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)                  // rows past N are loaded (clamped) but never stored
        wrow[nt] = w + (int64_t)min(n_base + nt * 16 + r16, N - 1) * K;
    const bf16_t* xrow[MT];
    bool xvalid[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16;
        xvalid[mt] = m < M;
        xrow[mt] = x + (int64_t)(xvalid[mt] ? m : 0) * K;
    }
    floatx4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // a lane covers k = kk + 16g .. +15 of every 64-wide step: two MFMAs of 8 k each
    int k = k_begin;
#pragma unroll 4
    for (; k + 64 <= k_end; k += 64) {
        const int ko = k + g * 16;
        bf16x8 a[NT][2], b[MT][2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) { a[nt][0] = load8(wrow[nt] + ko); a[nt][1] = load8(wrow[nt] + ko + 8); }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            b[mt][0] = xvalid[mt] ? load8(xrow[mt] + ko) : zero8();
            b[mt][1] = xvalid[mt] ? load8(xrow[mt] + ko + 8) : zero8();
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][0], b[mt][0], acc[nt][mt], 0, 0, 0);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][1], b[mt][1], acc[nt][mt], 0, 0, 0);
            }
    }
    if (k < k_end) {   // fewer than 64 k left (K % 8 == 0): guarded 8-wide pieces
        const int ko = k + g * 16;
        const bool v0 = ko + 8 <= k_end, v1 = ko + 16 <= k_end;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const bf16x8 a0 = v0 ? load8(wrow[nt] + ko) : zero8(), a1 = v1 ? load8(wrow[nt] + ko + 8) : zero8();
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const bf16x8 b0 = (xvalid[mt] && v0) ? load8(xrow[mt] + ko) : zero8();
                const bf16x8 b1 = (xvalid[mt] && v1) ? load8(xrow[mt] + ko + 8) : zero8();
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc[nt][mt], 0, 0, 0);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, acc[nt][mt], 0, 0, 0);
            }
        }
    }

    // sum the waves' partial tiles: upper half parks, lower half adds, halving each round
#pragma unroll
    for (int half = WAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    red[((wave - half) * (MT * NT) + nt * MT + mt) * 64 + lane] = acc[nt][mt];
        }
        __syncthreads();
        if (wave < half) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] += red[(wave * (MT * NT) + nt * MT + mt) * 64 + lane];
        }
        __syncthreads();
    }
    if (wave != 0) return;
    // acc[nt][mt][r] = y[m = mt*16 + r16][n = n_base + nt*16 + 4g + r]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r16, n0 = n_base + nt * 16 + 4 * g;
            if (m < M && n0 < N) store4<OUT_F32>(out, bias, residual, relu, m, n0, N, acc[nt][mt]);
        }
}

// ------------------------------------------------------------------------- tiled
// 128 (n) x 128 (m) tile per workgroup, K steps of 64 through LDS.  A row of a tile in
// LDS is 64 bf16 = 8 chunks of 16 bytes; chunk c of row r is stored at chunk c ^ (r & 7)
// so that the 16-byte reads of an MFMA operand spread over the banks.
constexpr int TB = 128;      // tile edge
constexpr int TK = 64;       // K step

__device__ inline int swz(int row, int chunk) { return row * 8 + (chunk ^ (row & 7)); }

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_tiled_mfma_kernel(
    void* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int relu) {
    __shared__ uint4 sw[TB * 8];     // W tile: [n][k chunk]
    __shared__ uint4 sx[TB * 8];     // x tile: [m][k chunk]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;             // wave's 64x64 quadrant
    const int n0 = blockIdx.x * TB, m0 = blockIdx.y * TB;
    const int l32 = lane & 31, lh = lane >> 5;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    uint4 rw[4], rx[4];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = c & 7;
            const int k = k0 + kc * 8;
            const int n = n0 + row, m = m0 + row;
            rw[i] = (n < N && k < K) ? *reinterpret_cast<const uint4*>(w + (int64_t)n * K + k) : make_uint4(0, 0, 0, 0);
            rx[i] = (m < M && k < K) ? *reinterpret_cast<const uint4*>(x + (int64_t)m * K + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_lds = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = c & 7;
            sw[swz(row, kc)] = rw[i];
            sx[swz(row, kc)] = rx[i];
        }
    };

    load_global(0);
    for (int k0 = 0; k0 < K; k0 += TK) {
        __syncthreads();               // the previous step's readers are done
        store_lds();
        __syncthreads();
        if (k0 + TK < K) load_global(k0 + TK);
#pragma unroll
        for (int kk = 0; kk < TK / 16; ++kk) {
            const int chunk = kk * 2 + lh;
            bf16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = __builtin_bit_cast(bf16x8, sw[swz(wn * 64 + i * 32 + l32, chunk)]);
                b[i] = __builtin_bit_cast(bf16x8, sx[swz(wm * 64 + i * 32 + l32, chunk)]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    // acc[i][j][e]: n = n0 + wn*64 + i*32 + 8*(e/4) + 4*lh + e%4,  m = m0 + wm*64 + j*32 + l32
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = m0 + wm * 64 + j * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * 64 + i * 32 + 8 * q + 4 * lh;
                if (n >= N) continue;
                const floatx4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                store4<OUT_F32>(out, bias, residual, relu, m, n, N, v);
            }
        }
}

template <int MT, int NT, int WAVES>
static void launch_skinny(void* out, const bf16_t* x, const bf16_t* w, const float* bias,
                          const float* residual, int M, int N, int K, int relu, int out_f32,
                          hipStream_t stream) {
    const int kw = ((K + WAVES - 1) / WAVES + 63) & ~63;
    const dim3 grid((N + 16 * NT - 1) / (16 * NT));
    const size_t lds = (size_t)(WAVES / 2) * MT * NT * 64 * sizeof(floatx4);
    if (out_f32)
        gemm_skinny_kernel<MT, NT, WAVES, true><<<grid, WAVES * 64, lds, stream>>>(out, x, w, bias, residual,
                                                                                  M, N, K, relu, kw);
    else
        gemm_skinny_kernel<MT, NT, WAVES, false><<<grid, WAVES * 64, lds, stream>>>(out, x, w, bias, residual,
                                                                                   M, N, K, relu, kw);
}

int gemm_bf16_fast(void* out, const void* x, const void* w, const float* bias, const float* residual,
                   int M, int N, int K, int relu, int out_f32, hipStream_t stream, bool* handled) {
    *handled = false;
    if (K % 8 != 0) return 0;                       // 16-byte operand loads need K % 8 == 0
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return 0;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    if (M <= 64) {
        // waves per workgroup: at least 128 k each
        if (M <= 16) {
            if (K >= 2048) launch_skinny<1, 1, 16>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
            else if (K >= 1024) launch_skinny<1, 1, 8>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
            else launch_skinny<1, 1, 4>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
        } else if (M <= 32) {
            if (K >= 1024) launch_skinny<2, 2, 8>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
            else launch_skinny<2, 2, 4>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
        } else {
            if (K >= 1024) launch_skinny<4, 2, 8>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
            else launch_skinny<4, 2, 4>(out, xb, wb, bias, residual, M, N, K, relu, out_f32, stream);
        }
        ST_LAUNCH_CHECK("gemm_skinny");
        *handled = true;
        return 0;
    }
    dim3 grid((N + TB - 1) / TB, (M + TB - 1) / TB);
    if (out_f32)
        gemm_tiled_mfma_kernel<true><<<grid, 256, 0, stream>>>(out, xb, wb, bias, residual, M, N, K, relu);
    else
        gemm_tiled_mfma_kernel<false><<<grid, 256, 0, stream>>>(out, xb, wb, bias, residual, M, N, K, relu);
    ST_LAUNCH_CHECK("gemm_tiled_mfma");
    *handled = true;
    return 0;
}

}  // namespace st

extern "C" int st_attn_prefill(void* out, const void* q, int64_t q_stride,
                    const void* k_cache, const void* v_cache, int64_t page_stride,
                    const int* tile_item, const int* tile_q0, int num_tiles,
                    const int* item_tok_off, const int* item_start, const int* item_len,
                    const int* block_table, int max_pages, int page_size,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window,
                    int dtype, hipStream_t stream) {
    st::set_error("attn_prefill: not built");
    return 1;
}

extern "C" int st_has_attn_prefill() { return 0; }
