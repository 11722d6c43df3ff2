// bfloat16 matrix products on the matrix cores: y = x * W^T (+bias)(ReLU)(+residual),
// x[M,K], W[N,K] both contiguous along K, float accumulation.
//
// Three kernels, all with W as the MFMA "A" operand (rows = output features n) and x
// as the "B" operand (columns = tokens m), so that a lane ends up with four
// consecutive n of one token and stores them as one vector:
//   * skinny resident (M <= 16, decoding): v_mfma_f32_16x16x32_bf16; a workgroup owns 16
//     (or 8, or with the norm prologue 24 or 32) output features, each of its waves loads its
//     whole K slab of W into registers at once, the waves' partial tiles are summed through
//     LDS; its input rows come from memory as stored, or through a prologue into LDS:
//     LayerNorm of the float rows, the merge of a decode attention still split over the keys
//     (up to 8 splits of 4 rows, or 2 splits of 16 rows), or a plain staging copy;
//   * skinny (M <= 64): the same split of K over the waves of a workgroup, W and x fetched
//     step by step, two 16-feature tiles per workgroup;
//   * tiled (any M): 128x128 tiles through LDS, v_mfma_f32_32x32x16_bf16.
// The lane -> k assignment inside one MFMA is the same for both operands, so the sum
// over k does not depend on which k values a lane holds.
//
// Reference: cuBLAS calls with half accumulation (src/csrc/util/cublas_wrapper.h:141-144)
// followed by separate bias/activation/residual kernels (src/csrc/layer/ffn.cc:85-92,
// src/csrc/kernel/addbias.cu:23-37).
#include "common.h"
#include "api.h"
#include "gemm_extras.h"
#include "activation.h"

#include <atomic>

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
__device__ inline void store4(void* out, const float* bias, const float* residual, int act,
                              int m, int n0, int N, floatx4 v, const StGemmExtras& ex) {
    float r[4] = {v[0], v[1], v[2], v[3]};
    if (bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n0 + i < N) r[i] += bias[n0 + i];
    }
    apply_activation4(act, r);
    if (residual) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n0 + i < N) r[i] += residual[(int64_t)m * N + n0 + i];
    }
    if (!OUT_F32 && ex.k_cache && n0 >= ex.q_size && n0 + 3 < N) {
        // four consecutive features of one key/value head (head_dim % 4 == 0, n0 % 4 == 0)
        int which;
        const int64_t dst = kv_scatter_offset(ex, m, n0, &which);
        if (dst >= 0) {
            uint2 p;
            p.x = pack_bf16x2(r[0], r[1]);
            p.y = pack_bf16x2(r[2], r[3]);
            *reinterpret_cast<uint2*>((bf16_t*)(which ? ex.v_cache : ex.k_cache) + dst) = p;
        }
    }
    if (n0 + 3 < N && (N & 3) == 0) {
        if (OUT_F32) {
            *reinterpret_cast<float4*>((float*)out + (int64_t)m * N + n0) = make_float4(r[0], r[1], r[2], r[3]);
        } else {
            uint2 p;
            p.x = pack_bf16x2(r[0], r[1]);
            p.y = pack_bf16x2(r[2], r[3]);
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
    int M, int N, int K, int act, int kw, const StGemmExtras ex) {
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
    auto xload = [&](int mt, int k) -> bf16x8 { return xvalid[mt] ? load8(xrow[mt] + k) : zero8(); };
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
            b[mt][0] = xload(mt, ko);
            b[mt][1] = xload(mt, ko + 8);
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
                const bf16x8 b0 = v0 ? xload(mt, ko) : zero8();
                const bf16x8 b1 = v1 ? xload(mt, ko + 8) : zero8();
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
            if (m < M && n0 < N) store4<OUT_F32>(out, bias, residual, act, m, n0, N, acc[nt][mt], ex);
        }
}

// ------------------------------------------------------- skinny, W slab in registers
// M <= 16.  A workgroup owns 16 output features; wave w owns k in [w*KSTEPS*64, +KSTEPS*64)
// and loads its whole slab of W (16 rows x KSTEPS*64 k) into registers with its first
// instructions, so every byte of W is in flight before anything waits.  With LN the
// workgroup meanwhile normalises the M input rows (float, from ex.ln_x) into LDS as
// bfloat16, and the x operand is read from there.
// With PRO == 2 the input is instead an attention output still split over the keys
// (ex.mg_o, ex.mg_lse): the workgroup merges the splits into LDS the same way (PRO == 4: the
// same for at most two splits, with registers for four times as many rows).  With PRO == 3
// the stored input rows are copied into LDS first (asked for before the W slab, so they arrive
// first): the K steps then read their x fragments from LDS instead of paying a trip to the L2
// each, one after the other.
// K % 8 == 0, K <= WAVES*KSTEPS*64; LN: K % 256 == 0 handled by guards, K <= 4096.
constexpr int kLnMaxVec = 16;            // float4 per lane of a row held in registers (K <= 4096)
constexpr int kMgElems = 2;              // merge prologue: float4 elements of the input per thread
constexpr int kMgSplits = 8;             // and splits per element, all held in registers;
constexpr int kMgElemsTwo = 8;           // or this many elements of at most two splits (PRO == 4: more rows)
constexpr int kMgMaxWeights = 2048;      // rows * heads * splits weights in LDS

template <int WAVES, int KSTEPS, bool OUT_F32, int PRO, int ROWS>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_resident_kernel(
    void* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int act, const StGemmExtras ex) {
    constexpr bool LN = PRO == 1, MG = PRO == 2 || PRO == 4, ST = PRO == 3;
    // merge prologue: elements of the input per thread x splits held in registers
    constexpr int MGE = PRO == 4 ? kMgElemsTwo : kMgElems, MGS = PRO == 4 ? 2 : kMgSplits;
    extern __shared__ uint4 dyn[];
    constexpr int NT = (ROWS + 15) / 16;                                   // 16-row MFMA tiles of W per workgroup
    floatx4* red = reinterpret_cast<floatx4*>(dyn);                       // [WAVES][NT][64]
    bf16_t* xs = nullptr;                                                  // [M][K + 8] input rows made here (LN, MG)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, r16 = lane & 15;
    // ROWS output features per workgroup.  8: half of each MFMA's rows stay empty, but a narrow
    // matrix (N = hidden) then spreads over twice as many compute units.  24 and 32 (two tiles):
    // a wide matrix then makes one workgroup a compute unit instead of one and a half or two,
    // and its prologue (the norm of all rows) is done half as often; with 16 waves the slabs of
    // two tiles are as long as those of one tile with 8, so as many bytes are in flight.
    const int n_base = blockIdx.x * ROWS;
    const int k_begin = wave * (KSTEPS * 64);
    bool wvalid[NT];
    const bf16_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        wvalid[t] = 16 * t + r16 < ROWS;
        wrow[t] = w + (int64_t)min(n_base + 16 * t + r16, N - 1) * K;
    }
    const int xstride = K + 8;

    // Loads return in order, so what is needed first is asked for first: the norm's gain and
    // bias (parked in LDS as soon as they arrive), the rows to normalise, then the W slab from
    // HBM, which stays in flight while the rows are normalised.
    constexpr int LNV = LN ? (WAVES * KSTEPS + 3) / 4 : 1;    // float4 per lane covering K <= WAVES*KSTEPS*64
    constexpr int GV = LN ? (LNV + WAVES - 1) / WAVES : 1;    // float4 per thread covering K
    const int nvec = K >> 2;
    float* sg = reinterpret_cast<float*>(dyn + WAVES * NT * 64);           // [K] gain   (LN only)
    float* sb = sg + K;                                               // [K] bias
    xs = reinterpret_cast<bf16_t*>(sb + K);
    float4 gv[GV], bv[GV];
    if (LN) {
#pragma unroll
        for (int i = 0; i < GV; ++i) {
            const int c = threadIdx.x + i * (WAVES * 64);
            gv[i] = (ex.ln_gamma && c < nvec) ? reinterpret_cast<const float4*>(ex.ln_gamma)[c]
                                              : make_float4(1.f, 1.f, 1.f, 1.f);
            bv[i] = (ex.ln_beta && c < nvec) ? reinterpret_cast<const float4*>(ex.ln_beta)[c]
                                             : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    // merge prologue: this thread's elements of every split, asked for before the W slab so that
    // they arrive first; the weights of the splits meanwhile go to LDS
    float4 mo[MG ? MGE : 1][MG ? MGS : 1];
    float* sw = sg;                                                   // [M * heads * splits] weights (MG only)
    if (MG) {
        xs = reinterpret_cast<bf16_t*>(sw + ((M * ex.mg_heads * ex.mg_splits + 3) & ~3));   // 16-byte aligned
        const int S = ex.mg_splits, hd4 = ex.mg_head_dim >> 2, total = M * nvec;
#pragma unroll
        for (int e = 0; e < MGE; ++e) {
            const int idx = threadIdx.x + e * (WAVES * 64);          // (row, float4 of K)
            const int m = idx / nvec, c = idx - m * nvec;
            const int head = c / hd4, d4 = c - head * hd4;
            const float4* po = reinterpret_cast<const float4*>(ex.mg_o) +
                               ((int64_t)(m * ex.mg_heads + head) * S) * hd4 + d4;
#pragma unroll
            for (int sp = 0; sp < MGS; ++sp)
                mo[e][sp] = (idx < total && sp < S) ? po[(int64_t)sp * hd4] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    // staged input: this thread's 16-byte pieces of the M rows
    constexpr int STV = 8;                                            // pieces per thread: M*K <= 8*8*threads
    uint4 sx[ST ? STV : 1];
    if (ST) {
        xs = reinterpret_cast<bf16_t*>(sg);
        const int pieces = K >> 3, total = M * pieces;
#pragma unroll
        for (int i = 0; i < STV; ++i) {
            const int idx = threadIdx.x + i * (WAVES * 64);
            const int m = idx / pieces, c = idx - m * pieces;
            sx[i] = idx < total ? *reinterpret_cast<const uint4*>(x + (int64_t)m * K + c * 8) : make_uint4(0, 0, 0, 0);
        }
    }
    float4 v[LNV];
    auto load_row = [&](int m) {
        const float* xr = ex.ln_x + (int64_t)m * K;
#pragma unroll
        for (int i = 0; i < LNV; ++i) {
            const int c = lane + i * 64;
            v[i] = c < nvec ? reinterpret_cast<const float4*>(xr)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    if (LN && wave < M) load_row(wave);
    bf16x8 a[NT][KSTEPS][2];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int ko = k_begin + s * 64 + g * 16;
            a[t][s][0] = (wvalid[t] && ko + 8 <= K) ? load8(wrow[t] + ko) : zero8();
            a[t][s][1] = (wvalid[t] && ko + 16 <= K) ? load8(wrow[t] + ko + 8) : zero8();
        }
    const bool xvalid = r16 < M;
    const bf16_t* xrow = x + (int64_t)(xvalid ? r16 : 0) * K;       // unused with LN, MG and ST
    if (ST) {
        const int pieces = K >> 3, total = M * pieces;
#pragma unroll
        for (int i = 0; i < STV; ++i) {
            const int idx = threadIdx.x + i * (WAVES * 64);
            if (idx < total) {
                const int m = idx / pieces, c = idx - m * pieces;
                *reinterpret_cast<uint4*>(xs + (int64_t)m * xstride + c * 8) = sx[i];
            }
        }
        __syncthreads();
        xrow = xs + (int64_t)(xvalid ? r16 : 0) * xstride;
    }
    if (MG) {
        const int S = ex.mg_splits, groups = M * ex.mg_heads;
        for (int gidx = threadIdx.x; gidx < groups; gidx += WAVES * 64) {
            const float* lse = ex.mg_lse + (int64_t)gidx * S;
            float ls[MGS], mx = -INFINITY;
#pragma unroll
            for (int sp = 0; sp < MGS; ++sp) {
                ls[sp] = sp < S ? lse[sp] : -INFINITY;
                mx = fmaxf(mx, ls[sp]);
            }
            float wsum = 0.f;
#pragma unroll
            for (int sp = 0; sp < MGS; ++sp) {
                ls[sp] = ls[sp] > -INFINITY ? __expf(ls[sp] - mx) : 0.f;
                wsum += ls[sp];
            }
            const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
#pragma unroll
            for (int sp = 0; sp < MGS; ++sp)
                if (sp < S) sw[gidx * S + sp] = ls[sp] * inv;
        }
        __syncthreads();
        const int hd4 = ex.mg_head_dim >> 2, total = M * nvec;
#pragma unroll
        for (int e = 0; e < MGE; ++e) {
            const int idx = threadIdx.x + e * (WAVES * 64);
            if (idx >= total) continue;
            const int m = idx / nvec, c = idx - m * nvec;
            const float* wg = sw + (m * ex.mg_heads + c / hd4) * S;
            float y0 = 0.f, y1 = 0.f, y2 = 0.f, y3 = 0.f;
#pragma unroll
            for (int sp = 0; sp < MGS; ++sp) {
                if (sp < S) {
                    const float ww = wg[sp];
                    y0 = fmaf(ww, mo[e][sp].x, y0); y1 = fmaf(ww, mo[e][sp].y, y1);
                    y2 = fmaf(ww, mo[e][sp].z, y2); y3 = fmaf(ww, mo[e][sp].w, y3);
                }
            }
            uint2 p;
            p.x = pack_bf16x2(y0, y1);
            p.y = pack_bf16x2(y2, y3);
            *reinterpret_cast<uint2*>(xs + (int64_t)m * xstride + c * 4) = p;
        }
        __syncthreads();
        xrow = xs + (int64_t)(xvalid ? r16 : 0) * xstride;
    }
    if (LN) {
#pragma unroll
        for (int i = 0; i < GV; ++i) {
            const int c = threadIdx.x + i * (WAVES * 64);
            if (c < nvec) {
                reinterpret_cast<float4*>(sg)[c] = gv[i];
                reinterpret_cast<float4*>(sb)[c] = bv[i];
            }
        }
        // rows beyond the first of a wave (M > WAVES) are loaded when their turn comes
        float mean = 0.f, rstd = 0.f;
        bool first = true;
        for (int m = wave; m < M; m += WAVES) {
            if (!first) load_row(m);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < LNV; ++i) sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
            mean = ex.ln_no_center ? 0.f : wave_sum(sum) / (float)K;
            float sq = 0.f;
#pragma unroll
            for (int i = 0; i < LNV; ++i) {
                if (lane + i * 64 < nvec) {
                    const float p = v[i].x - mean, q = v[i].y - mean, r = v[i].z - mean, t = v[i].w - mean;
                    sq += (p * p + q * q) + (r * r + t * t);
                }
            }
            rstd = 1.0f / sqrtf(wave_sum(sq) / (float)K + ex.ln_eps);
            if (first) __syncthreads();              // gain and bias are in LDS (every wave passes here once)
            first = false;
#pragma unroll
            for (int i = 0; i < LNV; ++i) {
                const int c = lane + i * 64;
                if (c >= nvec) continue;
                const float4 gm = reinterpret_cast<const float4*>(sg)[c];
                const float4 bt = reinterpret_cast<const float4*>(sb)[c];
                const float y0 = (v[i].x - mean) * rstd * gm.x + bt.x, y1 = (v[i].y - mean) * rstd * gm.y + bt.y;
                const float y2 = (v[i].z - mean) * rstd * gm.z + bt.z, y3 = (v[i].w - mean) * rstd * gm.w + bt.w;
                uint2 p;
                p.x = pack_bf16x2(y0, y1);
                p.y = pack_bf16x2(y2, y3);
                *reinterpret_cast<uint2*>(xs + (int64_t)m * xstride + c * 4) = p;
            }
        }
        if (first) __syncthreads();                  // waves without a row still meet the others
        __syncthreads();
        xrow = xs + (int64_t)(xvalid ? r16 : 0) * xstride;
    }
    // x fragments are fetched step by step (from cache or LDS): loads return in order, so they
    // queue behind the W slab already in flight and need no registers until then
    floatx4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
        const int ko = k_begin + s * 64 + g * 16;
        const bf16x8 b0 = (xvalid && ko + 8 <= K) ? load8(xrow + ko) : zero8();
        const bf16x8 b1 = (xvalid && ko + 16 <= K) ? load8(xrow + ko + 8) : zero8();
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][s][0], b0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][s][1], b1, acc[t], 0, 0, 0);
        }
    }
    // the waves' partial tiles meet in LDS (a slot per wave and tile); one barrier, then wave t sums tile t
#pragma unroll
    for (int t = 0; t < NT; ++t)
        if (wave != t) red[(wave * NT + t) * 64 + lane] = acc[t];
    __syncthreads();
    if (wave >= NT) return;
    floatx4 sum = acc[0];
#pragma unroll
    for (int t = 1; t < NT; ++t)
        if (wave == t) sum = acc[t];
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
        if (wv != wave) sum += red[(wv * NT + wave) * 64 + lane];
    const int n0 = n_base + 16 * wave + 4 * g;
    if (r16 < M && 16 * wave + 4 * g < ROWS && n0 < N) store4<OUT_F32>(out, bias, residual, act, r16, n0, N, sum, ex);
}

// ------------------------------------------------------------------------- tiled
// 128 (n) x 128 (m) tile per workgroup, K steps of 64 through LDS.  A row of a tile in
// LDS is 64 bf16 = 8 chunks of 16 bytes; chunk c of row r is stored at chunk c ^ ((r/2) & 7)
// so that the 16-byte reads of an MFMA operand spread over the banks.
constexpr int TB = 128;      // tile edge
constexpr int TK = 64;       // K step

// A 16-byte LDS access is served 16 lanes at a time over 64 banks (16 units of 16 bytes): rows r
// and r+2 of a 128-byte-row tile share their units, so the chunk is rotated by row/2.
__device__ inline int swz(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }

// NI = 32-row W subtiles per wave: 2 -> workgroup tile 128 (n) x 128 (m), 4 -> 256 x 128.  With 4 a
// wave does 8 MFMAs for 6 operand reads instead of 4 for 4, which relieves the LDS.
template <int NI, bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_tiled_mfma_kernel(
    void* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ residual,
    int M, int N, int K, int act, const StGemmExtras ex) {
    constexpr int TN = 64 * NI;      // n extent of the workgroup tile
    __shared__ uint4 sw[TN * 8];     // W tile: [n][k chunk]
    __shared__ uint4 sx[TB * 8];     // x tile: [m][k chunk]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;             // wave's (32*NI) x 64 part
    const int n0 = blockIdx.x * TN, m0 = blockIdx.y * TB;
    const int l32 = lane & 31, lh = lane >> 5;

    floatx16 acc[NI][2];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    uint4 rw[2 * NI], rx[4];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2 * NI; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = c & 7;
            const int k = k0 + kc * 8, n = n0 + row;
            rw[i] = (n < N && k < K) ? *reinterpret_cast<const uint4*>(w + (int64_t)n * K + k) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = c & 7;
            const int k = k0 + kc * 8, m = m0 + row;
            rx[i] = (m < M && k < K) ? *reinterpret_cast<const uint4*>(x + (int64_t)m * K + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_lds = [&]() {
#pragma unroll
        for (int i = 0; i < 2 * NI; ++i) {
            const int c = tid + i * 256;
            sw[swz(c >> 3, c & 7)] = rw[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256;
            sx[swz(c >> 3, c & 7)] = rx[i];
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
            bf16x8 a[NI], b[2];
#pragma unroll
            for (int i = 0; i < NI; ++i)
                a[i] = __builtin_bit_cast(bf16x8, sw[swz(wn * (32 * NI) + i * 32 + l32, chunk)]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j] = __builtin_bit_cast(bf16x8, sx[swz(wm * 64 + j * 32 + l32, chunk)]);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    // acc[i][j][e]: n = n0 + wn*32*NI + i*32 + 8*(e/4) + 4*lh + e%4,  m = m0 + wm*64 + j*32 + l32
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = m0 + wm * 64 + j * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * (32 * NI) + i * 32 + 8 * q + 4 * lh;
                if (n >= N) continue;
                const floatx4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                store4<OUT_F32>(out, bias, residual, act, m, n, N, v, ex);
            }
        }
}

template <int MT, int NT, int WAVES>
static void launch_skinny(void* out, const bf16_t* x, const bf16_t* w, const float* bias,
                          const float* residual, int M, int N, int K, int act, int out_f32,
                          const StGemmExtras& ex, hipStream_t stream) {
    const int kw = ((K + WAVES - 1) / WAVES + 63) & ~63;
    const dim3 grid((N + 16 * NT - 1) / (16 * NT));
    const size_t lds = (size_t)(WAVES / 2) * MT * NT * 64 * sizeof(floatx4);
#define ST_SK(F32)                                                                                    \
    gemm_skinny_kernel<MT, NT, WAVES, F32><<<grid, WAVES * 64, lds, stream>>>(out, x, w, bias, residual, \
                                                                             M, N, K, act, kw, ex)
    if (out_f32) ST_SK(true); else ST_SK(false);
#undef ST_SK
}

// 16 waves leave 128 registers a lane (enough for a W slab of 8 steps); with the norm the row
// held for the statistics needs more, so that variant runs 8 waves with slabs twice as long
constexpr int kResidentWaves = 16;
constexpr int kResidentWavesLn = 8;
constexpr size_t kMaxLds = 156 * 1024;     // of the 160 KB a gfx950 CU has

static size_t resident_lds(int waves, int M, int K, int pro, int mg_weights = 0, int tiles = 0) {
    if (tiles == 0) tiles = pro == 1 ? 2 : 1;     // only the norm variant has workgroups of two tiles
    size_t n = (size_t)waves * tiles * 64 * sizeof(floatx4);
    if (pro == 1) n += (size_t)2 * K * sizeof(float) + (size_t)M * (K + 8) * sizeof(bf16_t);
    if (pro == 2 || pro == 4) n += (size_t)((mg_weights + 3) & ~3) * sizeof(float) + (size_t)M * (K + 8) * sizeof(bf16_t);
    if (pro == 3) n += (size_t)M * (K + 8) * sizeof(bf16_t);
    return n;
}

// The resident skinny kernel merges a split attention output itself when every thread can hold
// its share of the partial results in registers.  Which of its merge prologues takes the shape:
// 2 (up to kMgSplits splits), 4 (two splits, four times the rows), 0 none.
static int merge_prologue(int M, int N, int K, int splits, int heads, int head_dim) {
    // (K beyond four steps a wave: the slab and the partial results no longer fit a lane's 128
    // registers together, and the spills cost more than the merge kernel: 52 us against 15 us + 5
    // for the 5120 x 5120 output projection of the OPT-13B shape)
    if (!(M >= 1 && M <= 16 && splits >= 2 && heads > 0 && head_dim % 8 == 0 && heads * head_dim == K &&
          K % 8 == 0 && K <= kResidentWaves * 4 * 64 && M * heads * splits <= kMgMaxWeights &&
          resident_lds(kResidentWaves, M, K, 2, M * heads * splits) <= kMaxLds)) return 0;
    const int64_t elems = (int64_t)M * (K / 4), threads = kResidentWaves * 64;
    if (splits <= kMgSplits && elems <= kMgElems * threads) return 2;
    // (the two-split form with its 64 registers of partial results: two steps a wave at most; at the
    // OPT-6.7B sizes, K = 4096, it spilled and lost 5 % of a step to the merge kernel + library product)
    if (splits <= 2 && elems <= kMgElemsTwo * threads && K <= kResidentWaves * 2 * 64) return 4;
    return 0;
}

bool gemm_bf16_can_fuse_merge(int M, int N, int K, int splits, int heads, int head_dim) {
    return merge_prologue(M, N, K, splits, heads, head_dim) != 0;
}

// The resident skinny kernel normalises its input itself when the rows fit its registers and LDS.
bool gemm_bf16_can_fuse_norm(int M, int N, int K) {
    return M <= 16 && K % 8 == 0 && K <= kLnMaxVec * 256 && K <= kResidentWavesLn * 8 * 64 &&
           resident_lds(kResidentWavesLn, M, K, 1) <= kMaxLds;
}

template <int WAVES, int KSTEPS, bool OUT_F32, int PRO, int ROWS>
static int launch_resident(void* out, const bf16_t* x, const bf16_t* w, const float* bias,
                           const float* residual, int M, int N, int K, int act,
                           const StGemmExtras& ex, hipStream_t stream) {
    auto kernel = gemm_skinny_resident_kernel<WAVES, KSTEPS, OUT_F32, PRO, ROWS>;
    const size_t lds = resident_lds(WAVES, M, K, PRO, M * ex.mg_heads * ex.mg_splits, (ROWS + 15) / 16);
    if (lds > 48 * 1024) {
        static bool raised = false;     // once per instantiation: allow more than the default dynamic LDS
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
            ST_CHECK(e == hipSuccess, "gemm: cannot raise the LDS limit: %s", hipGetErrorString(e));
            raised = true;
        }
    }
    kernel<<<dim3((N + ROWS - 1) / ROWS), WAVES * 64, lds, stream>>>(out, x, w, bias, residual, M, N, K, act, ex);
    ST_LAUNCH_CHECK("gemm_skinny_resident");
    return 0;
}

constexpr int kWideModeDefault = 3;
static std::atomic<int> g_wide_mode{kWideModeDefault};              // bits: 1 wide workgroups for the norm variant, 2 sixteen waves for them (and 32 features), 4 see below

static int compute_units() { return device_compute_units(); }

// Only the instances whose slabs, rows and partial results fit a lane's registers exist (the others
// would spill: 1,024 threads leave 128 registers a lane, 512 threads 256):
//  * K steps a wave: 2 with the norm prologue and 16 waves and with the two-split merge prologue,
//    4 with the other merge prologue, else 8;
//  * two tiles (24 or 32 features) with the norm prologue: up to 2 steps (16 waves) or 4 (8 waves),
//    32 features with 16 waves only; with 16 waves there is no one-tile instance.
template <int WAVES, int PRO>
constexpr int resident_max_ksteps() {
    return ((PRO == 1 && WAVES == 16) || PRO == 4) ? 2 : PRO == 2 ? 4 : 8;
}

// wide_rows: 0, or 24 / 32 features a workgroup (norm prologue only; see ln_workgroup_shape)
template <int WAVES, int KS, bool F32, int PRO>
static int launch_resident_rows(void* out, const bf16_t* x, const bf16_t* w, const float* bias,
                                const float* residual, int M, int N, int K, int act,
                                const StGemmExtras& ex, hipStream_t stream, int wide_rows, bool narrow) {
#define ST_ROWS_ARGS out, x, w, bias, residual, M, N, K, act, ex, stream
    if constexpr (PRO == 1) {
        if constexpr (KS <= (WAVES == 16 ? 2 : 4)) {
            if constexpr (WAVES == 16) {
                if (wide_rows == 32) return launch_resident<WAVES, KS, F32, 1, 32>(ST_ROWS_ARGS);
            }
            if (wide_rows == 24) return launch_resident<WAVES, KS, F32, 1, 24>(ST_ROWS_ARGS);
        }
        if constexpr (WAVES == 16) {
            ST_CHECK(false, "gemm: no instance of %d features a workgroup with 16 waves", wide_rows);
            return -1;
        } else {
            ST_CHECK(wide_rows == 0, "gemm: no instance of %d features a workgroup for K=%d", wide_rows, K);
            return launch_resident<WAVES, KS, F32, 1, 16>(ST_ROWS_ARGS);
        }
    } else {
        if (narrow) return launch_resident<WAVES, KS, F32, PRO, 8>(ST_ROWS_ARGS);
        return launch_resident<WAVES, KS, F32, PRO, 16>(ST_ROWS_ARGS);
    }
#undef ST_ROWS_ARGS
}

template <int WAVES, int PRO>
static int launch_resident_k(void* out, const bf16_t* x, const bf16_t* w, const float* bias,
                             const float* residual, int M, int N, int K, int act, int out_f32,
                             const StGemmExtras& ex, hipStream_t stream, int wide_rows = 0) {
    const int ksteps = (K + WAVES * 64 - 1) / (WAVES * 64);
    constexpr int kMax = resident_max_ksteps<WAVES, PRO>();
    ST_CHECK(ksteps <= kMax, "gemm: K=%d is too deep for this instance of the resident kernel", K);
    // tiles of 16 features for fewer than about three quarters of the compute units (200 of 256)
    // would leave the others idle: tiles of 8 then
    const bool narrow = PRO != 1 && (N + 15) / 16 < compute_units() * 25 / 32;
#define ST_RES(KS)                                                                                                 \
    (out_f32 ? launch_resident_rows<WAVES, KS, true, PRO>(out, x, w, bias, residual, M, N, K, act, ex, stream, wide_rows, narrow) \
             : launch_resident_rows<WAVES, KS, false, PRO>(out, x, w, bias, residual, M, N, K, act, ex, stream, wide_rows, narrow))
    if (ksteps <= 1) return ST_RES(1);
    if (ksteps <= 2) return ST_RES(2);
    if constexpr (kMax >= 4) {
        if (ksteps <= 4) return ST_RES(4);
    }
    if constexpr (kMax >= 8) return ST_RES(8);
    return -1;
#undef ST_RES
}

// Workgroup shape of a product with the norm prologue: (features a workgroup, waves).  Every
// workgroup normalises all rows, so fewer, larger workgroups do that less often, and a launch of
// one workgroup a compute unit is balanced where one and a half a unit is not.  Measured at 8
// rows (us a call in a chain, 256 units): N = 6144: 384 x 16 features 12.1, 256 x 24 features
// with 8 waves 10.8, 192 x 32 features with 16 waves 9.8, 256 x 24 features with 16 waves 9.7;
// N = 8192: 512 x 16 features 13.4, 256 x 32 features with 8 waves 13.3 (half the waves in
// flight), with 16 waves 10.8.  So: 24 or else 32 features where that makes between three
// quarters of and all the compute units' worth of workgroups, with 16 waves (a wave then
// normalises one row) where their partial sums fit LDS beside the rows.  (24 before 32: in
// recorded decode steps of 24 layers 895 against 887 tokens/s at batch 1, 6,130 against 6,010 at 12.)
static void ln_workgroup_shape(int M, int N, int K, int* rows, int* waves) {
    const int units = compute_units();
    *rows = 0;
    *waves = kResidentWavesLn;
    const int mode = g_wide_mode.load(std::memory_order_relaxed);
    if (!(mode & 1)) return;
    // 16 waves leave 128 registers a lane: room for a slab of two K steps of two tiles beside the
    // row being normalised, not for more (K <= 2048)
    const bool sixteen = (mode & 2) && K <= 16 * 2 * 64 && resident_lds(16, M, K, 1) <= kMaxLds;
    if (K > 2048) return;                           // two tiles of longer slabs do not fit the registers
    for (int i = 0; i < 2; ++i) {
        const int r = ((mode & 4) != 0) == (i == 0) ? 32 : 24;      // bit 4: 32 before 24
        if (r == 32 && !sixteen) continue;          // 32 features with 8 waves are no gain
        if (N % r == 0 && N / r <= units && N / r >= units * 3 / 4) {
            *rows = r;
            *waves = sixteen ? 16 : kResidentWavesLn;
            return;
        }
    }
}

int gemm_bf16_fast(void* out, const void* x, const void* w, const float* bias, const float* residual,
                   int M, int N, int K, int act, int out_f32, const StGemmExtras& ex,
                   hipStream_t stream, bool* handled) {
    *handled = false;
    if (K % 8 != 0) return 0;                       // 16-byte operand loads need K % 8 == 0
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(ex.ln_x) |
         reinterpret_cast<uintptr_t>(ex.ln_gamma) | reinterpret_cast<uintptr_t>(ex.ln_beta)) & 15) return 0;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    if (ex.ln_x && !gemm_bf16_can_fuse_norm(M, N, K)) return 0;
    if (ex.mg_o && (ex.ln_x || ((reinterpret_cast<uintptr_t>(ex.mg_o) | reinterpret_cast<uintptr_t>(ex.mg_lse)) & 15) ||
                    !gemm_bf16_can_fuse_merge(M, N, K, ex.mg_splits, ex.mg_heads, ex.mg_head_dim))) return 0;
    if (M <= 16 && K <= kResidentWaves * 8 * 64) {
        // the stored rows go through LDS when they fit it and the threads' registers
        const bool staged = (int64_t)M * K <= (int64_t)8 * 8 * kResidentWaves * 64 && K > kResidentWaves * 64 &&
                            resident_lds(kResidentWaves, M, K, 3) <= kMaxLds;
        int ln_rows = 0, ln_waves = kResidentWavesLn;
        if (ex.ln_x) ln_workgroup_shape(M, N, K, &ln_rows, &ln_waves);
        const int rc = ex.ln_x
            ? (ln_waves == 16
                   ? launch_resident_k<16, 1>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream, ln_rows)
                   : launch_resident_k<kResidentWavesLn, 1>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream, ln_rows))
            : ex.mg_o
            ? (merge_prologue(M, N, K, ex.mg_splits, ex.mg_heads, ex.mg_head_dim) == 4
                   ? launch_resident_k<kResidentWaves, 4>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream)
                   : launch_resident_k<kResidentWaves, 2>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream))
            : staged
            ? launch_resident_k<kResidentWaves, 3>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream)
            : launch_resident_k<kResidentWaves, 0>(out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream);
        *handled = rc == 0;
        if (rc == 0) count_gemm_path(ex.ln_x ? kPathResidentNorm : ex.mg_o ? kPathResidentMerge : staged ? kPathResidentStaged : kPathResident);
        return rc;
    }
    if (ex.ln_x) return 0;
    if (M <= 64) {
        // waves per workgroup: at least 128 k each
#define ST_ARGS out, xb, wb, bias, residual, M, N, K, act, out_f32, ex, stream
        if (M <= 16) {
            if (K >= 2048) launch_skinny<1, 1, 16>(ST_ARGS);
            else if (K >= 1024) launch_skinny<1, 1, 8>(ST_ARGS);
            else launch_skinny<1, 1, 4>(ST_ARGS);
        } else if (M <= 32) {
            if (K >= 1024) launch_skinny<2, 2, 8>(ST_ARGS);
            else launch_skinny<2, 2, 4>(ST_ARGS);
        } else {
            if (K >= 1024) launch_skinny<4, 2, 8>(ST_ARGS);
            else launch_skinny<4, 2, 4>(ST_ARGS);
        }
#undef ST_ARGS
        ST_LAUNCH_CHECK("gemm_skinny");
        count_gemm_path(M <= 16 ? kPathSkinny16 : M <= 32 ? kPathSkinny32 : kPathSkinny64);
        *handled = true;
        return 0;
    }
    if (ex.ln_x) return 0;
    // (A 256-wide tile, NI = 4, needs 269 registers a lane: one wave per SIMD, and then nothing
    // hides a step's loads and barriers; measured 130 us against 74 us on 2048 x 6144 x 2048.
    // The 128-wide tile runs three workgroups per compute unit.)
    dim3 grid((N + TB - 1) / TB, (M + TB - 1) / TB);
    if (out_f32)
        gemm_tiled_mfma_kernel<2, true><<<grid, 256, 0, stream>>>(out, xb, wb, bias, residual, M, N, K, act, ex);
    else
        gemm_tiled_mfma_kernel<2, false><<<grid, 256, 0, stream>>>(out, xb, wb, bias, residual, M, N, K, act, ex);
    ST_LAUNCH_CHECK("gemm_tiled_mfma");
    count_gemm_path(kPathTiledMfma);
    *handled = true;
    return 0;
}

}  // namespace st


// Which wide workgroup shapes products with the norm prologue may take (for measurements): bit 1
// any, bit 2 those of 32 features and 16 waves; a negative value puts the default back.  Read when
// a product is issued: a recorded step keeps the shapes it was recorded with.
extern "C" int st_gemm_wide_workgroups(int on) {
    st::g_wide_mode = on < 0 ? st::kWideModeDefault : on;
    return 0;
}
