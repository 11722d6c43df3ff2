// The product of a few rows with a very wide matrix (an output head over a vocabulary):
// y[M, N] = x[M, K] W[N, K]^T (+ bias), M <= 16, float results, bfloat16 operands.
//
// One workgroup of 16 waves per compute unit stays for the whole product and walks over tiles of
// 16 output features.  The waves split K: each holds its part of a tile's 16 x K slab of W in
// registers as the MFMA "A" operand, and its part of the input rows as the "B" operand, which it
// fetches once (the rows do not change from tile to tile).  The slab of the tile after next is
// asked for before the current one is multiplied (three slabs in registers, two of them on their
// way), so that a compute unit always has more than a hundred KB of W in flight; the waves'
// partial tiles meet in LDS, where the first wave sums them while the others go on.
//
// Before the walk the workgroup makes its input rows in LDS, once: a plain copy of stored rows,
// or LayerNorm of float rows picked by an index (the wanted rows of a step: the norm before a
// head acts on those only).  After it, each workgroup knows the best score of every row among
// its tiles (the lowest index on ties); a second small kernel picks the best of the workgroups'
// candidates: greedy token choice without another pass over the logits.
//
// Reference: cuBLAS for the head (src/csrc/model/gpt/gpt.cc:192-201) after a LayerNorm of every
// row and a gather kernel (:175-189, src/csrc/kernel/gather_last_tokens.cu:24-37), and a kernel
// of its own for the argmax (src/csrc/kernel/findmax.cu:16-39).
#include "common.h"
#include "api.h"
#include "gemm_extras.h"

namespace st {

typedef __bf16 bf16x8w __attribute__((ext_vector_type(8)));
typedef float floatx4w __attribute__((ext_vector_type(4)));

constexpr int kWideWaves = 16;
constexpr int kWideMaxRows = 16;
constexpr int kWideLnVec = 8;                 // float4 per lane of a row being normalised: K <= 2048

__device__ inline bf16x8w wide_load8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8w, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8w wide_zero8() { return __builtin_bit_cast(bf16x8w, make_uint4(0, 0, 0, 0)); }

__device__ inline void better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

// KSTEPS: 64-deep steps of K a wave (K <= 16 * KSTEPS * 64).  BIAS: whether a bias is added (an
// instance of its own, so that the other has no load between its tiles that it would wait for
// with the slabs on their way).
template <int KSTEPS, bool BIAS>
__global__ __launch_bounds__(kWideWaves * 64) void gemm_wide_kernel(
    float* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, int M, int N, int K,
    const float* __restrict__ ln_x, const int* __restrict__ ln_rows, const float* __restrict__ ln_gamma,
    const float* __restrict__ ln_beta, float ln_eps, int ln_no_center,
    float* __restrict__ cand_val, int* __restrict__ cand_idx) {
    extern __shared__ uint4 dyn[];
    floatx4w* red = reinterpret_cast<floatx4w*>(dyn);                       // [2][waves][64] partial tiles
    bf16_t* xs = reinterpret_cast<bf16_t*>(dyn + 2 * kWideWaves * 64);      // [M][K + 8] input rows
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, r16 = lane & 15;
    const int xstride = K + 8;
    const int tiles = (N + 15) / 16;
    const int k_begin = wave * (KSTEPS * 64);

    // Every load of a slab is unconditional (a tile beyond the last reads the last one again, a
    // piece beyond K the last piece of the row, and is cleared after it has arrived): the compiler
    // then counts the loads in flight and waits for the current slab's only; behind a branch it
    // would wait for all of them, the slabs just asked for included.
    auto load_slab = [&](bf16x8w (&a)[KSTEPS][2], int tile) {
        const bf16_t* wrow = w + (int64_t)min(min(tile, tiles - 1) * 16 + r16, N - 1) * K;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            // (the first product of a step takes k = 8g .. 8g + 7 of its 64, the second the same of
            // the upper 32: a load instruction then reads 64 contiguous bytes of each of its 16 rows)
            const int ko = k_begin + s * 64 + g * 8;
            const bf16x8w lo = wide_load8(wrow + min(ko, K - 8));
            const bf16x8w hi = wide_load8(wrow + min(ko + 32, K - 8));
            a[s][0] = ko + 8 <= K ? lo : wide_zero8();
            a[s][1] = ko + 40 <= K ? hi : wide_zero8();
        }
    };
    // Loads return in the order they were asked for: first this wave's row to normalise (wave m
    // has row m; there are at most as many rows as waves), then the first two slabs, which are on
    // their way while the rows are made.
    const int nvec = K >> 2;
    float4 v[kWideLnVec];
    if (ln_x && wave < M) {
        const float* xr = ln_x + (int64_t)(ln_rows ? ln_rows[wave] : wave) * K;
#pragma unroll
        for (int i = 0; i < kWideLnVec; ++i) {
            const int c = lane + i * 64;
            v[i] = c < nvec ? reinterpret_cast<const float4*>(xr)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    bf16x8w a0[KSTEPS][2], a1[KSTEPS][2], a2[KSTEPS][2];
    int tile = blockIdx.x;
    load_slab(a0, tile);
    load_slab(a1, tile + gridDim.x);

    if (ln_x) {
        // the row in registers, statistics by lane shuffles, the variance from the centred values
        if (wave < M) {
            const int m = wave;
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < kWideLnVec; ++i) sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
            const float mean = ln_no_center ? 0.f : wave_sum(sum) / (float)K;
            float sq = 0.f;
#pragma unroll
            for (int i = 0; i < kWideLnVec; ++i) {
                if (lane + i * 64 < nvec) {
                    const float p = v[i].x - mean, q = v[i].y - mean, r = v[i].z - mean, t = v[i].w - mean;
                    sq += (p * p + q * q) + (r * r + t * t);
                }
            }
            const float rstd = 1.0f / sqrtf(wave_sum(sq) / (float)K + ln_eps);
#pragma unroll
            for (int i = 0; i < kWideLnVec; ++i) {
                const int c = lane + i * 64;
                if (c >= nvec) continue;
                const float4 gm = ln_gamma ? reinterpret_cast<const float4*>(ln_gamma)[c] : make_float4(1.f, 1.f, 1.f, 1.f);
                const float4 bt = ln_beta ? reinterpret_cast<const float4*>(ln_beta)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
                uint2 p;
                p.x = pack_bf16x2((v[i].x - mean) * rstd * gm.x + bt.x, (v[i].y - mean) * rstd * gm.y + bt.y);
                p.y = pack_bf16x2((v[i].z - mean) * rstd * gm.z + bt.z, (v[i].w - mean) * rstd * gm.w + bt.w);
                *reinterpret_cast<uint2*>(xs + (int64_t)m * xstride + c * 4) = p;
            }
        }
    } else {
        const int pieces = K >> 3, total = M * pieces;
        for (int idx = threadIdx.x; idx < total; idx += kWideWaves * 64) {
            const int m = idx / pieces, c = idx - m * pieces;
            *reinterpret_cast<uint4*>(xs + (int64_t)m * xstride + c * 8) =
                *reinterpret_cast<const uint4*>(x + (int64_t)m * K + c * 8);
        }
    }
    __syncthreads();
    // this wave's part of the rows, as B operands, for all tiles
    bf16x8w b[KSTEPS][2];
    {
        const bool xvalid = r16 < M;
        const bf16_t* xrow = xs + (int64_t)(xvalid ? r16 : 0) * xstride;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int ko = k_begin + s * 64 + g * 8;
            b[s][0] = (xvalid && ko + 8 <= K) ? wide_load8(xrow + ko) : wide_zero8();
            b[s][1] = (xvalid && ko + 40 <= K) ? wide_load8(xrow + ko + 32) : wide_zero8();
        }
    }
    float best_v = -INFINITY;
    int best_i = 0x7fffffff;
    int buf = 0;
    // one tile: multiply the slab, park the partial tile, meet, and let the first wave sum and store
    auto do_tile = [&](bf16x8w (&a)[KSTEPS][2], int t) {
        const int n0 = t * 16 + 4 * g;
        float4 bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (BIAS) {          // asked for before the products, unconditionally (a tail reads the last four)
            const float* bp = bias + min(n0, N - 4);
            bias4 = N >= 4 ? make_float4(bp[0], bp[1], bp[2], bp[3]) : make_float4(bias[0], bias[min(1, N - 1)], bias[min(2, N - 1)], 0.f);
        }
        floatx4w acc = floatx4w{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][0], b[s][0], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][1], b[s][1], acc, 0, 0, 0);
        }
        floatx4w* slot = red + buf * (kWideWaves * 64);
        if (wave != 0) slot[wave * 64 + lane] = acc;
        __syncthreads();
        // (the next barrier, of the next tile, comes after this sum: nobody overwrites this half
        // of `red` before, since the tile after next is the first to use it again)
        if (wave == 0) {
#pragma unroll
            for (int wv = 1; wv < kWideWaves; ++wv) acc += slot[wv * 64 + lane];
            if (r16 < M && n0 < N) {
                float r[4] = {acc[0], acc[1], acc[2], acc[3]};
                if (BIAS) {
                    // the four values loaded belong to features min(n0, N - 4) ..: shift a tail into place
                    const float bb[4] = {bias4.x, bias4.y, bias4.z, bias4.w};
                    const int shift = N >= 4 ? n0 - min(n0, N - 4) : 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N) r[i] += bb[min(i + shift, 3)];
                }
                float* dst = out + (int64_t)r16 * N + n0;
                if (n0 + 3 < N && (N & 3) == 0) {
                    *reinterpret_cast<float4*>(dst) = make_float4(r[0], r[1], r[2], r[3]);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N) dst[i] = r[i];
                }
                if (cand_val) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N && r[i] == r[i]) better(best_v, best_i, r[i], n0 + i);   // a NaN is never the best
                }
            }
        }
        buf ^= 1;
    };
    // the walk, three tiles a round so that the three slabs keep their registers
    const int stride = gridDim.x;
    while (tile < tiles) {
        load_slab(a2, tile + 2 * stride);
        do_tile(a0, tile);
        tile += stride;
        if (tile >= tiles) break;
        load_slab(a0, tile + 2 * stride);
        do_tile(a1, tile);
        tile += stride;
        if (tile >= tiles) break;
        load_slab(a1, tile + 2 * stride);
        do_tile(a2, tile);
        tile += stride;
    }
    if (cand_val && wave == 0) {
        // the four lane groups of a row hold different features: the best of them, to lane r16
#pragma unroll
        for (int o = 32; o >= 16; o >>= 1) {
            const float ov = __shfl_xor(best_v, o, kWave);
            const int oi = __shfl_xor(best_i, o, kWave);
            better(best_v, best_i, ov, oi);
        }
        if (lane < kWideMaxRows) {
            cand_val[(int64_t)blockIdx.x * kWideMaxRows + lane] = best_v;
            cand_idx[(int64_t)blockIdx.x * kWideMaxRows + lane] = best_i;
        }
    }
}

// out[m] = the index of row m's best candidate over `groups` workgroups (lowest index on ties; 0
// if the row has none).  One wave per row.
__global__ __launch_bounds__(64) void best_of_candidates_kernel(
    int* __restrict__ out, const float* __restrict__ cand_val, const int* __restrict__ cand_idx, int groups) {
    const int m = blockIdx.x;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int gidx = threadIdx.x; gidx < groups; gidx += 64)
        better(bv, bi, cand_val[(int64_t)gidx * kWideMaxRows + m], cand_idx[(int64_t)gidx * kWideMaxRows + m]);
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, kWave);
        const int oi = __shfl_xor(bi, o, kWave);
        better(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) out[m] = bi == 0x7fffffff ? 0 : bi;
}

constexpr size_t kWideMaxLds = 140 * 1024;    // of the 160 KB a gfx950 compute unit has; one workgroup a unit

static size_t wide_lds(int M, int K) {
    return (size_t)2 * kWideWaves * 64 * sizeof(floatx4w) + (size_t)M * (K + 8) * sizeof(bf16_t);
}

// Whether the persistent kernel takes the shape: few rows, a matrix of many tiles for every
// compute unit, K within two steps a wave (three slabs then fit a lane's registers).
bool gemm_wide_offered(int M, int N, int K) {
    return M >= 1 && M <= kWideMaxRows && K % 8 == 0 && K <= kWideWaves * 2 * 64 &&
           (N + 15) / 16 >= 4 * device_compute_units() && wide_lds(M, K) <= kWideMaxLds;
}

// Workgroups the kernel runs (what a caller sizes the candidates' scratch for).
int gemm_wide_groups() { return device_compute_units(); }

int gemm_wide(float* out, const bf16_t* x, const bf16_t* w, const float* bias, int M, int N, int K,
              const StGemmExtras& ex, hipStream_t stream) {
    ST_CHECK(gemm_wide_offered(M, N, K), "gemm: the persistent kernel does not take M=%d N=%d K=%d", M, N, K);
    ST_CHECK(!ex.best_ids || (ex.best_val && ex.best_idx), "gemm: the best-of-row epilogue lacks its scratch");
    const int groups = gemm_wide_groups();
    const size_t lds = wide_lds(M, K);
    auto launch = [&](auto kernel, bool* raised) -> int {
        if (lds > 48 * 1024 && !*raised) {           // once per instance: more than the default dynamic LDS
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideMaxLds);
            ST_CHECK(e == hipSuccess, "gemm: cannot raise the LDS limit: %s", hipGetErrorString(e));
            *raised = true;
        }
        kernel<<<groups, kWideWaves * 64, lds, stream>>>(out, x, w, bias, M, N, K, ex.ln_x, ex.ln_rows, ex.ln_gamma,
                                                         ex.ln_beta, ex.ln_eps, ex.ln_no_center,
                                                         ex.best_ids ? ex.best_val : nullptr,
                                                         ex.best_ids ? ex.best_idx : nullptr);
        return 0;
    };
    static bool raised[4] = {false, false, false, false};
    const int ksteps = (K + kWideWaves * 64 - 1) / (kWideWaves * 64);
    const int rc = bias ? (ksteps <= 1 ? launch(gemm_wide_kernel<1, true>, &raised[0]) : launch(gemm_wide_kernel<2, true>, &raised[1]))
                        : (ksteps <= 1 ? launch(gemm_wide_kernel<1, false>, &raised[2]) : launch(gemm_wide_kernel<2, false>, &raised[3]));
    if (rc != 0) return rc;
    ST_LAUNCH_CHECK("gemm_wide");
    if (ex.best_ids) {
        best_of_candidates_kernel<<<M, 64, 0, stream>>>(ex.best_ids, ex.best_val, ex.best_idx, groups);
        ST_LAUNCH_CHECK("best_of_candidates");
    }
    return 0;
}

}  // namespace st
