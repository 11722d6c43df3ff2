// Token choice from float logits: argmax (lowest index on ties) and temperature
// sampling in Gumbel-max form, argmax_v(logit_v / temperature + g_v), with
// g_v = -log(-log(u_v)) and u_v from a counter-based hash of
// (seed, draw index, v).  The noise of a draw depends on nothing else, so the
// chosen token does not depend on the batch a request is in.
//
// Reference: greedy only, src/csrc/kernel/findmax.cu:16-39 (one block per row;
// on ties the last writer wins, here the lowest index wins).
#include "common.h"
#include "api.h"

namespace st {

__host__ __device__ inline uint32_t fmix32(uint32_t h) {
    h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
    return h;
}

// uniform in (0,1) with 24 random bits, from (seed_lo, seed_hi, draw, v)
__host__ __device__ inline float hash_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t draw, uint32_t v) {
    uint32_t h = fmix32(seed_lo ^ 0x9e3779b9u);
    h = fmix32(h ^ (seed_hi + 0x7f4a7c15u));
    h = fmix32(h ^ (draw * 0x85ebca6bu + 0xc2b2ae35u));
    h = fmix32(h ^ (v * 0x27d4eb2fu + 0x165667b1u));
    return ((float)(h >> 8) + 0.5f) * (1.0f / 16777216.0f);
}

__device__ inline void take_better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

// temperature[r] <= 0 selects plain argmax for row r.
__global__ __launch_bounds__(1024) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int vocab,
    const float* __restrict__ temperature, const uint32_t* __restrict__ seeds,
    const uint32_t* __restrict__ draws) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const int64_t r = blockIdx.x;
    const float* row = logits + r * vocab;
    const float temp = temperature ? temperature[r] : 0.f;
    const uint32_t s_lo = seeds ? seeds[2 * r] : 0u, s_hi = seeds ? seeds[2 * r + 1] : 0u;
    const uint32_t draw = draws ? draws[r] : 0u;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    // eight independent loads in flight per thread: the row comes from memory once, and a
    // chain of dependent single loads would cost a round trip each
    constexpr int U = 8;
    for (int base = threadIdx.x; base < vocab; base += U * blockDim.x) {
        float xs[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int v = base + u * blockDim.x;
            xs[u] = v < vocab ? row[v] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int v = base + u * blockDim.x;
            if (v >= vocab) break;
            float x = xs[u];
            if (temp > 0.f) {
                const float un = hash_uniform(s_lo, s_hi, draw, (uint32_t)v);
                x = x / temp - logf(-logf(un));
            }
            if (x != x) x = -INFINITY;   // a NaN logit is never chosen
            take_better(bv, bi, x, v);
        }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, kWave);
        const int oi = __shfl_xor(bi, o, kWave);
        take_better(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) take_better(bv, bi, sv[w], si[w]);
        out[r] = bi == 0x7fffffff ? 0 : bi;
    }
}

}  // namespace st

using namespace st;

extern "C" int st_sample(int* out, const float* logits, int num_rows, int vocab,
                         const float* temperature, const uint32_t* seeds, const uint32_t* draws,
                         hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", num_rows, vocab);
    ST_CHECK(out && logits, "sample: null operand");
    if (num_rows == 0) return 0;
    sample_kernel<<<num_rows, 1024, 0, stream>>>(out, logits, vocab, temperature, seeds, draws);
    ST_LAUNCH_CHECK("sample");
    return 0;
}

// host copy of the hash, so that a plain implementation can draw the same noise
extern "C" float st_hash_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t draw, uint32_t v) {
    return hash_uniform(seed_lo, seed_hi, draw, v);
}
