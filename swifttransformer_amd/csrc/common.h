// Shared device helpers for the gfx950 kernels: storage types, 64-wide wavefront
// reductions, and the host-side error channel of the C entry points.
//
// The reference's reductions are 32-wide warp shuffles
// (src/csrc/kernel/reduction.cuh:27-85); a CDNA wavefront has 64 lanes, so the
// helpers here reduce over 64 lanes and then across the waves of a workgroup
// through LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

namespace st {

constexpr int kWave = 64;

// bfloat16 is handled as its 16 stored bits; arithmetic is always float.
struct bf16_t { uint16_t bits; };

__host__ __device__ inline float bf16_to_float(uint16_t b) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)b) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN
__host__ __device__ inline uint16_t float_to_bf16(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// two floats -> two bfloat16 in one register, low half = a: the hardware's packed convert
// (round to nearest even), one instruction instead of a dozen
__device__ inline uint32_t pack_bf16x2(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float floatx2_t __attribute__((ext_vector_type(2)));
    const floatx2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
#else
    return (uint32_t)float_to_bf16(a) | ((uint32_t)float_to_bf16(b) << 16);
#endif
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int kVec = 4;   // elements in a 16-byte access
    __device__ static inline float load(const float* p) { return *p; }
    __device__ static inline void store(float* p, float v) { *p = v; }
    __device__ static inline void load_vec(const float* p, float* out) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
    __device__ static inline void store_vec(float* p, const float* in) {
        *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
    }
    __device__ static inline void store4(float* p, const float* in) {    // p 16-byte aligned
        *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
    }
    __device__ static inline void unpack(const uint4& v, float* out) {   // 16 loaded bytes -> floats
        out[0] = __uint_as_float(v.x); out[1] = __uint_as_float(v.y);
        out[2] = __uint_as_float(v.z); out[3] = __uint_as_float(v.w);
    }
};
template <> struct Elem<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static inline float load(const bf16_t* p) { return bf16_to_float(p->bits); }
    __device__ static inline void store(bf16_t* p, float v) { p->bits = float_to_bf16(v); }
    __device__ static inline void load_vec(const bf16_t* p, float* out) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static inline void unpack(const uint4& v, float* out) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static inline void store4(bf16_t* p, const float* in) {   // p 8-byte aligned
        *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(in[0], in[1]), pack_bf16x2(in[2], in[3]));
    }
    __device__ static inline void store_vec(bf16_t* p, const float* in) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = pack_bf16x2(in[2 * i], in[2 * i + 1]);
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

// Reductions over the four lanes l%16, l%16+16, l%16+32, l%16+48 of a wavefront (the four
// 16-lane rows), by the row-swap instructions of gfx950 instead of trips through LDS.
// Every lane gets the result.
// max without the quieting of signalling NaNs that fmaxf asks of the compiler (a second
// instruction per operand that comes out of a matrix instruction or a lane swap)
__device__ inline float max_raw(float a, float b) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ inline float max3_raw(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

__device__ inline float rows4_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const float y = max_raw(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t w = __float_as_uint(y);
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return max_raw(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float rows4_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const float y = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t w = __float_as_uint(y);
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `red` is LDS scratch of at least 16 floats; safe to call repeatedly.
__device__ inline float block_sum(float v, float* red) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int nwaves = (blockDim.x + kWave - 1) >> 6;
    v = wave_sum(v);
    __syncthreads();              // protect `red` from the previous call's readers
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nwaves; ++i) r += red[i];
    return r;
}

// ------------------------------------------------------------ host-side errors
void set_error(const char* fmt, ...);

// Compute units of the current device (asked of the runtime once per device); the launch
// shapes that depend on how many workgroups fill the chip take it from here.
int device_compute_units();

#define ST_CHECK(cond, ...)                      \
    do {                                         \
        if (!(cond)) {                           \
            st::set_error(__VA_ARGS__);          \
            return 1;                            \
        }                                        \
    } while (0)

#define ST_LAUNCH_CHECK(what)                                                        \
    do {                                                                             \
        hipError_t e__ = hipGetLastError();                                          \
        if (e__ != hipSuccess) {                                                     \
            st::set_error("%s: launch failed: %s", what, hipGetErrorString(e__));    \
            return 2;                                                                \
        }                                                                            \
    } while (0)

enum DType : int { kF32 = 0, kBF16 = 1 };

}  // namespace st
