// The functions a product applies between its bias and its residual sum, by number.  The number
// is the one the C interface takes (st_gemm's `activation`, st_activation's `kind`); every product
// kernel and the elementwise kernel call apply_activation, so a further function is one more case
// here and one more name in the host's table, and nothing else.
//
// The reference has the same three (src/csrc/kernel/activations.cuh:8-24): ReLU, SiLU as
// x / (1 + exp(-x)), and GELU in its tanh form 0.5 x (1 + tanh(0.79788456 (x + 0.044715 x^3))).
// Here they are always evaluated in float, with the accurate exp and tanh.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace st {

enum Activation : int { kActNone = 0, kActRelu = 1, kActSilu = 2, kActGeluTanh = 3, kNumActivations };

inline bool activation_known(int kind) { return kind >= 0 && kind < kNumActivations; }
// the vendor library's epilogues are asked for these only; the others run in this library's kernels
inline bool activation_in_library(int kind) { return kind == kActNone || kind == kActRelu; }

__host__ __device__ inline float apply_activation(int kind, float v) {
    switch (kind) {
        case kActRelu: return fmaxf(v, 0.f);
        case kActSilu: return v / (1.f + expf(-v));
        case kActGeluTanh: return 0.5f * v * (1.f + tanhf(0.79788456f * (v + 0.044715f * v * v * v)));
        default: return v;
    }
}

// the same on four values: the kind is uniform over a launch, so one branch serves all four
__device__ inline void apply_activation4(int kind, float* r) {
    switch (kind) {
        case kActNone: break;
        case kActRelu:
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = fmaxf(r[i], 0.f);
            break;
        default:
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = apply_activation(kind, r[i]);
    }
}

}  // namespace st
