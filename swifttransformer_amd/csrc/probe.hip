// Two measurement kernels, for the floors that the benchmark quotes: what a plain streaming read
// of this device reaches, and what a kernel costs in a chain of dependent kernels before it
// streams anything.  Nothing of the model runs through them.
#include "common.h"
#include "api.h"

namespace st {

// Read of `n16` 16-byte words; consecutive lanes read consecutive words.  DEPTH independent loads
// are in flight per thread.  TILED: a workgroup reads tiles of DEPTH KB (its threads' DEPTH loads
// are 4 KB apart inside the tile) dealt round-robin to the workgroups, as a kernel that walks over
// slabs of a matrix does; else the whole grid strides over the buffer.  Every workgroup leaves
// the sum of what it read in sink[workgroup], so that the loads cannot be dropped.
template <int DEPTH, bool TILED>
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, int64_t n16,
                                                         uint32_t* __restrict__ sink) {
    uint32_t acc = 0;
    if (TILED) {
        const int64_t tile_words = (int64_t)DEPTH * 256;
        const int64_t tiles = n16 / tile_words;
        for (int64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
            const uint4* p = src + t * tile_words + threadIdx.x;
            uint4 v[DEPTH];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) v[d] = p[d * 256];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) acc += v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
        }
        for (int64_t i = tiles * tile_words + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) {
            const uint4 a = src[i];
            acc += a.x ^ a.y ^ a.z ^ a.w;
        }
    } else {
        const int64_t stride = (int64_t)gridDim.x * blockDim.x;
        int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        for (; i + (DEPTH - 1) * stride < n16; i += DEPTH * stride) {
            uint4 v[DEPTH];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) v[d] = src[i + d * stride];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) acc += v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
        }
        for (; i < n16; i += stride) {
            const uint4 a = src[i];
            acc += a.x ^ a.y ^ a.z ^ a.w;
        }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    if ((threadIdx.x & 63) == 0) atomicAdd(&sink[blockIdx.x], acc);
}

__global__ void probe_empty_kernel(uint32_t* sink) {
    if (sink == nullptr) return;        // always taken as called below with a live pointer: one store
    if (threadIdx.x == 0 && blockIdx.x == 0) sink[0] += 1;
}

}  // namespace st

using namespace st;

// Reads `bytes` (a multiple of 16) from src with `workgroups` workgroups of 256 threads.
// pattern: 0 the grid strides over the buffer with 4 loads in flight per thread, 1 with 8,
// 2 tiles of 8 KB dealt round-robin to the workgroups, 3 tiles of 16 KB.
// sink: at least `workgroups` 32-bit words.
extern "C" int st_probe_read(const void* src, int64_t bytes, void* sink, int workgroups, int pattern,
                             hipStream_t stream) {
    ST_CHECK(src && sink && bytes >= 16 && bytes % 16 == 0 && workgroups >= 1, "probe_read: bad arguments");
    const uint4* p = (const uint4*)src;
    uint32_t* s = (uint32_t*)sink;
    switch (pattern) {
        case 0: probe_read_kernel<4, false><<<workgroups, 256, 0, stream>>>(p, bytes / 16, s); break;
        case 1: probe_read_kernel<8, false><<<workgroups, 256, 0, stream>>>(p, bytes / 16, s); break;
        case 2: probe_read_kernel<8, true><<<workgroups, 256, 0, stream>>>(p, bytes / 16, s); break;
        case 3: probe_read_kernel<16, true><<<workgroups, 256, 0, stream>>>(p, bytes / 16, s); break;
        default: ST_CHECK(false, "probe_read: unknown pattern %d", pattern);
    }
    ST_LAUNCH_CHECK("probe_read");
    return 0;
}

// A kernel of one workgroup that does one store: what is left of a kernel when its work is taken away.
extern "C" int st_probe_empty(void* sink, hipStream_t stream) {
    ST_CHECK(sink, "probe_empty: no sink");
    probe_empty_kernel<<<1, 64, 0, stream>>>((uint32_t*)sink);
    ST_LAUNCH_CHECK("probe_empty");
    return 0;
}
