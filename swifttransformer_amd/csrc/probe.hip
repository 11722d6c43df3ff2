// Measurement kernels, for the floors that the benchmark quotes: what a plain streaming read of
// this device reaches, what a kernel costs in a chain of dependent kernels before it streams
// anything, how fast a compute unit is filled from the caches (the limit of a tiled matrix
// product) and at what rate one or two waves a SIMD issue matrix-core products.  Nothing of the
// model runs through them.
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

// The access pattern of a matrix-core operand read straight from memory: the buffer is rows of
// `row_bytes`; a wave takes 16 rows at a time, lane (row l % 16, group l / 16) reads 16 bytes at
// byte 64 c + 16 (l / 16) of its row for c = 0, 1, ...: one load instruction touches 64 bytes of
// each of 16 rows, the next one the 64 bytes beside them.  8 loads in flight a lane.
__global__ __launch_bounds__(256) void probe_rows_kernel(const char* __restrict__ src, int64_t rows, int row_bytes,
                                                         uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    uint32_t acc = 0;
    const int64_t groups = rows / 16;
    for (int64_t grp = (int64_t)blockIdx.x * 4 + wave; grp < groups; grp += (int64_t)gridDim.x * 4) {
        const char* p = src + (grp * 16 + r16) * (int64_t)row_bytes + g * 16;
        for (int c = 0; c + 8 <= row_bytes / 64; c += 8) {
            uint4 v[8];
#pragma unroll
            for (int d = 0; d < 8; ++d) v[d] = *reinterpret_cast<const uint4*>(p + (c + d) * 64);
#pragma unroll
            for (int d = 0; d < 8; ++d) acc += v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
        }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    if (lane == 0) atomicAdd(&sink[blockIdx.x], acc);
}

__global__ void probe_empty_kernel(uint32_t* sink) {
    if (sink == nullptr) return;        // always taken as called below with a live pointer: one store
    if (threadIdx.x == 0 && blockIdx.x == 0) sink[0] += 1;
}

// A workgroup of 256 threads goes round and round its own region of `region` bytes (a multiple of
// 32 KB), 32 KB a turn, 16 bytes a lane and load, two turns in flight.  TO_LDS: by the direct load
// into LDS (global_load_lds_dwordx4), else into registers.  With all regions together smaller than
// the L2s this is the rate at which a compute unit is filled from its L2; with large regions, from
// beyond it.
template <bool TO_LDS>
__global__ __launch_bounds__(256) void probe_fill_kernel(const char* __restrict__ src, int64_t region, int turns,
                                                         uint32_t* __restrict__ sink) {
    __shared__ uint4 lds[2 * 2048];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const char* base = src + (int64_t)blockIdx.x * region;
    uint32_t acc = 0;
    int64_t off = 0;
    for (int it = 0; it < turns; ++it) {
        if (TO_LDS) {
            char* dst = reinterpret_cast<char*>(lds) + (it & 1) * 32768;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + off + (j * 256 + tid) * 16),
                                                 (__attribute__((address_space(3))) void*)(dst + (j * 4 + wave) * 1024), 16, 0, 0);
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        } else {
            uint4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const uint4*>(base + off + (j * 256 + tid) * 16);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc += v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
        }
        off += 32768;
        if (off >= region) off = 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (TO_LDS) acc = lds[tid].x ^ lds[2048 + tid].x;
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    if ((tid & 63) == 0) atomicAdd(&sink[blockIdx.x], acc);
}

// `rounds` rounds of 16 independent matrix-core products a wave (four waves a workgroup, no memory
// traffic).  WIDE: v_mfma_f32_32x32x16_bf16, else v_mfma_f32_16x16x32_bf16; both do 2 * 16384 or
// 16384 multiply-adds an instruction.
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_floatx4 __attribute__((ext_vector_type(4)));
typedef float probe_floatx16 __attribute__((ext_vector_type(16)));
template <bool WIDE>
__global__ __launch_bounds__(256) void probe_mfma_kernel(uint32_t* __restrict__ sink, int rounds) {
    probe_bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(float)(threadIdx.x & 3);
        b[i] = (__bf16)1.0f;
    }
    float total = 0.f;
    if (WIDE) {
        probe_floatx16 c[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) c[i][e] = 0.f;
        for (int r = 0; r < rounds; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) c[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[i & 3], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) total += c[i][0];
    } else {
        probe_floatx4 c[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) c[i] = probe_floatx4{0.f, 0.f, 0.f, 0.f};
        for (int r = 0; r < rounds; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) c[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; ++i) total += c[i][0];
    }
    if (threadIdx.x == 0) sink[blockIdx.x] = (uint32_t)total;
}

}  // namespace st

using namespace st;

// Reads `bytes` (a multiple of 16) from src with `workgroups` workgroups of 256 threads.
// pattern: 0 the grid strides over the buffer with 4 loads in flight per thread, 1 with 8,
// 2 tiles of 8 KB dealt round-robin to the workgroups, 3 tiles of 16 KB, 4 / 5 rows of 4 / 16 KB read
// as a matrix-core operand is (16 rows a wave, 64 bytes of each row an instruction).
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
        case 4:
        case 5: {
            const int row_bytes = pattern == 4 ? 4096 : 16384;
            ST_CHECK(bytes % (16 * (int64_t)row_bytes) == 0, "probe_read: pattern %d reads groups of 16 rows of %d bytes", pattern, row_bytes);
            probe_rows_kernel<<<workgroups, 256, 0, stream>>>((const char*)src, bytes / row_bytes, row_bytes, s);
            break;
        }
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

// `workgroups` workgroups of 256 threads each go `turns` times 32 KB through their own region of
// `region` bytes (a multiple of 32 KB) of src, which holds workgroups * region bytes.
// to_lds != 0: by direct loads into LDS.  sink: at least `workgroups` 32-bit words.
extern "C" int st_probe_fill(const void* src, int64_t region, void* sink, int workgroups, int turns, int to_lds,
                             hipStream_t stream) {
    ST_CHECK(src && sink && region >= 32768 && region % 32768 == 0 && workgroups >= 1 && turns >= 1,
             "probe_fill: bad arguments");
    if (to_lds) probe_fill_kernel<true><<<workgroups, 256, 0, stream>>>((const char*)src, region, turns, (uint32_t*)sink);
    else probe_fill_kernel<false><<<workgroups, 256, 0, stream>>>((const char*)src, region, turns, (uint32_t*)sink);
    ST_LAUNCH_CHECK("probe_fill");
    return 0;
}

// `workgroups` workgroups of four waves each issue 16 * rounds matrix-core products a wave:
// wide != 0 the 32x32x16 bfloat16 form (32768 multiply-adds), else 16x16x32 (16384).
extern "C" int st_probe_mfma(void* sink, int workgroups, int rounds, int wide, hipStream_t stream) {
    ST_CHECK(sink && workgroups >= 1 && rounds >= 1, "probe_mfma: bad arguments");
    if (wide) probe_mfma_kernel<true><<<workgroups, 256, 0, stream>>>((uint32_t*)sink, rounds);
    else probe_mfma_kernel<false><<<workgroups, 256, 0, stream>>>((uint32_t*)sink, rounds);
    ST_LAUNCH_CHECK("probe_mfma");
    return 0;
}
