// Row-wise kernels: table lookup (token + learned position), LayerNorm, the
// write of new keys and values into cache pages, and a cast.
//
// Reference counterparts: src/csrc/kernel/embedding.cu:17-36 (lookup + position
// add), src/csrc/kernel/layernorm.cu:17-98 (LayerNorm with fused residual),
// src/csrc/kernel/gather_last_tokens.cu:24-37 (row gather, folded into the
// LayerNorm's row index here), src/csrc/kernel/kvcache_mgmt.cu:34-80 (page write).
#include "common.h"
#include "api.h"
#include "activation.h"

#include <atomic>
#include <stdarg.h>
#include <stdio.h>

namespace st {

static thread_local char g_error[1024] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int device_compute_units() {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> units[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = units[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        hipDeviceProp_t prop;
        n = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
                ? prop.multiProcessorCount : 256;
        units[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// ---------------------------------------------------------------------- lookup
// out[t,:] = (accumulate ? out[t,:] : 0) + table[ids[t],:] + add_table[add_ids[t]+add_offset,:]
// Either table may be absent.  Sums are formed in float; `out_f32` and `out_t`
// are both optional destinations.  An index outside its table (the padding rows of a
// recorded step carry position -1) contributes zeros instead of being read.
// VEC: width is a multiple of a 16-byte access' elements and every row starts on 16 bytes.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void lookup_kernel(
    float* __restrict__ out_f32, T* __restrict__ out_t,
    const int* __restrict__ ids, const T* __restrict__ table,
    const int* __restrict__ add_ids, int add_offset, const T* __restrict__ add_table,
    int table_rows, int add_rows, int width, int accumulate) {
    const int64_t t = blockIdx.x;
    const int64_t id = table ? (int64_t)ids[t] : -1;
    const int64_t aid = add_table ? (int64_t)add_ids[t] + add_offset : -1;
    const T* row = (id >= 0 && id < table_rows) ? table + id * width : nullptr;
    const T* arow = (aid >= 0 && aid < add_rows) ? add_table + aid * width : nullptr;
    if (VEC) {
        // 16 bytes of each table a thread and turn, both asked for before either is used: a row
        // comes from memory (the tables are far larger than the caches), and a chain of narrow
        // dependent loads would pay that latency once per turn
        constexpr int V = Elem<T>::kVec;
        for (int i = threadIdx.x * V; i < width; i += blockDim.x * V) {
            float a[V], b[V], v[V];
#pragma unroll
            for (int e = 0; e < V; ++e) a[e] = b[e] = 0.f;
            if (row) Elem<T>::load_vec(row + i, a);
            if (arow) Elem<T>::load_vec(arow + i, b);
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = accumulate ? out_f32[t * width + i + e] : 0.f;
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = (v[e] + a[e]) + b[e];
            if (out_f32) {
#pragma unroll
                for (int e = 0; e < V; e += 4) Elem<float>::store4(out_f32 + t * width + i + e, v + e);
            }
            if (out_t) Elem<T>::store_vec(out_t + t * width + i, v);
        }
        return;
    }
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = accumulate ? out_f32[t * width + i] : 0.f;
        if (row) v += Elem<T>::load(row + i);
        if (arow) v += Elem<T>::load(arow + i);
        if (out_f32) out_f32[t * width + i] = v;
        if (out_t) Elem<T>::store(out_t + t * width + i, v);
    }
}

// ------------------------------------------------------------------- LayerNorm
// y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last dimension, all
// in float, variance from the centred values (two passes over registers/cache,
// no E[x^2]-E[x]^2 cancellation).  Row r of the output is computed from input row
// rows[r] when `rows` is given (gather of the wanted positions).  With center == 0 no
// mean is taken off: y = x * rsqrt(mean(x^2) + eps) * gamma + beta, the root-mean-square
// norm (the reference has it as a kernel of its own, src/csrc/kernel/rmsnorm.cu).
template <typename T>
__global__ __launch_bounds__(256) void layernorm_kernel(
    T* __restrict__ out_t, float* __restrict__ out_f32, const float* __restrict__ x,
    const int* __restrict__ rows, const float* __restrict__ gamma, const float* __restrict__ beta,
    int width, float eps, int center) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    const float* xr = x + (int64_t)(rows ? rows[r] : r) * width;
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) s += xr[i];
    const float mean = center ? block_sum(s, red) / (float)width : 0.f;
    float q = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float d = xr[i] - mean;
        q += d * d;
    }
    const float var = block_sum(q, red) / (float)width;
    const float rstd = 1.0f / sqrtf(var + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float y = (xr[i] - mean) * rstd;
        if (gamma) y *= gamma[i];
        if (beta) y += beta[i];
        if (out_t) Elem<T>::store(out_t + r * width + i, y);
        if (out_f32) out_f32[r * width + i] = y;
    }
}

// One wavefront per row, the row held in registers (VPT float4 per lane): one read of the
// row, reductions by lane shuffles only, no barrier.  width % 4 == 0, width <= 256 * VPT.
template <typename T, int VPT>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(
    T* __restrict__ out_t, float* __restrict__ out_f32, const float* __restrict__ x,
    const int* __restrict__ rows, const float* __restrict__ gamma, const float* __restrict__ beta,
    int num_rows, int width, float eps, int center) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= num_rows) return;
    const float* xr = x + (int64_t)(rows ? rows[r] : r) * width;
    const int nvec = width >> 2;
    // everything the row needs is asked for at once: the gain and bias come from memory while
    // the statistics are computed, instead of in a second round trip after them
    float4 v[VPT], gm[VPT], bt[VPT];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = lane + i * 64;
        v[i] = c < nvec ? reinterpret_cast<const float4*>(xr)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = lane + i * 64;
        gm[i] = (gamma && c < nvec) ? reinterpret_cast<const float4*>(gamma)[c] : make_float4(1.f, 1.f, 1.f, 1.f);
        bt[i] = (beta && c < nvec) ? reinterpret_cast<const float4*>(beta)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    const float mean = center ? wave_sum(s) / (float)width : 0.f;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (lane + i * 64 < nvec) {
            const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
            q += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = lane + i * 64;
        if (c >= nvec) continue;
        const float y[4] = {(v[i].x - mean) * rstd * gm[i].x + bt[i].x, (v[i].y - mean) * rstd * gm[i].y + bt[i].y,
                            (v[i].z - mean) * rstd * gm[i].z + bt[i].z, (v[i].w - mean) * rstd * gm[i].w + bt[i].w};
        if (out_f32) reinterpret_cast<float4*>(out_f32 + r * width)[c] = make_float4(y[0], y[1], y[2], y[3]);
        if (out_t) Elem<T>::store4(out_t + r * width + c * 4, y);
    }
}

template <typename T>
static bool launch_layernorm_wave(void* out_t, void* out_f32, const float* x, const int* rows,
                                  const float* gamma, const float* beta, int num_rows, int width,
                                  float eps, int center, hipStream_t stream) {
    if (width % 4 != 0 || width > 256 * 32) return false;
    const int vpt = (width / 4 + 63) / 64;
    const dim3 grid((num_rows + 3) / 4);
#define ST_LN(V)                                                                                         \
    layernorm_wave_kernel<T, V><<<grid, 256, 0, stream>>>((T*)out_t, (float*)out_f32, x, rows, gamma,    \
                                                          beta, num_rows, width, eps, center)
    if (vpt <= 1) ST_LN(1);
    else if (vpt <= 2) ST_LN(2);
    else if (vpt <= 4) ST_LN(4);
    else if (vpt <= 8) ST_LN(8);
    else if (vpt <= 16) ST_LN(16);
    else ST_LN(32);
#undef ST_LN
    return true;
}

// ------------------------------------------------------------- page write (K,V)
// For token t at position p of batch item b: page = block_table[b][p / page_size],
// row = p % page_size; the token's key and value head slices go to
// cache[page][kv_head][row][:].  k_src/v_src point at the first key/value element
// of token 0 and advance by src_stride elements per token.
template <typename T>
__global__ __launch_bounds__(256) void kv_write_kernel(
    T* __restrict__ k_cache, T* __restrict__ v_cache, int64_t page_stride,
    const T* __restrict__ k_src, const T* __restrict__ v_src, int64_t src_stride,
    const int* __restrict__ token_item, const int* __restrict__ positions,
    const int* __restrict__ block_table, int max_pages, int page_size,
    int num_kv_heads, int head_dim, int vectors) {
    const int64_t t = blockIdx.x;
    const int pos = positions[t];
    const int item = token_item[t];
    if (item < 0 || pos < 0) return;   // padding rows of a fixed-size batch
    const int page = block_table[(int64_t)item * max_pages + pos / page_size];
    if (page < 0) return;
    const int row = pos % page_size;
    const int n = num_kv_heads * head_dim;
    if (vectors) {                     // 16 bytes at a time: everything is 16-byte aligned
        constexpr int V = 16 / sizeof(T);
        for (int i = threadIdx.x * V; i < n; i += blockDim.x * V) {
            const int h = i / head_dim, d = i - h * head_dim;
            const int64_t dst = (int64_t)page * page_stride + ((int64_t)h * page_size + row) * head_dim + d;
            *reinterpret_cast<uint4*>(k_cache + dst) = *reinterpret_cast<const uint4*>(k_src + t * src_stride + i);
            *reinterpret_cast<uint4*>(v_cache + dst) = *reinterpret_cast<const uint4*>(v_src + t * src_stride + i);
        }
        return;
    }
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int h = i / head_dim, d = i - h * head_dim;
        const int64_t dst = (int64_t)page * page_stride + ((int64_t)h * page_size + row) * head_dim + d;
        k_cache[dst] = k_src[t * src_stride + i];
        v_cache[dst] = v_src[t * src_stride + i];
    }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void cast_kernel(TO* __restrict__ out, const TI* __restrict__ in, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) Elem<TO>::store(out + i, Elem<TI>::load(in + i));
}

// ------------------------------------------------------- activation, multiply
// out[r, c] = act(a[r, c]) * b[r, c] (b absent: times one), float arithmetic.  One thread per
// vector of 16 bytes where strides, width and addresses allow it, else per element.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void activation_multiply_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ a, int64_t a_stride,
    const T* __restrict__ b, int64_t b_stride, int rows, int width, int kind) {
    constexpr int V = VEC ? Elem<T>::kVec : 1;
    const int per_row = width / V;
    const int64_t total = (int64_t)rows * per_row;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(i / per_row), c = (int)(i - (int64_t)r * per_row) * V;
        float x[V], y[V];
        if (VEC) {
            Elem<T>::load_vec(a + r * a_stride + c, x);
            if (b) Elem<T>::load_vec(b + r * b_stride + c, y);
        } else {
            x[0] = Elem<T>::load(a + r * a_stride + c);
            if (b) y[0] = Elem<T>::load(b + r * b_stride + c);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) {
            x[j] = apply_activation(kind, x[j]);
            if (b) x[j] *= y[j];
        }
        if (VEC) Elem<T>::store_vec(out + r * out_stride + c, x);
        else Elem<T>::store(out + r * out_stride + c, x[0]);
    }
}

template <typename T>
static void launch_activation_multiply(void* out, int64_t out_stride, const void* a, int64_t a_stride, const void* b,
                                       int64_t b_stride, int rows, int width, int kind, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const uintptr_t align = (uintptr_t)out | (uintptr_t)a | (uintptr_t)b;
    const bool vec = width % V == 0 && out_stride % V == 0 && a_stride % V == 0 && (!b || b_stride % V == 0) &&
                     (align & 15) == 0;
    const int64_t work = (int64_t)rows * (vec ? width / V : width);
    const int64_t want = (work + 255) / 256, most = (int64_t)device_compute_units() * 16;
    const unsigned grid = (unsigned)(want < most ? want : most);
    if (vec)
        activation_multiply_kernel<T, true><<<grid, 256, 0, stream>>>((T*)out, out_stride, (const T*)a, a_stride,
                                                                      (const T*)b, b_stride, rows, width, kind);
    else
        activation_multiply_kernel<T, false><<<grid, 256, 0, stream>>>((T*)out, out_stride, (const T*)a, a_stride,
                                                                       (const T*)b, b_stride, rows, width, kind);
}

}  // namespace st

using namespace st;

extern "C" const char* st_last_error() { return g_error; }

extern "C" int st_lookup(void* out_f32, void* out_t, const int* ids, const void* table,
                         const int* add_ids, int add_offset, const void* add_table,
                         int table_rows, int add_rows,
                         int num_rows, int width, int accumulate, int dtype, hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0, "lookup: bad sizes rows=%d width=%d", num_rows, width);
    ST_CHECK(out_f32 || out_t, "lookup: no destination");
    ST_CHECK(!accumulate || out_f32, "lookup: accumulate needs the float destination");
    ST_CHECK(!table || ids, "lookup: table without ids");
    ST_CHECK(!add_table || add_ids, "lookup: add_table without add_ids");
    ST_CHECK((!table || table_rows > 0) && (!add_table || add_rows > 0), "lookup: a table without rows");
    if (num_rows == 0) return 0;
    const uintptr_t align = (uintptr_t)out_f32 | (uintptr_t)out_t | (uintptr_t)table | (uintptr_t)add_table;
    const bool vec = (align & 15) == 0 && width % (dtype == kF32 ? 4 : 8) == 0;
#define ST_LOOKUP(T, V) lookup_kernel<T, V><<<num_rows, 256, 0, stream>>>((float*)out_f32, (T*)out_t, ids,         \
        (const T*)table, add_ids, add_offset, (const T*)add_table, table_rows, add_rows, width, accumulate)
    if (dtype == kF32) { if (vec) ST_LOOKUP(float, true); else ST_LOOKUP(float, false); }
    else if (dtype == kBF16) { if (vec) ST_LOOKUP(bf16_t, true); else ST_LOOKUP(bf16_t, false); }
    else ST_CHECK(false, "lookup: unknown dtype %d", dtype);
#undef ST_LOOKUP
    ST_LAUNCH_CHECK("lookup");
    return 0;
}

extern "C" int st_layernorm(void* out_t, void* out_f32, const float* x, const int* rows,
                            const float* gamma, const float* beta, int num_rows, int width,
                            float eps, int center, int dtype, hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0, "layernorm: bad sizes rows=%d width=%d", num_rows, width);
    ST_CHECK(out_t || out_f32, "layernorm: no destination");
    ST_CHECK(eps > 0.f, "layernorm: eps must be positive");
    if (num_rows == 0) return 0;
    ST_CHECK(dtype == kF32 || dtype == kBF16, "layernorm: unknown dtype %d", dtype);
    const uintptr_t align = (uintptr_t)out_t | (uintptr_t)out_f32 | (uintptr_t)x | (uintptr_t)gamma |
                            (uintptr_t)beta;
    bool done = false;
    if ((align & 15) == 0) {
        done = dtype == kF32
            ? launch_layernorm_wave<float>(out_t, out_f32, x, rows, gamma, beta, num_rows, width, eps, center, stream)
            : launch_layernorm_wave<bf16_t>(out_t, out_f32, x, rows, gamma, beta, num_rows, width, eps, center, stream);
    }
    if (done) {
    } else if (dtype == kF32)
        layernorm_kernel<float><<<num_rows, 256, 0, stream>>>((float*)out_t, (float*)out_f32, x, rows,
                                                             gamma, beta, width, eps, center);
    else
        layernorm_kernel<bf16_t><<<num_rows, 256, 0, stream>>>((bf16_t*)out_t, (float*)out_f32, x, rows,
                                                              gamma, beta, width, eps, center);
    ST_LAUNCH_CHECK("layernorm");
    return 0;
}

extern "C" int st_kv_write(void* k_cache, void* v_cache, int64_t page_stride,
                           const void* k_src, const void* v_src, int64_t src_stride,
                           const int* token_item, const int* positions,
                           const int* block_table, int max_pages, int page_size,
                           int num_tokens, int num_kv_heads, int head_dim, int dtype,
                           hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && num_kv_heads > 0 && head_dim > 0 && page_size > 0 && max_pages > 0,
             "kv_write: bad sizes");
    ST_CHECK(page_stride >= (int64_t)num_kv_heads * page_size * head_dim,
             "kv_write: page stride %lld smaller than a page", (long long)page_stride);
    if (num_tokens == 0) return 0;
    const int per16 = dtype == kF32 ? 4 : 8;         // elements in 16 bytes
    const int vectors = head_dim % per16 == 0 && src_stride % per16 == 0 && page_stride % per16 == 0 &&
        ((reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) |
          reinterpret_cast<uintptr_t>(k_src) | reinterpret_cast<uintptr_t>(v_src)) & 15) == 0;
    if (dtype == kF32)
        kv_write_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)k_cache, (float*)v_cache, page_stride,
            (const float*)k_src, (const float*)v_src, src_stride, token_item, positions, block_table,
            max_pages, page_size, num_kv_heads, head_dim, vectors);
    else if (dtype == kBF16)
        kv_write_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)k_cache, (bf16_t*)v_cache, page_stride,
            (const bf16_t*)k_src, (const bf16_t*)v_src, src_stride, token_item, positions, block_table,
            max_pages, page_size, num_kv_heads, head_dim, vectors);
    else ST_CHECK(false, "kv_write: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("kv_write");
    return 0;
}

extern "C" int st_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype,
                       hipStream_t stream) {
    ST_CHECK(n >= 0, "cast: negative size");
    if (n == 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (in_dtype == kF32 && out_dtype == kBF16)
        cast_kernel<float, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const float*)in, n);
    else if (in_dtype == kBF16 && out_dtype == kF32)
        cast_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((float*)out, (const bf16_t*)in, n);
    else if (in_dtype == kF32 && out_dtype == kF32)
        cast_kernel<float, float><<<grid, 256, 0, stream>>>((float*)out, (const float*)in, n);
    else if (in_dtype == kBF16 && out_dtype == kBF16)
        cast_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)in, n);
    else ST_CHECK(false, "cast: unknown dtypes %d -> %d", in_dtype, out_dtype);
    ST_LAUNCH_CHECK("cast");
    return 0;
}

extern "C" int st_activation_multiply(void* out, int64_t out_stride, const void* a, int64_t a_stride,
                                      const void* b, int64_t b_stride, int rows, int width, int kind,
                                      int dtype, hipStream_t stream) {
    ST_CHECK(rows >= 0 && width > 0, "activation_multiply: bad sizes rows=%d width=%d", rows, width);
    ST_CHECK(out && a, "activation_multiply: null operand");
    ST_CHECK(activation_known(kind), "activation_multiply: activation %d has no kernel", kind);
    ST_CHECK(out_stride >= width && a_stride >= width && (!b || b_stride >= width),
             "activation_multiply: a row stride is smaller than the width %d", width);
    ST_CHECK(dtype == kF32 || dtype == kBF16, "activation_multiply: unknown dtype %d", dtype);
    if (rows == 0) return 0;
    if (dtype == kF32) launch_activation_multiply<float>(out, out_stride, a, a_stride, b, b_stride, rows, width, kind, stream);
    else launch_activation_multiply<bf16_t>(out, out_stride, a, a_stride, b, b_stride, rows, width, kind, stream);
    ST_LAUNCH_CHECK("activation_multiply");
    return 0;
}
