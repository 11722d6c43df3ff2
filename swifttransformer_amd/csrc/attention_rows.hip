// Attention of single query rows over the paged cache, split over the keys.
//
// One workgroup handles (query head, token, key split).  The token at position p
// of its request attends to the cached keys [lo, p] of that request
// (lo = max(0, p + 1 - window) when a window is set), read through the request's
// block table.  This is the decode kernel; it is also the general fallback for
// any row of a prompt portion, since the portion's keys are in the cache before
// attention runs.
//
// Reference: src/csrc/kernel/fused_decoding_stage_attention_mha.cu:85-319 — one
// block per (head, request), scores in shared memory sized by the context
// (:372), probabilities normalised with 1/(sum + 1e-6) (:241), P*V accumulated in
// the storage type (:272-279).  Differences here: keys are split over several
// workgroups and merged by log-sum-exp so that one request fills the chip and no
// LDS grows with the context; softmax is online; every sum is in float; the
// normaliser is exact; the new token's K/V are written by a separate kernel
// before this one runs.
//
// Lane layout: LPK lanes share one key, each holding 16 bytes of the head
// dimension; a wave therefore holds 64/LPK keys at a time and every such lane
// group runs its own online softmax over the keys it visits, U keys per round: the round's
// scores are all computed (and summed over the group's lanes by data-parallel moves) before
// one update of maximum, normaliser and accumulator, and the next round's keys and values
// are already on their way from memory meanwhile.  The groups are merged once at the end
// through LDS.
#include "common.h"
#include "api.h"

#include <mutex>

namespace st {

// Scratch of st_attn_rows_static: the partial results and log-sum-exps of a key split, which
// st_attn_rows takes from its caller as a workspace.  4 MiB that each GPU the library runs on
// holds until the process ends.  In host code this name is a stand-in, not a device address:
// host code uses the pointer that static_scratch() resolves per device.
constexpr size_t kStaticScratchFloats = size_t(1) << 20;
static __device__ __align__(256) __attribute__((used)) float scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// The current device's copy of `scratch` (every GPU has its own, at its own address), resolved
// once per device.
static int static_scratch(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    ST_CHECK(e == hipSuccess, "attention: hipGetDevice: %s", hipGetErrorString(e));
    ST_CHECK(dev >= 0 && dev < kMaxDevices, "attention: device %d is beyond the %d this library keeps scratch for",
             dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        ST_CHECK(e == hipSuccess && p, "attention: hipGetSymbolAddress(scratch) on device %d: %s", dev,
                 hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

template <bool ACCURATE>
__device__ inline float exp_(float x) { return ACCURATE ? expf(x) : __expf(x); }

// x + (x of the lane a data-parallel move names); CTRL: 0xB1 lane^1, 0x4E lane^2 (quad
// permutations), 0x141 mirror inside 8 lanes, 0x140 mirror inside 16 lanes
template <int CTRL>
__device__ inline float add_moved(float x) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false);
    return x + __int_as_float(moved);
}

// Sum over the LPK consecutive lanes that share a key; every lane gets the total.  Mirrors
// followed by the two quad permutations reach all lanes of a group of 8 or 16; wider groups
// add the row swaps.
template <int LPK>
__device__ inline float group_sum(float s) {
    if (LPK >= 64) {
        const uint32_t u = __float_as_uint(s);
        const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        s = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    }
    if (LPK >= 32) {
        const uint32_t u = __float_as_uint(s);
        const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        s = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    }
    if (LPK >= 16) s = add_moved<0x140>(s);
    if (LPK >= 8) s = add_moved<0x141>(s);
    if (LPK >= 4) s = add_moved<0x4E>(s);
    if (LPK >= 2) s = add_moved<0xB1>(s);
    return s;
}

template <typename T, int LPK>
__global__ __launch_bounds__(512) void attn_rows_kernel(
    T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_lse,
    const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, int64_t page_stride,
    const int* __restrict__ row_ids, const int* __restrict__ token_item, const int* __restrict__ positions,
    const int* __restrict__ block_table, const float* __restrict__ head_slopes, int max_pages, int page_size,
    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, int num_splits) {
    constexpr int VEC = Elem<T>::kVec;
    constexpr int KPW = kWave / LPK;        // keys per wave per step
    const int G = (blockDim.x >> 6) * KPW;  // lane groups in the workgroup (4 or 8 waves)
    constexpr bool ACC = sizeof(T) == 4;    // float path: accurate expf
    extern __shared__ float lds[];
    float* s_m = lds;                       // [G]
    float* s_l = lds + G;                   // [G]
    float* s_acc = lds + 2 * G;             // [G][head_dim]
    float* s_red = lds + 2 * G + G * head_dim;   // [16] per-wave partial results of the final merge
    int* s_bt = reinterpret_cast<int*>(s_red + 16);   // [max_pages] pages of this request

    const int h = blockIdx.x, ri = blockIdx.y, split = blockIdx.z;
    const int t = row_ids ? row_ids[ri] : ri;      // batch row of this query
    if (t < 0) return;                             // a padding entry of a row list of fixed length
    const int item = token_item[t];
    const int pos = positions[t];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / LPK, sub = lane % LPK;
    const int gi = wave * KPW + g;
    const int d0 = sub * VEC;
    const bool dvalid = d0 < head_dim;

    int kb = 0, ke = 0;
    if (item >= 0 && pos >= 0) {
        const int hi = pos + 1;
        const int lo = (window > 0 && hi > window) ? hi - window : 0;
        const int chunk = (hi - lo + num_splits - 1) / num_splits;
        kb = lo + split * chunk;
        ke = min(hi, kb + chunk);
    }
    // the pages this workgroup will touch go to LDS first: key addresses then need no
    // dependent global load
    int p_lo = 0;
    if (kb < ke) {
        p_lo = kb / page_size;
        const int p_n = (ke - 1) / page_size - p_lo + 1;
        const int* bt = block_table + (int64_t)item * max_pages + p_lo;
        for (int i = threadIdx.x; i < p_n; i += blockDim.x) s_bt[i] = bt[i];
    }
    // The query: in float, scaled, for the float instance; as stored for the bfloat16 one, whose
    // scores come from the packed dot instruction (two products of bfloat16 pairs summed into a
    // float: a quarter of the unpack-and-multiply-add instructions) and are scaled after the sum.
    constexpr bool DOT2 = sizeof(T) == 2;
    float qv[VEC];
    uint4 qraw = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < VEC; ++i) qv[i] = 0.f;
    if (dvalid && kb < ke) {
        if (DOT2) {
            qraw = *reinterpret_cast<const uint4*>(q + (int64_t)t * q_stride + (int64_t)h * head_dim + d0);
        } else {
            Elem<T>::load_vec(q + (int64_t)t * q_stride + (int64_t)h * head_dim + d0, qv);
#pragma unroll
            for (int i = 0; i < VEC; ++i) qv[i] *= scale;
        }
    }
    const float post_scale = DOT2 ? scale : 1.f;
    const int kvh = h / (num_q_heads / num_kv_heads);
    const int64_t head_off = (int64_t)kvh * page_size * head_dim + d0;
    // a position encoding may add slope * (key position - query position) to this head's scores
    const float slope = head_slopes ? head_slopes[h] : 0.f;
    __syncthreads();

    float m = -INFINITY, l = 0.f, acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;

    // U keys of this lane group per round, two rounds in registers: one being used, one in flight
    constexpr int U = 4;
    uint4 kA[U], vA[U], kB[U], vB[U];
    const int round_keys = G * U;
    auto issue = [&](uint4* kr, uint4* vr, int j0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = j0 + u * G;
            if (j < ke && dvalid) {
                const int pi = j / page_size;
                const int64_t off = (int64_t)s_bt[pi - p_lo] * page_stride + head_off +
                                    (int64_t)(j - pi * page_size) * head_dim;
                kr[u] = *reinterpret_cast<const uint4*>(k_cache + off);
                vr[u] = *reinterpret_cast<const uint4*>(v_cache + off);
            } else {
                kr[u] = make_uint4(0, 0, 0, 0);
                vr[u] = make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto consume = [&](const uint4* kr, const uint4* vr, int j0) {
        float s[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float d = 0.f;
            if (DOT2) {
                d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr[u].x), __builtin_bit_cast(bf16x2, qraw.x), d, false);
                d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr[u].y), __builtin_bit_cast(bf16x2, qraw.y), d, false);
                d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr[u].z), __builtin_bit_cast(bf16x2, qraw.z), d, false);
                d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr[u].w), __builtin_bit_cast(bf16x2, qraw.w), d, false);
            } else {
                float kf[VEC];
                Elem<T>::unpack(kr[u], kf);
#pragma unroll
                for (int i = 0; i < VEC; ++i) d = fmaf(qv[i], kf[i], d);
            }
            s[u] = d;
        }
        float mn = m;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            s[u] = fmaf(slope, (float)(j0 + u * G - pos), group_sum<LPK>(s[u]) * post_scale);   // slope 0: the score itself
            if (j0 + u * G >= ke) s[u] = -INFINITY;      // the same for all lanes of a group
            mn = fmaxf(mn, s[u]);
        }
        const float alpha = exp_<ACC>(m - mn);           // m = -inf in the first round: 0
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] *= alpha;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float p = exp_<ACC>(s[u] - mn);        // a key past the end: exp(-inf) = 0
            psum += p;
            float vf[VEC];
            Elem<T>::unpack(vr[u], vf);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = fmaf(p, vf[i], acc[i]);
        }
        l = l * alpha + psum;
        m = mn;
    };
    {
        int j0 = kb + gi;                                // this group's first key; j0 < ke: it has work
        if (j0 < ke) issue(kA, vA, j0);
        while (j0 < ke) {
            if (j0 + round_keys < ke) issue(kB, vB, j0 + round_keys);
            consume(kA, vA, j0);
            j0 += round_keys;
            if (j0 >= ke) break;
            if (j0 + round_keys < ke) issue(kA, vA, j0 + round_keys);
            consume(kB, vB, j0);
            j0 += round_keys;
        }
    }

    if (sub == 0) { s_m[gi] = m; s_l[gi] = l; }
    if (dvalid) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) s_acc[gi * head_dim + d0 + i] = acc[i];
    }
    __syncthreads();

    // merge of the groups: common maximum, one weight per group, then the weighted sums
    const int nwaves = blockDim.x >> 6;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < G; i += blockDim.x) mx = fmaxf(mx, s_m[i]);
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, kWave));
    if (lane == 0) s_red[wave] = mx;
    __syncthreads();
    float M = -INFINITY;
    for (int w = 0; w < nwaves; ++w) M = fmaxf(M, s_red[w]);
    float lsum = 0.f;
    for (int i = threadIdx.x; i < G; i += blockDim.x) {
        const float mi = s_m[i];
        const float w = mi > -INFINITY ? exp_<ACC>(mi - M) : 0.f;
        s_m[i] = w;                                      // the group's weight takes its maximum's place
        lsum += w * s_l[i];
    }
    lsum = wave_sum(lsum);
    if (lane == 0) s_red[8 + wave] = lsum;
    __syncthreads();
    float L = 0.f;
    for (int w = 0; w < nwaves; ++w) L += s_red[8 + w];
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float o = 0.f;
#pragma unroll 4
        for (int i = 0; i < G; ++i) o = fmaf(s_m[i], s_acc[i * head_dim + d], o);
        const float res = L > 0.f ? o / L : 0.f;
        if (num_splits == 1) {
            Elem<T>::store(out + ((int64_t)t * num_q_heads + h) * head_dim + d, res);
        } else {
            const int64_t pidx = ((int64_t)ri * num_q_heads + h) * num_splits + split;
            part_o[pidx * head_dim + d] = res;
            if (d == 0) part_lse[pidx] = L > 0.f ? M + logf(L) : -INFINITY;
        }
    }
}

// out[t,h,:] = sum_s w_s * part_o[ri,h,s,:] / sum_s w_s,  w_s = exp(lse_s - max lse)
template <typename T>
__global__ __launch_bounds__(64) void attn_merge_kernel(
    T* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_lse,
    const int* __restrict__ row_ids, int num_q_heads, int head_dim, int num_splits) {
    const int64_t row = blockIdx.x;   // ri * num_q_heads + h
    const int64_t ri = row / num_q_heads, h = row - ri * num_q_heads;
    if (row_ids && row_ids[ri] < 0) return;        // padding entry: its partial results were never written
    const int64_t orow = (int64_t)(row_ids ? row_ids[ri] : ri) * num_q_heads + h;
    const float* lse = part_lse + row * num_splits;
    float M = -INFINITY;
    for (int s = 0; s < num_splits; ++s) M = fmaxf(M, lse[s]);
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float W = 0.f, o = 0.f;
        if (M > -INFINITY) {
            for (int s = 0; s < num_splits; ++s) {
                const float ls = lse[s];
                if (ls > -INFINITY) {
                    const float w = expf(ls - M);
                    W += w;
                    o += w * part_o[(row * num_splits + s) * head_dim + d];
                }
            }
        }
        Elem<T>::store(out + orow * head_dim + d, W > 0.f ? o / W : 0.f);
    }
}

template <typename T>
static int launch_rows(void* out, float* part_o, float* part_lse, const void* q, int64_t q_stride,
                       const void* k_cache, const void* v_cache, int64_t page_stride,
                       const int* row_ids, const int* token_item, const int* positions,
                       const int* block_table, const float* head_slopes,
                       int max_pages, int page_size, int num_tokens, int num_q_heads,
                       int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                       int num_waves, hipStream_t stream) {
    constexpr int VEC = Elem<T>::kVec;
    const int need = (head_dim + VEC - 1) / VEC;
    int lpk = 1;
    while (lpk < need) lpk <<= 1;
    ST_CHECK(lpk <= 64, "attention: head_dim %d is too large for this kernel (at most %d)",
             head_dim, 64 * VEC);
    const int G = num_waves * (64 / lpk);
    const size_t lds = (size_t)(2 * G + G * head_dim + 16 + max_pages) * sizeof(float);
    dim3 grid(num_q_heads, num_tokens, num_splits);
#define ST_ROWS(L)                                                                              \
    attn_rows_kernel<T, L><<<grid, num_waves * 64, lds, stream>>>((T*)out, part_o, part_lse, (const T*)q,  \
        q_stride, (const T*)k_cache, (const T*)v_cache, page_stride, row_ids, token_item, positions, \
        block_table, head_slopes, max_pages, page_size, num_q_heads, num_kv_heads, head_dim, scale, window, \
        num_splits)
    switch (lpk) {
        case 1: ST_ROWS(1); break;
        case 2: ST_ROWS(2); break;
        case 4: ST_ROWS(4); break;
        case 8: ST_ROWS(8); break;
        case 16: ST_ROWS(16); break;
        case 32: ST_ROWS(32); break;
        default: ST_ROWS(64); break;
    }
#undef ST_ROWS
    ST_LAUNCH_CHECK("attn_rows");
    if (num_splits > 1 && out) {      // without `out` the caller merges the partial results itself
        attn_merge_kernel<T><<<num_tokens * num_q_heads, 64, 0, stream>>>((T*)out, part_o, part_lse,
                                                                          row_ids, num_q_heads, head_dim,
                                                                          num_splits);
        ST_LAUNCH_CHECK("attn_merge");
    }
    return 0;
}

}  // namespace st

using namespace st;

// q: first query element of batch row 0; q_stride elements between rows.
// out: [rows of the batch, num_q_heads, head_dim] in the storage type.
// row_ids (optional, [num_tokens]): the batch rows to compute; otherwise rows
// 0..num_tokens-1.  token_item and positions are indexed by batch row.
// head_slopes (optional, [num_q_heads] floats): slope * (key position - query position) is added
// to the scaled scores of a head (a position encoding that biases scores by distance).
// part_o [num_tokens*num_q_heads*num_splits*head_dim] and part_lse
// [num_tokens*num_q_heads*num_splits] floats are needed when num_splits > 1; `out` may then be
// null: the splits are left unmerged in them (each partial normalised, with its log-sum-exp).
extern "C" int st_attn_rows(void* out, float* part_o, float* part_lse, const void* q, int64_t q_stride,
                            const void* k_cache, const void* v_cache, int64_t page_stride,
                            const int* row_ids, const int* token_item, const int* positions,
                            const int* block_table, const float* head_slopes,
                            int max_pages, int page_size, int num_tokens, int num_q_heads,
                            int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                            int num_waves, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0 && page_size > 0 &&
             max_pages > 0, "attention: bad sizes");
    ST_CHECK(num_q_heads % num_kv_heads == 0, "attention: %d query heads do not divide into %d key heads",
             num_q_heads, num_kv_heads);
    ST_CHECK(head_dim % 16 == 0, "attention: head_dim %d is not a multiple of 16", head_dim);
    ST_CHECK(num_splits >= 1 && num_splits <= 65535, "attention: bad num_splits %d", num_splits);
    ST_CHECK(num_tokens <= 65535, "attention: more than 65535 rows in one launch");
    ST_CHECK(num_splits == 1 || (part_o && part_lse), "attention: split needs partial buffers");
    ST_CHECK(out || num_splits > 1, "attention: no destination");
    ST_CHECK(window >= 0, "attention: negative window");
    ST_CHECK(num_waves == 4 || num_waves == 8, "attention: %d waves per workgroup (4 or 8)", num_waves);
    if (num_tokens == 0) return 0;
    if (dtype == kF32)
        return launch_rows<float>(out, part_o, part_lse, q, q_stride, k_cache, v_cache, page_stride,
                                  row_ids, token_item, positions, block_table, head_slopes, max_pages, page_size, num_tokens,
                                  num_q_heads, num_kv_heads, head_dim, scale, window, num_splits, num_waves, stream);
    if (dtype == kBF16)
        return launch_rows<bf16_t>(out, part_o, part_lse, q, q_stride, k_cache, v_cache, page_stride,
                                   row_ids, token_item, positions, block_table, head_slopes, max_pages, page_size, num_tokens,
                                   num_q_heads, num_kv_heads, head_dim, scale, window, num_splits, num_waves, stream);
    ST_CHECK(false, "attention: unknown dtype %d", dtype);
    return 0;
}

extern "C" int st_attn_rows_static_init() {
    float* p = nullptr;
    return static_scratch(&p);
}

extern "C" size_t st_attn_rows_static_capacity() { return kStaticScratchFloats * sizeof(float); }

// st_attn_rows with the key split's partial results in the library's own static scratch
// instead of a caller's workspace: nothing here allocates.  Every workgroup of the row kernel
// writes its own partial result and log-sum-exp before the merge reads them, so nothing in the
// scratch has to start at zero; it keeps the last call's contents, and two calls that overlap
// on one GPU (different streams, or threads) race for it.
extern "C" int st_attn_rows_static(void* out, const void* q, int64_t q_stride,
                                   const void* k_cache, const void* v_cache, int64_t page_stride,
                                   const int* row_ids, const int* token_item, const int* positions,
                                   const int* block_table, const float* head_slopes,
                                   int max_pages, int page_size, int num_tokens, int num_q_heads,
                                   int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                                   int num_waves, int dtype, hipStream_t stream) {
    ST_CHECK(out, "attention: no destination");
    ST_CHECK(num_tokens >= 0 && num_q_heads > 0 && head_dim > 0 && num_splits >= 1, "attention: bad sizes");
    float* part_o = nullptr;
    float* part_lse = nullptr;
    if (num_splits > 1) {
        const size_t rows = (size_t)num_tokens * (size_t)num_q_heads * (size_t)num_splits;
        const size_t need = rows * ((size_t)head_dim + 1);
        ST_CHECK(need <= kStaticScratchFloats,
                 "attention: %d rows x %d heads x %d splits x (%d + 1) floats = %zu bytes of partial results "
                 "exceed the static scratch of %zu bytes", num_tokens, num_q_heads, num_splits, head_dim,
                 need * sizeof(float), kStaticScratchFloats * sizeof(float));
        float* base = nullptr;
        if (static_scratch(&base) != 0) return 1;
        part_o = base;
        part_lse = base + rows * (size_t)head_dim;
    }
    return st_attn_rows(out, part_o, part_lse, q, q_stride, k_cache, v_cache, page_stride, row_ids,
                        token_item, positions, block_table, head_slopes, max_pages, page_size, num_tokens, num_q_heads,
                        num_kv_heads, head_dim, scale, window, num_splits, num_waves, dtype, stream);
}
