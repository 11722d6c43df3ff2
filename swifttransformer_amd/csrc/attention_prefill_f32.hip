// Attention of prompt portions over the paged cache, 32-bit throughout: the float twin of
// attention_prefill.hip.  Same tiles (64 consecutive query rows of one batch item and one
// head to a workgroup, 16 rows to a wave), same key blocks of 64 shared through LDS, same
// transposed formulation, with the float matrix instruction (v_mfma_f32_16x16x4_f32: float
// operands, float accumulation, no reduced-precision mode) and the accurate expf.
//
//   S^T = K Q^T : A = 16 keys x 4 dims, B = Q^T.  The instruction's four "k" slots belong to
//                 the four lane groups g; slot g of product (j, i) is given dim 16j + 4g + i, so
//                 that a lane reads its four values of four consecutive products as one float4
//                 (any assignment of dims to slots is right as long as A and B agree).
//                 A lane ends up with S^T[key 4g+r][query l%16] of each 16-key subtile.
//   O^T += V^T P^T : slot g of product i of subtile t is key 16t + 4g + i: the B operand is
//                 the lane's own probability r = i, and A a float4 of the transposed V block.
//
// Reference: the float branch of src/csrc/kernel/fused_context_stage_attention.cu:266-280 and
// :405-449 (plain multiply-adds on whole prompts); masked scores are -inf here and the
// normaliser exact, as in the bfloat16 kernel.
#include "common.h"
#include "api.h"

namespace st {

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int PQ = 64;              // query rows per tile
constexpr int PK = 64;              // keys per block
constexpr int VT_STRIDE = PK + 4;   // floats between rows of the transposed V block

// DT = head_dim / 16
template <int DT>
__global__ __launch_bounds__(256) void attn_prefill_f32_kernel(
    float* __restrict__ out, const float* __restrict__ q, int64_t q_stride,
    const float* __restrict__ k_cache, const float* __restrict__ v_cache, int64_t page_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_start, const int* __restrict__ item_len,
    const int* __restrict__ block_table, const float* __restrict__ head_slopes, int max_pages, int page_size,
    int num_q_heads, int num_kv_heads, float scale, int window, int num_tiles, int deal_period) {
    constexpr int HD = 16 * DT;
    constexpr int K_STRIDE = HD + 4;                 // floats between keys of the K block
    extern __shared__ uint4 dyn[];
    float* ks = reinterpret_cast<float*>(dyn);       // K [PK][K_STRIDE]
    float* vt = ks + PK * K_STRIDE;                  // V^T [HD][VT_STRIDE]
    int* s_bt = reinterpret_cast<int*>(vt + HD * VT_STRIDE);   // [max_pages]

    const int h = blockIdx.x;
    // grid row -> tile as in the bfloat16 kernel: the whole launch is resident at once, so tiles
    // (listed in order of their work) are dealt to the compute units in serpentine order, rows of
    // `deal_period` tiles from the list's heavy end, every other row backwards
    int tile;
    {
        const int slot = blockIdx.y, row = slot / deal_period, base = row * deal_period;
        const int in_row = min(deal_period, num_tiles - base), c = slot - base;
        tile = num_tiles - 1 - (base + ((row & 1) ? in_row - 1 - c : c));
    }
    const int item = tile_item[tile], q0 = tile_q0[tile];
    if (item < 0) return;                            // a padding entry of a tile list of fixed length
    const int start = item_start[item], n = item_len[item], row0 = item_tok_off[item];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, r16 = lane & 15;
    const int kvh = h / (num_q_heads / num_kv_heads);
    // a position encoding may add slope * (key position - query position) to this head's scaled scores
    const float slope = head_slopes ? head_slopes[h] : 0.f;

    const int qi = q0 + wave * 16 + r16;             // this lane's query row within the item
    const bool qvalid = qi < n;
    const int qpos = start + qi;
    const int rows_in_tile = min(PQ, n - q0);
    const int pos_first = start + q0, pos_last = start + q0 + rows_in_tile - 1;
    const int key_lo = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;
    const int key_hi = pos_last + 1;                 // exclusive

    {
        const int p_lo = key_lo / page_size, p_hi = (key_hi - 1) / page_size;
        const int* bt = block_table + (int64_t)item * max_pages;
        for (int i = p_lo + tid; i <= p_hi; i += 256) s_bt[i] = bt[i];
    }
    // Q^T: lane (query r16, group g) holds dims 16j + 4g .. +3
    floatx4 qf[DT];
    {
        const float* qrow = q + (int64_t)(row0 + (qvalid ? qi : q0)) * q_stride + (int64_t)h * HD;
#pragma unroll
        for (int j = 0; j < DT; ++j)
            qf[j] = qvalid ? *reinterpret_cast<const floatx4*>(qrow + 16 * j + 4 * g) : floatx4{0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY, l = 0.f;
    floatx4 acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Staging: a thread moves DT 16-byte pieces of ONE key (key = 16 * wave + lane % 16, pieces
    // lane / 16 + 4 * it); a wave's stores into the transposed V block (16 keys x 4 pieces)
    // fall on 64 different banks.  The next block's pieces travel while this one is consumed.
    const int my_key = 16 * wave + r16;
    floatx4 sk[DT], sv[DT];
    auto fetch = [&](int kb) {
        const int j = kb + my_key;
        if (j >= key_lo && j < key_hi) {
            const int pi = j / page_size;
            const int64_t off = (int64_t)s_bt[pi] * page_stride +
                                ((int64_t)kvh * page_size + (j - pi * page_size)) * HD + 4 * g;
#pragma unroll
            for (int it = 0; it < DT; ++it) {
                sk[it] = *reinterpret_cast<const floatx4*>(k_cache + off + 16 * it);
                sv[it] = *reinterpret_cast<const floatx4*>(v_cache + off + 16 * it);
            }
        } else {                                     // never NaN * 0: keys outside are zeros
#pragma unroll
            for (int it = 0; it < DT; ++it) { sk[it] = floatx4{0.f, 0.f, 0.f, 0.f}; sv[it] = sk[it]; }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int it = 0; it < DT; ++it) {
            const int d = 16 * it + 4 * g;
            *reinterpret_cast<floatx4*>(ks + my_key * K_STRIDE + d) = sk[it];
#pragma unroll
            for (int e = 0; e < 4; ++e) vt[(d + e) * VT_STRIDE + my_key] = sv[it][e];
        }
    };
    const int wave_first = pos_first + wave * 16;
    const int wave_last = min(pos_last, wave_first + 15);

    auto consume = [&](int kb) {
        if (kb > wave_last) return;                  // nothing here for this wave
        // ---- S^T: st[t][r] = q . k of key kb + 16t + 4g + r with this lane's query
        floatx4 st[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < DT; ++j) {
            floatx4 a[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                a[t] = *reinterpret_cast<const floatx4*>(ks + (16 * t + r16) * K_STRIDE + 16 * j + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][i], qf[j][i], st[t], 0, 0, 0);
        }
        // ---- scale, distance bias of the head if any, mask, online softmax (a lane's values all
        // belong to one query row)
        float bmax = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = kb + 16 * t + 4 * g + r;
                const bool ok = qvalid && j <= qpos && j >= key_lo && (window <= 0 || j > qpos - window);
                const float s = ok ? fmaf(slope, (float)(j - qpos), st[t][r] * scale) : -INFINITY;   // slope 0: the score itself
                st[t][r] = s;
                bmax = fmaxf(bmax, s);
            }
        bmax = rows4_max(bmax);
        const float mn = fmaxf(m, bmax);
        const float msafe = mn == -INFINITY ? 0.f : mn;          // a row with nothing visible yet
        const float alpha = expf(m - msafe);                     // m = -inf: 0
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = expf(st[t][r] - msafe);          // masked: 0
                st[t][r] = p;
                psum += p;
            }
        l = l * alpha + psum;                                     // this lane's keys only; summed at the end
        m = mn;
        // ---- O^T = O^T * alpha + V^T P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt] *= alpha;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            floatx4 a[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                a[dt] = *reinterpret_cast<const floatx4*>(vt + (16 * dt + r16) * VT_STRIDE + 16 * t + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[dt][i], st[t][i], acc[dt], 0, 0, 0);
        }
    };

    const int kb_first = (key_lo / PK) * PK;
    __syncthreads();                                 // the block table is in LDS
    fetch(kb_first);
    for (int kb = kb_first; kb < key_hi; kb += PK) {
        __syncthreads();                             // previous block fully consumed
        stash();
        __syncthreads();
        if (kb + PK < key_hi) fetch(kb + PK);
        consume(kb);
    }
    // acc[dt][r] = O[query r16][dim 16dt + 4g + r]
    l = rows4_sum(l);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (qvalid) {
        float* orow = out + ((int64_t)(row0 + qi) * num_q_heads + h) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<floatx4*>(orow + 16 * dt + 4 * g) = acc[dt] * inv;
    }
}

constexpr size_t kMaxLds = 156 * 1024;

template <int DT>
int launch(float* out, const float* q, int64_t q_stride, const float* k_cache, const float* v_cache,
           int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
           const int* item_tok_off, const int* item_start, const int* item_len, const int* block_table,
           const float* head_slopes, int max_pages, int page_size, int num_q_heads, int num_kv_heads, float scale,
           int window, hipStream_t stream) {
    constexpr int HD = 16 * DT;
    auto kernel = attn_prefill_f32_kernel<DT>;
    const size_t lds = (size_t)(PK * (HD + 4) + HD * VT_STRIDE) * sizeof(float) + (size_t)max_pages * sizeof(int);
    ST_CHECK(lds <= kMaxLds, "attn_prefill: a block table of %d pages does not fit LDS beside float blocks of head_dim %d",
             max_pages, HD);
    if (lds > 48 * 1024) {
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
            ST_CHECK(e == hipSuccess, "attn_prefill: cannot raise the LDS limit: %s", hipGetErrorString(e));
            raised = true;
        }
    }
    // workgroups with equal (linear index mod compute units) share a compute unit
    const int compute_units = device_compute_units();
    const int deal_period = compute_units / num_q_heads > 0 ? compute_units / num_q_heads : 1;
    kernel<<<dim3(num_q_heads, num_tiles), 256, lds, stream>>>(
        out, q, q_stride, k_cache, v_cache, page_stride, tile_item, tile_q0, item_tok_off, item_start, item_len,
        block_table, head_slopes, max_pages, page_size, num_q_heads, num_kv_heads, scale, window, num_tiles,
        deal_period);
    ST_LAUNCH_CHECK("attn_prefill (float)");
    return 0;
}

}  // namespace

// The float instance behind st_attn_prefill; arguments as there (already checked by it).
int attn_prefill_f32(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                     int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                     const int* item_tok_off, const int* item_start, const int* item_len,
                     const int* block_table, const float* head_slopes, int max_pages, int page_size,
                     int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, hipStream_t stream) {
    ST_CHECK(q_stride % 4 == 0 && ((uintptr_t)q & 15) == 0, "attn_prefill: query rows must be 16-byte aligned");
#define ST_PF(D) case D: return launch<D>((float*)out, (const float*)q, q_stride, (const float*)k_cache,          \
        (const float*)v_cache, page_stride, tile_item, tile_q0, num_tiles, item_tok_off, item_start, item_len,    \
        block_table, head_slopes, max_pages, page_size, num_q_heads, num_kv_heads, scale, window, stream)
    switch (head_dim / 16) {
        ST_PF(1); ST_PF(2); ST_PF(3); ST_PF(4); ST_PF(5); ST_PF(6); ST_PF(7); ST_PF(8);
        ST_PF(9); ST_PF(10); ST_PF(11); ST_PF(12); ST_PF(13); ST_PF(14); ST_PF(15); ST_PF(16);
        default: break;
    }
#undef ST_PF
    ST_CHECK(false, "attn_prefill: head_dim %d is not a multiple of 16 in [16, 256]", head_dim);
    return -1;
}

}  // namespace st
