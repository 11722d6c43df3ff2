// Attention of prompt portions over the paged cache on the matrix cores (bfloat16).
//
// A workgroup takes a tile of 64 consecutive query rows of one batch item and one query
// head; four waves take 16 rows each.  With KS > 1 the workgroup has KS such groups of four
// waves, each going through its own contiguous share of the tile's key blocks (its own LDS
// buffer); their partial results are merged through LDS at the end.  That shortens the
// longest chain of dependent key blocks, which is what bounds the kernel when few tiles are
// in flight: a late tile of a long prompt, or a portion that attends to a long cache.  The portion's own keys and values are already
// in the cache, so the keys of a row at position p are simply the cached positions
// [lo, p] of its request (lo > 0 only with a window), read through the block table in
// blocks of 64 keys that all four waves share through LDS.  Softmax is online in float;
// both products accumulate in float.
//
// Formulation (transposed, so that no operand needs a shuffle between the two products):
//   S^T = K Q^T : MFMA 16x16x32 with A = 16 keys x 32 dims (from LDS), B = Q^T (registers).
//                 A lane ends up with S^T[key 4g+r][query l%16]: all its values belong to
//                 ONE query row, so max, sum and rescale are per-lane scalars plus two
//                 lane shuffles (across the four groups g).
//   O^T += V^T P^T : A = V^T (16 dims x 32 keys, from a transposed LDS copy of V),
//                 B = P^T taken straight from the S^T registers: a lane's 8 values of two
//                 16-key subtiles serve as its 8 "k" entries; V^T is read with the same
//                 key order, and a sum does not depend on the order of its terms.
//
// Reference: src/csrc/kernel/fused_context_stage_attention.cu:87-453 (16x16 WMMA tiles,
// additive mask -10000 :287-291, denominators l + 1e-6 :362-363, half accumulation of PV,
// whole prompts only, keys from the QKV buffer) and the xformers call it uses for half
// precision (src/csrc/kernel/xformers_attention.cu:345-391).  Here masked scores are
// -inf, the normaliser is exact, and a portion may start anywhere in its request.
//
// Balance: a tile's work grows with its position (causal), and a launch of this size is
// resident all at once (four workgroups a compute unit), so no dispatcher evens it out: with
// tiles in plain order the compute units that hold the long tiles run four times as long as
// the others.  Workgroups are handed out round-robin, so workgroups whose linear indices are
// congruent modulo the number of compute units share one.  With the tile list ordered by
// work (the caller's business; a single prompt is already ordered) the kernel deals the tiles
// to grid rows in serpentine order with that period: each compute unit gets a long, a short
// and two middling ones.  If the hardware places workgroups otherwise only the balance
// suffers.  The head is the fast grid index so that the workgroups of a head, which share its
// keys and values, land on the same XCD and its L2.
#include "common.h"
#include "api.h"

namespace st {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int PQ = 64;     // query rows per tile
constexpr int PK = 64;     // keys per block
constexpr int VT_STRIDE = PK + 4;   // elements between rows of the transposed V block

// HDP = ceil(head_dim / 32): number of 32-wide steps over the head dimension
// (small heads: four waves a SIMD are asked of the compiler, i.e. at most 128 registers a lane)
template <int HDP, int KS>
__global__ __launch_bounds__(256 * KS, HDP <= 2 ? 4 : 1) void attn_prefill_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, int64_t page_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_start, const int* __restrict__ item_len,
    const int* __restrict__ block_table, const float* __restrict__ head_slopes, int max_pages, int page_size,
    int page_shift, int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, int num_tiles,
    int deal_period) {
    constexpr int KS_STRIDE = 32 * HDP + 8;          // elements between keys of the K block
    extern __shared__ uint4 dyn[];
    constexpr int BUF = PK * KS_STRIDE + (32 * HDP) * VT_STRIDE;   // elements of the block buffer
    bf16_t* lds_all = reinterpret_cast<bf16_t*>(dyn);            // per wave group: K [PK][KS_STRIDE], V^T [head_dim][VT_STRIDE]
    int* s_bt = reinterpret_cast<int*>(lds_all + KS * BUF);      // then [max_pages]

    const int h = blockIdx.x;
    // grid row -> tile: rows of `deal_period` tiles of the list taken from its heavy end,
    // every other row backwards
    int tile;
    {
        const int slot = blockIdx.y, row = slot / deal_period, base = row * deal_period;
        const int in_row = min(deal_period, num_tiles - base), c = slot - base;
        tile = num_tiles - 1 - (base + ((row & 1) ? in_row - 1 - c : c));
    }
    const int item = tile_item[tile], q0 = tile_q0[tile];
    if (item < 0) return;                            // a padding entry of a tile list of fixed length
    const int start = item_start[item], n = item_len[item], row0 = item_tok_off[item];
    const int part = threadIdx.x >> 8;                // wave group: its share of the key blocks
    bf16_t* lds0 = lds_all + part * BUF;
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;   // within the wave group
    const int g = lane >> 4, r16 = lane & 15;
    const int kvh = h / (num_q_heads / num_kv_heads);
    const int DT = head_dim >> 4;                    // 16-wide output subtiles

    // this lane's query row (all of a lane's scores belong to it)
    const int qi = q0 + wave * 16 + r16;             // row within the item
    const bool qvalid = qi < n;
    const int qpos = start + qi;                     // its position in the request
    // keys needed by the tile
    const int rows_in_tile = min(PQ, n - q0);
    const int pos_first = start + q0, pos_last = start + q0 + rows_in_tile - 1;
    const int key_lo = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;
    const int key_hi = pos_last + 1;                 // exclusive

    // block table of the request -> LDS
    {
        const int p_lo = key_lo / page_size, p_hi = (key_hi - 1) / page_size;
        const int* bt = block_table + (int64_t)item * max_pages;
        for (int i = p_lo + (int)threadIdx.x; i <= p_hi; i += 256 * KS) s_bt[i] = bt[i];
    }
    // Q^T fragments: lane (query r16, group g) holds dims 32*s + 8g .. +7, pre-scaled scores come later
    bf16x8 qf[HDP];
    {
        const bf16_t* qrow = q + (int64_t)(row0 + (qvalid ? qi : q0)) * q_stride + (int64_t)h * head_dim;
#pragma unroll
        for (int s = 0; s < HDP; ++s) {
            const int d = 32 * s + 8 * g;
            qf[s] = (qvalid && d < head_dim) ? __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(qrow + d))
                                             : __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
        }
    }
    // zero the padding dims of the K block once (head_dim not a multiple of 32)
    if ((head_dim & 31) != 0) {
        for (int i = tid; i < PK * 16; i += 256) {
            const int key = i >> 4, e = i & 15;
            lds0[key * KS_STRIDE + head_dim + e].bits = 0;
        }
    }

    float m = -INFINITY, l = 0.f;
    floatx4 acc[2 * HDP];
#pragma unroll
    for (int i = 0; i < 2 * HDP; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Staging of a block: a thread moves one 16-byte chunk (8 dims) of TWO neighbouring keys, so
    // that the transposed copy of V is written as pairs (one dword = dims d of keys 2p, 2p+1).
    // A wave holds 16 key pairs x 4 chunks: its dword stores then fall on 64 different banks.
    // The next block's chunks are fetched into registers while the current block is consumed.
    constexpr int ITER = (HDP + 1) / 2;              // 128 work items (32 pairs x 4 chunks) per 128 threads
    const int chunks = head_dim >> 3;                // 16-byte chunks per key
    struct Stage { uint4 k0, k1, v0, v1; };
    // the next block (small heads: the next two), in flight during the products
    constexpr int PF = HDP <= 2 ? 2 : 1;
    Stage stg0[ITER], stg1[PF == 2 ? ITER : 1];
    auto item_of = [&](int it, int& kp, int& ch) {
        const int i = tid + it * 256;
        kp = (i & 15) + 16 * ((i >> 6) & 1);
        ch = ((i >> 4) & 3) + 4 * (i >> 7);
    };
    // A page size that is a power of two from 2 to 64 keeps a key pair inside one page and a
    // block's pages aligned to it: the address of a thread's chunk is then its page's base plus
    // a constant, one table look-up and one multiply-add per pair and block.
    const bool fast_pages = page_shift >= 1 && page_size <= PK;
    int64_t pair_const[ITER];                        // offset of the pair's first key inside its page, in elements
    int pair_page[ITER];                             // page index of the pair relative to the block's first page
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        int kp, ch;
        item_of(it, kp, ch);
        pair_page[it] = fast_pages ? (2 * kp) >> page_shift : 0;
        pair_const[it] = ((int64_t)kvh * page_size + ((2 * kp) & (page_size - 1))) * head_dim + ch * 8;
    }
    auto fetch = [&](Stage* stg, int kb) {
        if (fast_pages && kb >= key_lo && kb + PK <= key_hi) {     // a whole block of valid keys
            const int first_page = kb >> page_shift;
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                int kp, ch;
                item_of(it, kp, ch);
                if (ch < chunks) {
                    const int64_t off = (int64_t)s_bt[first_page + pair_page[it]] * page_stride + pair_const[it];
                    stg[it].k0 = *reinterpret_cast<const uint4*>(k_cache + off);
                    stg[it].k1 = *reinterpret_cast<const uint4*>(k_cache + off + head_dim);
                    stg[it].v0 = *reinterpret_cast<const uint4*>(v_cache + off);
                    stg[it].v1 = *reinterpret_cast<const uint4*>(v_cache + off + head_dim);
                }
            }
            return;
        }
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            int kp, ch;
            item_of(it, kp, ch);
            const uint4 z = make_uint4(0, 0, 0, 0);
            stg[it].k0 = z; stg[it].k1 = z; stg[it].v0 = z; stg[it].v1 = z;
            if (ch < chunks) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int j = kb + 2 * kp + half;
                    if (j >= key_lo && j < key_hi) {
                        const int pi = page_shift >= 0 ? (j >> page_shift) : j / page_size;
                        const int64_t off = (int64_t)s_bt[pi] * page_stride +
                                            ((int64_t)kvh * page_size + (j - pi * page_size)) * head_dim + ch * 8;
                        const uint4 kk = *reinterpret_cast<const uint4*>(k_cache + off);
                        const uint4 vv = *reinterpret_cast<const uint4*>(v_cache + off);
                        if (half == 0) { stg[it].k0 = kk; stg[it].v0 = vv; } else { stg[it].k1 = kk; stg[it].v1 = vv; }
                    }
                }
            }
        }
    };
    auto stash = [&](const Stage* stg, int buf) {
        bf16_t* ks = lds0 + buf * BUF;
        uint32_t* vt32 = reinterpret_cast<uint32_t*>(ks + PK * KS_STRIDE);
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            int kp, ch;
            item_of(it, kp, ch);
            if (ch < chunks) {
                *reinterpret_cast<uint4*>(ks + (2 * kp) * KS_STRIDE + ch * 8) = stg[it].k0;
                *reinterpret_cast<uint4*>(ks + (2 * kp + 1) * KS_STRIDE + ch * 8) = stg[it].k1;
                const uint32_t a0[4] = {stg[it].v0.x, stg[it].v0.y, stg[it].v0.z, stg[it].v0.w};
                const uint32_t a1[4] = {stg[it].v1.x, stg[it].v1.y, stg[it].v1.z, stg[it].v1.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    // dims ch*8 + 2e and + 2e+1 of keys 2kp (low half) and 2kp+1 (high half)
                    vt32[((ch * 8 + 2 * e) * VT_STRIDE) / 2 + kp] = (a0[e] & 0xffffu) | (a1[e] << 16);
                    vt32[((ch * 8 + 2 * e + 1) * VT_STRIDE) / 2 + kp] = (a0[e] >> 16) | (a1[e] & 0xffff0000u);
                }
            }
        }
    };
    // last key this wave's rows can see: blocks and 16-key subtiles beyond it are skipped
    const int wave_first = pos_first + wave * 16;
    const int wave_last = min(pos_last, wave_first + 15);
    const float sl = scale * 1.44269504088896340736f;            // scores in units of log2
    // A position encoding may add slope * (key position - query position) to this head's scaled
    // scores.  The scores of such a head are turned into their final log2 units right after the
    // product (c = 1 from then on); all others stay raw and are scaled inside the exponential.
    const float bias_l2 = head_slopes ? head_slopes[h] * 1.44269504088896340736f : 0.f;
    const bool biased = bias_l2 != 0.f;
    const float c = biased ? 1.f : sl;

    auto consume = [&](int kb, int buf) {
        if (kb > wave_last) return;                  // nothing here for this wave
        const bf16_t* ks = lds0 + buf * BUF;
        const bf16_t* vt = ks + PK * KS_STRIDE;
        // ---- S^T subtiles: st[t][r] = score of key kb + 16t + 4g + r with this lane's query.
        // No branch in here: the four subtiles' products are independent chains, and only as one
        // straight run of instructions do their LDS reads and MFMAs overlap (a subtile beyond the
        // wave's last row is computed for nothing and masked below).
        floatx4 st[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < HDP; ++s) {
            bf16x8 a[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                a[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
                    ks + (16 * t + r16) * KS_STRIDE + 32 * s + 8 * g));
#pragma unroll
            for (int t = 0; t < 4; ++t)
                st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], qf[s], st[t], 0, 0, 0);
        }
        // ---- mask, online softmax (per lane = per query row, then across the 4 groups).
        // The maximum is tracked in raw score units; a probability is exp2(s*c - m*c) with
        // c = scale * log2(e): one multiply-add and one exp2 per score.  Blocks entirely visible
        // to all rows of the wave (the common case away from the diagonal and the window's
        // edge) skip the masking.
        if (biased) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    st[t][r] = fmaf(st[t][r], sl, bias_l2 * (float)(kb + 16 * t + 4 * g + r - qpos));
        }
        const bool interior = kb + PK - 1 <= wave_first && kb >= key_lo &&
                              (window <= 0 || kb > wave_last - window);
        float bmax = -INFINITY;
        if (interior) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) bmax = fmaxf(bmax, st[t][r]);
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = kb + 16 * t + 4 * g + r;
                    const bool ok = qvalid && j <= qpos && j >= key_lo && (window <= 0 || j > qpos - window);
                    const float sv = ok ? st[t][r] : -INFINITY;
                    st[t][r] = sv;
                    bmax = fmaxf(bmax, sv);
                }
        }
        bmax = rows4_max(bmax);
        const float mn = fmaxf(m, bmax);
        const float msafe = mn == -INFINITY ? 0.f : mn;          // a row with nothing visible yet
        const float mc = msafe * c;
        const float alpha = __builtin_amdgcn_exp2f(m * c - mc);   // m = -inf: 0
        float psum = 0.f;
        bf16x8 pf[2];                                             // P^T fragments of key halves 0-31, 32-63
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            uint32_t packed[4];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int t = 2 * u + half;
                float p[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[r] = __builtin_amdgcn_exp2f(fmaf(st[t][r], c, -mc));
                    psum += p[r];
                }
                packed[2 * half] = pack_bf16x2(p[0], p[1]);
                packed[2 * half + 1] = pack_bf16x2(p[2], p[3]);
            }
            pf[u] = __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
        }
        l = l * alpha + psum;                                     // this lane's keys only; summed at the end
        m = mn;
        // ---- O^T = O^T * alpha + V^T P^T, again without a branch: all subtiles of the head
        // dimension (a last one beyond head_dim works on unwritten LDS and is never stored), key
        // halves outermost so that consecutive MFMAs belong to different accumulators
#pragma unroll
        for (int dt = 0; dt < 2 * HDP; ++dt) acc[dt] *= alpha;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int dt = 0; dt < 2 * HDP; ++dt) {
                // this lane's 8 keys of half u: 32u + 4g + {0..3} and 32u + 16 + 4g + {0..3}
                const bf16_t* vrow = vt + (16 * dt + r16) * VT_STRIDE + 32 * u + 4 * g;
                const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
                const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 16);
                const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf[u], acc[dt], 0, 0, 0);
            }
        }
    };

    // Block i+1 travels from memory into registers while block i is consumed from LDS.
    // The tile's key blocks are dealt to the wave groups in KS contiguous shares; every group
    // goes through the loop the same number of times (the barriers are the workgroup's).
    const int kb_first = (key_lo / PK) * PK;
    const int nblk = (key_hi - kb_first + PK - 1) / PK;
    const int per = (nblk + KS - 1) / KS;
    const int kb0 = kb_first + part * per * PK;
    const int kb_end = min(key_hi, kb0 + per * PK);  // this group's keys end here
    __syncthreads();                                 // the block table is in LDS
    if (kb0 < kb_end) fetch(stg0, kb0);
    if (PF == 2 && kb0 + PK < kb_end) fetch(stg1, kb0 + PK);
    if (PF == 2) {
        // two blocks ahead: two register sets used in turn (unrolled by two so that each keeps its name)
        for (int it = 0; it < per; it += 2) {
            const int kb = kb0 + it * PK;
            __syncthreads();                         // previous block fully consumed
            stash(stg0, 0);
            __syncthreads();
            if (kb + 2 * PK < kb_end) fetch(stg0, kb + 2 * PK);
            if (kb < kb_end) consume(kb, 0);
            if (it + 1 >= per) break;
            __syncthreads();
            stash(stg1, 0);
            __syncthreads();
            if (kb + 3 * PK < kb_end) fetch(stg1, kb + 3 * PK);
            if (kb + PK < kb_end) consume(kb + PK, 0);
        }
    } else {
        for (int it = 0; it < per; ++it) {
            const int kb = kb0 + it * PK;
            __syncthreads();                         // previous block fully consumed
            stash(stg0, 0);
            __syncthreads();
            if (kb + PK < kb_end) fetch(stg0, kb + PK);
            if (kb < kb_end) consume(kb, 0);
        }
    }
    // the wave groups' partial results (maximum, this lane's share of the normaliser, this lane's
    // share of the output) meet in LDS; the first group merges them
    if (KS > 1) {
        constexpr int E = 2 + 8 * HDP;                // floats per lane
        float* mg = reinterpret_cast<float*>(lds_all);
        __syncthreads();                             // every group has consumed its last block
        if (part > 0) {
            float* dst = mg + (size_t)((part - 1) * 4 + wave) * E * 64 + lane;
            dst[0] = m;
            dst[64] = l;
#pragma unroll
            for (int dt = 0; dt < 2 * HDP; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(2 + 4 * dt + r) * 64] = acc[dt][r];
        }
        __syncthreads();
        if (part > 0) return;
#pragma unroll
        for (int p = 1; p < KS; ++p) {
            const float* src = mg + (size_t)((p - 1) * 4 + wave) * E * 64 + lane;
            const float mo = src[0], lo = src[64];
            const float mn = fmaxf(m, mo);
            const float msafe = mn == -INFINITY ? 0.f : mn;
            const float a = __builtin_amdgcn_exp2f((m - msafe) * c), b = __builtin_amdgcn_exp2f((mo - msafe) * c);
            l = l * a + lo * b;
#pragma unroll
            for (int dt = 0; dt < 2 * HDP; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[dt][r] = acc[dt][r] * a + src[(2 + 4 * dt + r) * 64] * b;
            m = mn;
        }
    }
    // acc[dt][r] = O[query r16][dim 16dt + 4g + r]
    l = rows4_sum(l);                                // the row's normaliser from its four lanes
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (qvalid) {
        bf16_t* orow = out + ((int64_t)(row0 + qi) * num_q_heads + h) * head_dim;
#pragma unroll
        for (int dt = 0; dt < 2 * HDP; ++dt) {
            if (dt < DT) {
                uint2 p;
                p.x = pack_bf16x2(acc[dt][0] * inv, acc[dt][1] * inv);
                p.y = pack_bf16x2(acc[dt][2] * inv, acc[dt][3] * inv);
                *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * g) = p;
            }
        }
    }
}

constexpr size_t kPrefillMaxLds = 128 * 1024;

// bytes of LDS of a workgroup with KS wave groups: their block buffers (which also hold the
// merge of the groups' results at the end) and the request's block table
static size_t prefill_lds(int hdp, int ks, int max_pages) {
    const size_t buf = (size_t)(PK * (32 * hdp + 8) + (32 * hdp) * VT_STRIDE) * sizeof(bf16_t);
    const size_t merge = (size_t)(ks - 1) * 256 * (2 + 8 * hdp) * sizeof(float);
    return (ks * buf > merge ? ks * buf : merge) + (size_t)max_pages * sizeof(int);
}

template <int HDP, int KS>
static int launch_prefill(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                          int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                          const int* item_tok_off, const int* item_start, const int* item_len,
                          const int* block_table, const float* head_slopes, int max_pages, int page_size,
                          int num_q_heads, int num_kv_heads, int head_dim, float scale, int window,
                          hipStream_t stream) {
    auto kernel = attn_prefill_kernel<HDP, KS>;
    const size_t lds = prefill_lds(HDP, KS, max_pages);
    if (lds > 48 * 1024) {
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPrefillMaxLds);
            ST_CHECK(e == hipSuccess, "attn_prefill: cannot raise the LDS limit: %s", hipGetErrorString(e));
            raised = true;
        }
    }
    ST_CHECK(lds <= kPrefillMaxLds, "attn_prefill: a block table of %d pages does not fit LDS", max_pages);
    int page_shift = -1;                             // log2(page_size) when it is a power of two
    if ((page_size & (page_size - 1)) == 0)
        for (page_shift = 0; (1 << page_shift) < page_size; ++page_shift) {}
    // workgroups with equal (linear index mod compute units) share a compute unit: that many
    // grid rows apart
    const int compute_units = device_compute_units();
    const int deal_period = compute_units / num_q_heads > 0 ? compute_units / num_q_heads : 1;
    kernel<<<dim3(num_q_heads, num_tiles), 256 * KS, lds, stream>>>(
        (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, page_stride,
        tile_item, tile_q0, item_tok_off, item_start, item_len, block_table, head_slopes, max_pages, page_size,
        page_shift, num_q_heads, num_kv_heads, head_dim, scale, window, num_tiles, deal_period);
    ST_LAUNCH_CHECK("attn_prefill");
    return 0;
}

// How many wave groups share a tile's key blocks: more when few tiles are in flight (their
// chains of blocks are then what takes the time), as far as LDS allows.
static int prefill_key_split(int hdp, int num_tiles, int num_q_heads, int max_pages) {
    const int64_t workgroups = (int64_t)num_tiles * num_q_heads;
    // fitted on 256 compute units: one group above two workgroups a unit, four below half a one
    const int units = device_compute_units();
    int ks = workgroups > 2 * units ? 1 : workgroups > units / 2 ? 2 : 4;
    // (the variants left out would not fit their accumulators into the registers of so many waves)
    if (ks == 4 && (hdp > 2 || prefill_lds(hdp, 4, max_pages) > kPrefillMaxLds)) ks = 2;
    if (ks == 2 && (hdp > 6 || prefill_lds(hdp, 2, max_pages) > kPrefillMaxLds)) ks = 1;
    return ks;
}

// the float instance (attention_prefill_f32.hip)
int attn_prefill_f32(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                     int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                     const int* item_tok_off, const int* item_start, const int* item_len,
                     const int* block_table, const float* head_slopes, int max_pages, int page_size,
                     int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, hipStream_t stream);

// the direct-load instance (attention_prefill_dma.hip)
bool attn_prefill_dma_offered(int head_dim, int page_size, int tile_rows, int max_pages);
int attn_prefill_dma(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                     int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                     const int* item_tok_off, const int* item_start, const int* item_len,
                     const int* block_table, int max_pages, int page_size, int num_q_heads, int num_kv_heads,
                     int head_dim, float scale, int window, int tile_rows, int key_split, hipStream_t stream);

}  // namespace st

using namespace st;

// Tile i covers query rows [tile_q0[i], tile_q0[i] + tile_rows) of batch item tile_item[i] (rows past
// the item's length are skipped).  A list in order of the tiles' last positions lets the
// kernel deal long and short tiles evenly over the compute units.  Row r of item b is batch row item_tok_off[b] + r and sits at
// position item_start[b] + r of its request.  q: first query element of batch row 0; out:
// [batch rows, num_q_heads, head_dim].  key_split: wave groups per tile (1, 2 or 4), 0 = chosen
// here from the number of tiles; the float instance has one group only and ignores it.
// head_slopes (optional, [num_q_heads] floats): slope * (key position - query position) is added
// to the scaled scores of a head.
// tile_rows: 64, or 128 where st_attn_prefill_tile_rows says so (the direct-load kernel only).
// algo: 0 = chosen here, 1 = the kernel that stages blocks through registers, 2 = the direct-load
// kernel (an error where it is not offered).
extern "C" int st_attn_prefill(void* out, const void* q, int64_t q_stride,
                    const void* k_cache, const void* v_cache, int64_t page_stride,
                    const int* tile_item, const int* tile_q0, int num_tiles,
                    const int* item_tok_off, const int* item_start, const int* item_len,
                    const int* block_table, const float* head_slopes, int max_pages, int page_size,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window,
                    int key_split, int tile_rows, int algo, int dtype, hipStream_t stream) {
    ST_CHECK(dtype == kBF16 || dtype == kF32, "attn_prefill: unknown dtype %d", dtype);
    ST_CHECK(num_tiles >= 0 && num_q_heads > 0 && num_kv_heads > 0 && page_size > 0 && max_pages > 0,
             "attn_prefill: bad sizes");
    ST_CHECK(num_q_heads % num_kv_heads == 0, "attn_prefill: %d query heads do not divide into %d key heads",
             num_q_heads, num_kv_heads);
    ST_CHECK(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256,
             "attn_prefill: head_dim %d is not a multiple of 16 in [16, 256]", head_dim);
    ST_CHECK(num_tiles <= 65535, "attn_prefill: too many tiles for one launch");
    ST_CHECK(window >= 0, "attn_prefill: negative window");
    ST_CHECK(scale == scale && scale >= -3.0e38f && scale <= 3.0e38f, "attn_prefill: the score scale must be finite");
    ST_CHECK(tile_rows == 64 || tile_rows == 128, "attn_prefill: tiles of %d rows (64 or 128)", tile_rows);
    ST_CHECK(algo >= 0 && algo <= 2, "attn_prefill: unknown algo %d", algo);
    // (the direct-load kernel has no score bias: heads with slopes go through the staging kernel)
    // (and it orders maxima in scaled units, which needs a positive, finite scale)
    const bool dma_ok = dtype == kBF16 && !head_slopes && scale > 0.f && scale <= 3.0e38f &&
                        attn_prefill_dma_offered(head_dim, page_size, tile_rows, max_pages);
    ST_CHECK(tile_rows == 64 || (dma_ok && algo != 1),
             "attn_prefill: tiles of 128 rows need the direct-load kernel (bfloat16, head_dim 64 or 128, "
             "page size a power of two, no score slopes), not dtype %d head_dim %d page_size %d", dtype, head_dim,
             page_size);
    ST_CHECK(algo != 2 || dma_ok, "attn_prefill: the direct-load kernel is not offered for dtype %d head_dim %d "
             "page_size %d%s", dtype, head_dim, page_size, head_slopes ? " with score slopes" : "");
    if (num_tiles == 0) return 0;
    if (dtype == kF32)
        return attn_prefill_f32(out, q, q_stride, k_cache, v_cache, page_stride, tile_item, tile_q0, num_tiles,
                                item_tok_off, item_start, item_len, block_table, head_slopes, max_pages, page_size,
                                num_q_heads, num_kv_heads, head_dim, scale, window, stream);
    ST_CHECK(q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0, "attn_prefill: query rows must be 16-byte aligned");
    const int hdp = (head_dim + 31) / 32;
    // the direct-load kernel wherever it is offered
    if (algo == 2 || tile_rows == 128 || (algo == 0 && dma_ok)) {
        ST_CHECK(((uintptr_t)q & 15) == 0 && q_stride % 8 == 0, "attn_prefill: query rows must be 16-byte aligned");
        return attn_prefill_dma(out, q, q_stride, k_cache, v_cache, page_stride, tile_item, tile_q0, num_tiles,
                                item_tok_off, item_start, item_len, block_table, max_pages, page_size,
                                num_q_heads, num_kv_heads, head_dim, scale, window, tile_rows, key_split, stream);
    }
    const int ks = key_split > 0 ? key_split : prefill_key_split(hdp, num_tiles, num_q_heads, max_pages);
    ST_CHECK(ks == 1 || (ks == 2 && hdp <= 6) || (ks == 4 && hdp <= 2),
             "attn_prefill: %d wave groups are not offered for head_dim %d", ks, head_dim);
#define ST_PF(H, S) launch_prefill<H, S>(out, q, q_stride, k_cache, v_cache, page_stride, tile_item, tile_q0, num_tiles, \
        item_tok_off, item_start, item_len, block_table, head_slopes, max_pages, page_size, num_q_heads, num_kv_heads, \
        head_dim, scale, window, stream)
    switch (hdp * 8 + ks) {
        case 1 * 8 + 1: return ST_PF(1, 1);
        case 1 * 8 + 2: return ST_PF(1, 2);
        case 1 * 8 + 4: return ST_PF(1, 4);
        case 2 * 8 + 1: return ST_PF(2, 1);
        case 2 * 8 + 2: return ST_PF(2, 2);
        case 2 * 8 + 4: return ST_PF(2, 4);
        case 3 * 8 + 1: return ST_PF(3, 1);
        case 3 * 8 + 2: return ST_PF(3, 2);
        case 4 * 8 + 1: return ST_PF(4, 1);
        case 4 * 8 + 2: return ST_PF(4, 2);
        case 5 * 8 + 1: return ST_PF(5, 1);
        case 5 * 8 + 2: return ST_PF(5, 2);
        case 6 * 8 + 1: return ST_PF(6, 1);
        case 6 * 8 + 2: return ST_PF(6, 2);
        case 7 * 8 + 1: return ST_PF(7, 1);
        default: return ST_PF(8, 1);
    }
#undef ST_PF
}

extern "C" int st_has_attn_prefill() { return 1; }

// Rows per tile that st_attn_prefill serves best for a launch of `num_rows` query rows in items
// long enough for tiles: 128 where the direct-load kernel is offered, the head is large (at head
// size 64 the registers of a second row subtile cost more occupancy than the shared key blocks
// save: 43 against 35 us for 2,048 rows of 32 heads) and 128-row tiles still fill the chip; else 64.
extern "C" int st_attn_prefill_tile_rows(int head_dim, int page_size, int max_pages, int num_q_heads, int num_rows,
                                         int dtype) {
    if (dtype != kBF16 || head_dim < 128 || !attn_prefill_dma_offered(head_dim, page_size, 128, max_pages)) return 64;
    // 128-row tiles must still make one and a half workgroups a compute unit
    return (int64_t)(num_rows / 128) * num_q_heads * 2 >= (int64_t)device_compute_units() * 3 ? 128 : 64;
}
