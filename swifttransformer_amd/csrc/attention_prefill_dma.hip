// Attention of prompt portions over the paged cache (bfloat16), keys and values moved from
// memory straight into LDS.
//
// Same mathematics, tile description and masking as attention_prefill.hip (transposed flash
// formulation on v_mfma_f32_16x16x32_bf16: S^T = K Q^T, O^T += V^T P^T, online softmax per lane
// in float), with the work per score cut where that kernel spends its vector instructions:
//
//  * A key block (64 keys) travels memory -> LDS by the direct load (global_load_lds_dwordx4):
//    no staging registers, no LDS stores, no packing.  A wave's load writes 1 KB of LDS in lane
//    order, so rows cannot be padded against bank conflicts; instead each lane fetches the 16-byte
//    chunk that an XOR swizzle assigns to its LDS slot, and the readers apply the same swizzle.
//    Two buffers: block i+1 is in flight while block i is consumed; one barrier a block.
//  * V stays row-major in LDS like K.  The transposed operand of the second product comes from
//    the transposing LDS read (ds_read_b64_tr_b16): within 16 lanes, lane 4k+m reads 4 dims of
//    key k and lane i receives dim i of keys 0..3.
//  * The softmax normaliser is summed by the matrix core (a row of ones in V^T) and the running
//    maximum is kept in scaled units from a finite floor, which takes additions, a special case
//    and, while the maximum stands still, the rescale of the accumulators out of the loop.
//  * A workgroup's tile holds 64 or 128 query rows (QT = 1 or 2 subtiles of 16 rows a wave): with
//    128, every LDS read and every byte moved serves twice as many scores.
//
// Instances for rows of 64, 96 and 128 dims in LDS; a head size up to 16 dims below one of them
// (48, 80, 112) runs in the next larger instance with the missing chunks of every LDS row zero
// (they are cleared once and never loaded).  Page sizes are powers of two.  The staged kernel
// serves everything else.
//
// Reference: src/csrc/kernel/fused_context_stage_attention.cu:87-453 (see attention_prefill.hip).
#include "common.h"
#include "api.h"

namespace st {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define ST_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))
#define ST_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int DK = 64;     // keys per block

// XOR swizzles of the 16-byte chunk index inside a row, by row: chosen so that the 16 lanes of a
// ds_read_b128 phase (16 key rows, one chunk) and the 32 lanes of a transposing read phase (8 key
// rows, two neighbouring chunks each) fall on distinct banks.  Rows of 128 bytes (HD 64) share a
// 256-byte bank row in pairs, rows of 256 bytes (HD 128) fill one each; rows of 192 bytes (HD 96)
// start a quarter of a bank row later each, so four rows apart meet again and the swizzle tells
// those apart (it stays inside aligned groups of 4 chunks, of which such a row has three).  None
// depends on a row's multiple of 16: readers add those to a row's offset afterwards.
template <int HD> __device__ inline int swizzle_k(int row) {
    return HD == 64 ? ((row >> 1) & 7) : HD == 96 ? ((row >> 2) & 3) : (row & 15);
}
template <int HD> __device__ inline int swizzle_v(int row) {
    return HD == 64 ? (((row >> 1) & 3) << 1) : HD == 96 ? (((row >> 2) & 1) << 1) : ((row & 7) << 1);
}

// KS > 1 (QT = 1 only): the workgroup has KS groups of four waves, each with LDS buffers of its own,
// going through a contiguous share of the tile's key blocks; their partial results meet in LDS at
// the end.  That shortens the chain of blocks when few tiles are in flight.
template <int HD, int QT, int KS>
__global__ __launch_bounds__(256 * KS, (HD == 64 && KS == 1) ? 2 : 1) void attn_prefill_dma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, int64_t page_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_start, const int* __restrict__ item_len,
    const int* __restrict__ block_table, int max_pages, int page_shift,
    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window, int num_tiles, int deal_period) {
    // head_dim: dims of a head in memory, HD - 16 or HD; the LDS rows and the products have HD
    constexpr int HDP = HD / 32;                     // 32-wide steps over the head dimension
    constexpr int DT = HD / 16;                      // 16-wide output subtiles
    constexpr int CH = HD / 8;                       // 16-byte chunks per row
    constexpr int ROWB = HD * 2;                     // bytes per row
    constexpr int MAT = DK * ROWB;                   // bytes of one matrix of a block
    constexpr int NI = HD / 32;                      // direct loads per wave and matrix (1 KB each)
    constexpr int TILE = 64 * QT;
    extern __shared__ uint4 dyn[];
    char* lds_all = reinterpret_cast<char*>(dyn);    // per wave group: [2 buffers][K, V][64 rows][ROWB]
    int* s_bt = reinterpret_cast<int*>(lds_all + KS * 4 * MAT);

    const int h = blockIdx.x;
    int tile;
    {   // grid row -> tile, serpentine over rows of `deal_period` tiles from the list's heavy end
        const int slot = blockIdx.y, row = slot / deal_period, base = row * deal_period;
        const int in_row = min(deal_period, num_tiles - base), c = slot - base;
        tile = num_tiles - 1 - (base + ((row & 1) ? in_row - 1 - c : c));
    }
    const int item = tile_item[tile], q0 = tile_q0[tile];
    if (item < 0) return;                            // a padding entry of a tile list of fixed length
    const int start = item_start[item], n = item_len[item], row0 = item_tok_off[item];
    const int page_size = 1 << page_shift;
    const int tid = threadIdx.x, lane = tid & 63;
    // the wave's index in a scalar register: what depends on it alone (its rows' positions, the
    // LDS places of its loads, whether a block needs masking) is then scalar too, and branches on
    // it are real branches
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int part = wave_all >> 2, wave = wave_all & 3;      // wave group, wave within it
    char* lds = lds_all + part * 4 * MAT;
    const int g = lane >> 4, r16 = lane & 15;
    const int kvh = h / (num_q_heads / num_kv_heads);

    const int rows_in_tile = min(TILE, n - q0);
    const int pos_first = start + q0, pos_last = start + q0 + rows_in_tile - 1;
    const int key_lo = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;
    const int key_hi = pos_last + 1;                 // exclusive

    {   // block table of the request -> LDS
        const int p_lo = key_lo >> page_shift, p_hi = (key_hi - 1) >> page_shift;
        const int* bt = block_table + (int64_t)item * max_pages;
        for (int i = p_lo + tid; i <= p_hi; i += 256 * KS) s_bt[i] = bt[i];
    }
    // this lane's query rows: subtile t of wave w holds rows 64t + 16w .. +15 of the tile
    int qi[QT], qpos[QT];
    bool qvalid[QT];
    bf16x8 qf[QT][HDP];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        qi[t] = q0 + 64 * t + wave * 16 + r16;
        qvalid[t] = qi[t] < n;
        qpos[t] = start + qi[t];
        const bf16_t* qrow = q + (int64_t)(row0 + (qvalid[t] ? qi[t] : q0)) * q_stride + (int64_t)h * head_dim;
#pragma unroll
        for (int s = 0; s < HDP; ++s)
            qf[t][s] = (qvalid[t] && 32 * s + 8 * g < head_dim)
                           ? __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(qrow + 32 * s + 8 * g))
                           : __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
    }

    // ---- direct loads: load j of this wave fills LDS bytes [(wave*NI + j) * 1024, +1024) of a matrix
    // in lane order; slot (row, physical chunk) takes the logical chunk (physical ^ swizzle(row)).
    int ld_row[NI];
    uint32_t ld_k[NI], ld_v[NI];                     // element offset inside a page, without the key's row
    bool ld_k_ok[NI], ld_v_ok[NI];                   // the chunk exists (head_dim < HD: the last two of a row do not)
    const int chunks = head_dim >> 3;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int slot = (wave * NI + j) * 64 + lane;
        const int row = slot / CH, pc = slot % CH;
        const int ck = pc ^ swizzle_k<HD>(row), cv = pc ^ swizzle_v<HD>(row);
        ld_row[j] = row;
        ld_k_ok[j] = ck < chunks;
        ld_v_ok[j] = cv < chunks;
        ld_k[j] = (uint32_t)(kvh * page_size * head_dim + ((ld_k_ok[j] ? ck : 0) << 3));
        ld_v[j] = (uint32_t)(kvh * page_size * head_dim + ((ld_v_ok[j] ? cv : 0) << 3));
    }
    const uint32_t stride32 = (uint32_t)page_stride; // elements between pages (checked on the host: < 2^31)
    auto issue = [&](int kb, int buf) {
        char* kdst = lds + buf * 2 * MAT + wave * (NI * 1024);
        const bool whole = kb >= key_lo && kb + DK <= key_hi;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            // a key outside the tile's range is replaced by one inside it (its scores are masked):
            // every address is that of a written key
            int key = kb + ld_row[j];
            if (!whole) key = min(max(key, key_lo), key_hi - 1);
            const uint32_t page = (uint32_t)s_bt[key >> page_shift];
            const uint64_t base = (uint64_t)page * stride32 + (uint32_t)((key & (page_size - 1)) * head_dim);
            // (a lane whose chunk does not exist loads nothing: its LDS slot keeps the zeros it was given)
            if (ld_k_ok[j])
                __builtin_amdgcn_global_load_lds(ST_GLOBAL_PTR(k_cache + (base + ld_k[j])),
                                                 ST_LDS_PTR(void, kdst + j * 1024), 16, 0, 0);
            if (ld_v_ok[j])
                __builtin_amdgcn_global_load_lds(ST_GLOBAL_PTR(v_cache + (base + ld_v[j])),
                                                 ST_LDS_PTR(void, kdst + MAT + j * 1024), 16, 0, 0);
        }
    };

    // ---- readers' offsets (bytes inside a matrix).  K: lane (key row r16, chunk 4s + g) of key
    // subtile t; the swizzle of row 16t + r16 does not depend on t.  V: lane L of a 16-lane group
    // reads 4 dims (8 bytes) of key 4g + L/4 of a 16-key half: chunk 2dt + (L&3)/2, byte 8(L&1).
    int koff[HDP], voff[DT];
#pragma unroll
    for (int s = 0; s < HDP; ++s) koff[s] = r16 * ROWB + (((4 * s + g) ^ swizzle_k<HD>(r16)) << 4);
    {
        const int vrow = 4 * g + (r16 >> 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            voff[dt] = vrow * ROWB + (((2 * dt + ((r16 & 3) >> 1)) ^ swizzle_v<HD>(vrow)) << 4) + ((r16 & 1) << 3);
    }

    // Running maximum of a row in units of log2 (score * sl), starting from a finite floor: a
    // row that has seen nothing yet then needs no special case (exp2 of floor minus anything real
    // is 0, floor minus floor is exactly 0).  The normaliser is one more row of the second
    // product: a V^T row of ones makes the matrix core sum the very probabilities (rounded to
    // bfloat16) that it multiplies, instead of 16 additions a block.
    float ms[QT];
    floatx4 acc[QT][DT], accl[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        ms[t] = -1.0e30f;
        accl[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[t][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const float sl = scale * 1.44269504088896340736f;            // scores in units of log2
    const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
    int sub_first[QT], sub_last[QT];                              // positions of the wave's rows, per subtile
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        sub_first[t] = pos_first + 64 * t + wave * 16;
        sub_last[t] = min(pos_last, sub_first[t] + 15);
    }

    auto consume = [&](int kb, int buf) {
        const char* ks = lds + buf * 2 * MAT;
        const char* vs = ks + MAT;
        if (kb > sub_last[QT - 1]) return;           // beyond the last row of this wave
        // ---- S^T: st[t][kt][r] = score of key kb + 16 kt + 4g + r with query row t of this lane
        floatx4 st[QT][4];
#pragma unroll
        for (int t = 0; t < QT; ++t)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) st[t][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < HDP; ++s) {
            bf16x8 a[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                a[kt] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(ks + kt * 16 * ROWB + koff[s]));
#pragma unroll
            for (int t = 0; t < QT; ++t)
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
                    st[t][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[kt], qf[t][s], st[t][kt], 0, 0, 0);
        }
        // ---- mask (only blocks on the diagonal, at the window's edge or at the range's ends),
        // then online softmax per lane = per query row, and across the 4 lane groups
        bf16x8 pf[QT][2];
#pragma unroll
        for (int t = 0; t < QT; ++t) {
            const bool interior = kb + DK - 1 <= sub_first[t] && kb >= key_lo &&
                                  (window <= 0 || kb > sub_last[t] - window);
            if (!interior) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = kb + 16 * kt + 4 * g + r;
                        const bool ok = qvalid[t] && j <= qpos[t] && j >= key_lo && (window <= 0 || j > qpos[t] - window);
                        st[t][kt][r] = ok ? st[t][kt][r] : -INFINITY;
                    }
            }
            float bmax = max3_raw(st[t][0][0], st[t][0][1], st[t][0][2]);
            bmax = max3_raw(bmax, st[t][0][3], st[t][1][0]);
            bmax = max3_raw(bmax, st[t][1][1], st[t][1][2]);
            bmax = max3_raw(bmax, st[t][1][3], st[t][2][0]);
            bmax = max3_raw(bmax, st[t][2][1], st[t][2][2]);
            bmax = max3_raw(bmax, st[t][2][3], st[t][3][0]);
            bmax = max3_raw(bmax, st[t][3][1], st[t][3][2]);
            bmax = rows4_max(max_raw(bmax, st[t][3][3]));
            const float mc = max_raw(ms[t], bmax * sl);           // sl > 0: the order of scores is that of their scaled values
            const float alpha = __builtin_amdgcn_exp2f(ms[t] - mc);
            ms[t] = mc;
            // the rescale is skipped while no row of the wave has moved its maximum (alpha is exactly 1)
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) acc[t][dt] *= alpha;
                accl[t] *= alpha;
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                uint32_t packed[4];
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int kt = 2 * u + half;
                    float p[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(fmaf(st[t][kt][r], sl, -mc));
                    packed[2 * half] = pack_bf16x2(p[0], p[1]);
                    packed[2 * half + 1] = pack_bf16x2(p[2], p[3]);
                }
                pf[t][u] = __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
            }
        }
        // ---- O^T += V^T P^T, and the row of ones for the normaliser
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int t = 0; t < QT; ++t)
                accl[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[t][u], accl[t], 0, 0, 0);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                // this lane's 8 keys of half u: 32u + 4g + {0..3} and 32u + 16 + 4g + {0..3}, dim 16dt + r16
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    ST_LDS_PTR(short4v, vs + (32 * u) * ROWB + voff[dt]));
                const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    ST_LDS_PTR(short4v, vs + (32 * u + 16) * ROWB + voff[dt]));
                const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
                const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(lo2.x, lo2.y, hi2.x, hi2.y));
#pragma unroll
                for (int t = 0; t < QT; ++t)
                    acc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf[t][u], acc[t][dt], 0, 0, 0);
            }
        }
    };

    // The tile's key blocks are dealt to the wave groups in KS contiguous shares; every group
    // goes through the loop the same number of times (the barriers are the workgroup's).
    const int kb_first = (key_lo / DK) * DK;
    const int nblk = (key_hi - kb_first + DK - 1) / DK;
    const int per = (nblk + KS - 1) / KS;
    const int kb0 = kb_first + part * per * DK;
    const int kb_end = min(key_hi, kb0 + per * DK);  // this group's keys end here
    if (head_dim < HD) {
        // the chunks that no load fills are zero for good: clear the buffers once
        uint4* z = reinterpret_cast<uint4*>(lds_all);
        for (int i = tid; i < KS * 4 * MAT / 16; i += 256 * KS) z[i] = make_uint4(0, 0, 0, 0);
    }
    __syncthreads();                                 // the block table is in LDS (and the buffers are clear)
    if (kb0 < kb_end) issue(kb0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int it = 0; it < per; ++it) {
        const int kb = kb0 + it * DK;
        // the other buffer was consumed before the barrier that ended the previous round
        if (kb + DK < kb_end) issue(kb + DK, (it + 1) & 1);
        if (kb < kb_end) consume(kb, it & 1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    // the wave groups' partial results (maximum, normaliser, output) meet in LDS; the first group merges them
    if (KS > 1) {
        constexpr int E = 2 + 4 * DT;                 // floats per lane (QT = 1)
        float* mg = reinterpret_cast<float*>(lds_all);
        if (part > 0) {
            float* dst = mg + (size_t)((part - 1) * 4 + wave) * E * 64 + lane;
            dst[0] = ms[0];
            dst[64] = accl[0][0];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(2 + 4 * dt + r) * 64] = acc[0][dt][r];
        }
        __syncthreads();
        if (part > 0) return;
#pragma unroll
        for (int p = 1; p < KS; ++p) {
            const float* src = mg + (size_t)((p - 1) * 4 + wave) * E * 64 + lane;
            const float mo = src[0], lo = src[64];
            const float mn = max_raw(ms[0], mo);
            const float a = __builtin_amdgcn_exp2f(ms[0] - mn), b = __builtin_amdgcn_exp2f(mo - mn);
            accl[0][0] = accl[0][0] * a + lo * b;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[0][dt][r] = acc[0][dt][r] * a + src[(2 + 4 * dt + r) * 64] * b;
            ms[0] = mn;
        }
    }

    // acc[t][dt][r] = O[query row t of this lane][dim 16dt + 4g + r]; every entry of accl[t] is the
    // row's normaliser
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const float lsum = accl[t][0];
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
        if (qvalid[t]) {
            bf16_t* orow = out + ((int64_t)(row0 + qi[t]) * num_q_heads + h) * head_dim;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if (16 * dt >= head_dim) continue;
                uint2 p;
                p.x = pack_bf16x2(acc[t][dt][0] * inv, acc[t][dt][1] * inv);
                p.y = pack_bf16x2(acc[t][dt][2] * inv, acc[t][dt][3] * inv);
                *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * g) = p;
            }
        }
    }
}

constexpr size_t kDmaMaxLds = 156 * 1024;            // of the 160 KB a gfx950 compute unit has

// The instance (dims of an LDS row) that serves a head size: itself, or the next one 16 above; 0: none.
static int dma_instance(int head_dim) {
    for (int hd : {64, 96, 128})
        if (head_dim == hd || head_dim == hd - 16) return hd;
    return 0;
}

static size_t dma_lds(int head_dim, int ks, int max_pages) {
    return (size_t)ks * 4 * DK * dma_instance(head_dim) * 2 + (size_t)max_pages * sizeof(int);
}

// Whether the direct-load kernel takes this case (tiles of 128 rows: the instances of 64 and 128 only).
bool attn_prefill_dma_offered(int head_dim, int page_size, int tile_rows, int max_pages) {
    const int hd = dma_instance(head_dim);
    return hd != 0 && page_size >= 1 && (page_size & (page_size - 1)) == 0 &&
           (tile_rows == 64 || (tile_rows == 128 && hd != 96)) && dma_lds(head_dim, 1, max_pages) <= kDmaMaxLds;
}

// Wave groups per tile: more when few tiles are in flight, as far as LDS allows.
static int dma_key_split(int head_dim, int tile_rows, int num_tiles, int num_q_heads, int max_pages) {
    if (tile_rows != 64) return 1;
    const int64_t workgroups = (int64_t)num_tiles * num_q_heads;
    const int units = device_compute_units();     // fitted on 256: two workgroups a unit, one
    int ks = workgroups > 2 * units ? 1 : workgroups > units ? 2 : 4;
    while (ks > 1 && dma_lds(head_dim, ks, max_pages) > kDmaMaxLds) ks >>= 1;
    return ks;
}

template <int HD, int QT, int KS>
static int launch_dma(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                      int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                      const int* item_tok_off, const int* item_start, const int* item_len,
                      const int* block_table, int max_pages, int page_size, int num_q_heads,
                      int num_kv_heads, int head_dim, float scale, int window, hipStream_t stream) {
    auto kernel = attn_prefill_dma_kernel<HD, QT, KS>;
    const size_t lds = dma_lds(HD, KS, max_pages);
    if (lds > 48 * 1024) {
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaMaxLds);
            ST_CHECK(e == hipSuccess, "attn_prefill: cannot raise the LDS limit: %s", hipGetErrorString(e));
            raised = true;
        }
    }
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    const int compute_units = device_compute_units();
    const int deal_period = compute_units / num_q_heads > 0 ? compute_units / num_q_heads : 1;
    kernel<<<dim3(num_q_heads, num_tiles), 256 * KS, lds, stream>>>(
        (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, page_stride,
        tile_item, tile_q0, item_tok_off, item_start, item_len, block_table, max_pages, page_shift,
        num_q_heads, num_kv_heads, head_dim, scale, window, num_tiles, deal_period);
    ST_LAUNCH_CHECK("attn_prefill_dma");
    return 0;
}

// key_split: wave groups per tile (1, 2 or 4; tiles of 64 rows), 0 = chosen here.
int attn_prefill_dma(void* out, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                     int64_t page_stride, const int* tile_item, const int* tile_q0, int num_tiles,
                     const int* item_tok_off, const int* item_start, const int* item_len,
                     const int* block_table, int max_pages, int page_size, int num_q_heads, int num_kv_heads,
                     int head_dim, float scale, int window, int tile_rows, int key_split, hipStream_t stream) {
    ST_CHECK(page_stride > 0 && page_stride < ((int64_t)1 << 31), "attn_prefill: a page of %lld elements",
             (long long)page_stride);
    // the running maximum is kept as (block maximum) * scale: only a positive scale keeps its order
    ST_CHECK(scale > 0.f && scale <= 3.0e38f, "attn_prefill: the direct-load kernel needs a positive, finite score "
             "scale, not %g", (double)scale);
    ST_CHECK(attn_prefill_dma_offered(head_dim, page_size, tile_rows, max_pages),
             "attn_prefill: the direct-load kernel takes head sizes 48 to 128 in steps of 16, page sizes that are "
             "powers of two and tiles of 64 rows (128 too but for head sizes 80 and 96), not head_dim %d, "
             "page_size %d, tile_rows %d", head_dim, page_size, tile_rows);
    const int ks = key_split > 0 ? key_split : dma_key_split(head_dim, tile_rows, num_tiles, num_q_heads, max_pages);
    ST_CHECK(ks == 1 || ((ks == 2 || ks == 4) && tile_rows == 64 && dma_lds(head_dim, ks, max_pages) <= kDmaMaxLds),
             "attn_prefill: %d wave groups are not offered for head_dim %d and tiles of %d rows", ks, head_dim,
             tile_rows);
#define ST_DMA(H, Q, S) launch_dma<H, Q, S>(out, q, q_stride, k_cache, v_cache, page_stride, tile_item, tile_q0,    \
        num_tiles, item_tok_off, item_start, item_len, block_table, max_pages, page_size, num_q_heads, num_kv_heads, \
        head_dim, scale, window, stream)
    const int hd = dma_instance(head_dim);
    if (hd == 64) {
        if (tile_rows == 128) return ST_DMA(64, 2, 1);
        return ks == 4 ? ST_DMA(64, 1, 4) : ks == 2 ? ST_DMA(64, 1, 2) : ST_DMA(64, 1, 1);
    }
    if (hd == 96) return ks == 2 ? ST_DMA(96, 1, 2) : ST_DMA(96, 1, 1);
    if (tile_rows == 128) return ST_DMA(128, 2, 1);
    return ks == 2 ? ST_DMA(128, 1, 2) : ST_DMA(128, 1, 1);
#undef ST_DMA
}

}  // namespace st
