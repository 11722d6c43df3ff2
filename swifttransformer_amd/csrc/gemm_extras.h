// Optional work fused into a matrix product, shared by the product kernels.
//
//  * Norm prologue: the product's input is LayerNorm(ln_x) (or its root-mean-square form,
//    which takes no mean off) computed on the fly from the
//    float residual stream instead of a stored activation (saves the norm kernel and its
//    round trip through memory).  Only the skinny matrix-core kernel offers it.
//  * Merge prologue: the product's input is the attention output still split over the keys:
//    per (row, head, split) a normalised partial result and its log-sum-exp, merged on the
//    fly (saves the merge kernel between a split decode attention and the output projection).
//    Only the skinny matrix-core kernel offers it.
//    The persistent wide-matrix kernel (gemm_wide.hip) also takes the rows through an index.
//  * Best-of-row epilogue: the index of every row's largest output (greedy token choice over a
//    vocabulary without another pass over the logits).  Only the persistent wide-matrix kernel.
//  * K/V scatter epilogue: output features [q_size, q_size + 2*kv_size) of a fused QKV
//    product are the new tokens' keys and values; besides the normal store they go
//    straight into their cache pages (the reference does this with a separate kernel,
//    src/csrc/kernel/kvcache_mgmt.cu:34-80).  Every product kernel offers it.
#pragma once
#include <stdint.h>

extern "C" struct StGemmExtras {
    // norm prologue (all null / 0: none)
    const float* ln_x;        // [M, K] float input rows
    const float* ln_gamma;    // [K] or null
    const float* ln_beta;     // [K] or null
    float ln_eps;
    int ln_no_center;         // 0: LayerNorm; 1: no mean is taken off (root-mean-square norm)
    // K/V scatter epilogue (k_cache null: none)
    void* k_cache;            // first element of page 0 of this layer's key pool
    void* v_cache;
    int64_t page_stride;      // elements between pages
    const int* token_item;    // [M] batch item of each row (-1: padding row)
    const int* positions;     // [M] position of each row in its request
    const int* block_table;   // [items, max_pages]
    int max_pages;
    int page_size;
    int q_size;               // query features come first
    int kv_size;              // num_kv_heads * head_dim
    int head_dim;
    int _pad1;
    // merge prologue (mg_o null: none); K of the product = mg_heads * mg_head_dim
    const float* mg_o;        // [M, mg_heads, mg_splits, mg_head_dim] partial outputs
    const float* mg_lse;      // [M, mg_heads, mg_splits] log-sum-exp of each partial (-inf: empty)
    int mg_splits;
    int mg_heads;
    int mg_head_dim;
    int _pad2;
    // with the norm prologue: row m of the product's input is LayerNorm(ln_x[ln_rows[m]]) (null: row m)
    const int* ln_rows;
    // best-of-row epilogue (best_ids null: none): best_ids[m] = the output feature with the largest
    // value in row m, the lowest index on ties; best_val / best_idx: scratch of 16 entries for every
    // workgroup of the kernel (st_gemm_wide_groups).  Only the persistent wide-matrix kernel offers
    // these two.
    int* best_ids;
    float* best_val;
    int* best_idx;
};

namespace st {
// Which kernel family a product went to; st_gemm counts its calls per path on the host
// (st_gemm_path_counts), so that tests can show which dispatch branches a run has taken.
enum GemmPath {
    kPathLibrary = 0,        // vendor library
    kPathGenericF32,         // plain tiled kernel, float operands
    kPathGenericBf16,        // plain tiled kernel, bfloat16 operands
    kPathResident,           // resident-slab kernel, stored rows read by every wave
    kPathResidentNorm,       // ... with the LayerNorm prologue
    kPathResidentMerge,      // ... with the split-attention merge prologue
    kPathResidentStaged,     // ... with the stored rows staged through LDS
    kPathSkinny16,           // skinny kernel, up to 16 rows (K beyond the resident kernel's reach)
    kPathSkinny32,
    kPathSkinny64,
    kPathTiledMfma,          // 128x128 matrix-core tiles
    kPathWide,               // persistent walk over a very wide matrix (few rows)
    kNumGemmPaths
};
void count_gemm_path(int path);
}  // namespace st

#ifdef __HIPCC__
namespace st {

// Destination of output feature n (>= q_size) of row m inside the caches, or -1.
// which: 0 = key, 1 = value.
__device__ inline int64_t kv_scatter_offset(const StGemmExtras& e, int m, int n, int* which) {
    const int item = e.token_item[m];
    const int pos = e.positions[m];
    if (item < 0 || pos < 0) return -1;
    int c = n - e.q_size;
    *which = c >= e.kv_size ? 1 : 0;
    if (*which) c -= e.kv_size;
    const int head = c / e.head_dim, d = c - head * e.head_dim;
    const int pi = pos / e.page_size;
    const int page = e.block_table[(int64_t)item * e.max_pages + pi];
    if (page < 0) return -1;
    return (int64_t)page * e.page_stride + ((int64_t)head * e.page_size + (pos - pi * e.page_size)) * e.head_dim + d;
}

}  // namespace st
#endif
