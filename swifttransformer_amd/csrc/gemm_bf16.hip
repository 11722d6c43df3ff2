// bfloat16 matrix products on the matrix cores (placeholder until the MFMA kernels land).
#include "common.h"
#include "api.h"

namespace st {

int gemm_bf16_fast(void* out, const void* x, const void* w, const float* bias, const float* residual,
                   int M, int N, int K, int relu, int out_f32, hipStream_t stream, bool* handled) {
    *handled = false;
    return 0;
}

}  // namespace st

extern "C" int st_attn_prefill(void* out, const void* q, int64_t q_stride,
                    const void* k_cache, const void* v_cache, int64_t page_stride,
                    const int* tile_item, const int* tile_q0, int num_tiles,
                    const int* item_tok_off, const int* item_start, const int* item_len,
                    const int* block_table, int max_pages, int page_size,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window,
                    int dtype, hipStream_t stream) {
    st::set_error("attn_prefill: not built");
    return 1;
}

extern "C" int st_has_attn_prefill() { return 0; }
