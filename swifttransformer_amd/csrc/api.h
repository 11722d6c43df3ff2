// C entry points of the kernel library.  Every function returns 0 on success;
// otherwise st_last_error() describes the refusal (bad sizes, unsupported head
// size, ...).  Pointers are device pointers unless noted; `stream` is the HIP
// stream to launch on.  dtype: 0 = float32, 1 = bfloat16 storage.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

extern "C" {

const char* st_last_error();

int st_lookup(void* out_f32, void* out_t, const int* ids, const void* table,
              const int* add_ids, int add_offset, const void* add_table,
              int table_rows, int add_rows, int num_rows, int width, int accumulate, int dtype, hipStream_t stream);

// center != 0: LayerNorm; center == 0: no mean is taken off (root-mean-square norm).
int st_layernorm(void* out_t, void* out_f32, const float* x, const int* rows,
                 const float* gamma, const float* beta, int num_rows, int width,
                 float eps, int center, int dtype, hipStream_t stream);

int st_kv_write(void* k_cache, void* v_cache, int64_t page_stride,
                const void* k_src, const void* v_src, int64_t src_stride,
                const int* token_item, const int* positions,
                const int* block_table, int max_pages, int page_size,
                int num_tokens, int num_kv_heads, int head_dim, int dtype, hipStream_t stream);

int st_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype, hipStream_t stream);

// out[r, c] = act(a[r, c]) * (b ? b[r, c] : 1) over rows x width elements; the three row strides
// (in elements) are free, so a and b may be the two halves of one product's output.  `kind` as
// st_gemm's activation.  The reference's counterpart multiplies two whole arrays
// (src/csrc/kernel/fused_activ_multiply.cu:19-36).
int st_activation_multiply(void* out, int64_t out_stride, const void* a, int64_t a_stride,
                           const void* b, int64_t b_stride, int rows, int width, int kind, int dtype,
                           hipStream_t stream);

struct StGemmExtras;
// activation: the function between bias and residual, by number (csrc/activation.h): 0 none,
// 1 ReLU, 2 SiLU, 3 GELU in its tanh form; others are refused.
int st_gemm(void* out, const void* x, const void* w, const float* bias, const float* residual,
            int M, int N, int K, int activation, int dtype, int out_f32, int algo,
            const StGemmExtras* extras, hipStream_t stream);
int st_gemm_path_counts(uint64_t* out, int reset);
int st_gemm_library_rule(int min_rows, int64_t min_weights, int min_depth);
// Which workgroup shapes a product with the norm prologue may take (for measurements and tests):
// bit 1 the wide ones (24 features) at all, bit 2 sixteen waves for them, and 32 features, bit 4
// 32 features tried before 24; 3 is the default.
int st_gemm_wide_workgroups(int mode);
int st_gemm_can_fuse_norm(int M, int N, int K, int dtype);
int st_gemm_wide_offered(int M, int N, int K, int dtype);
int st_gemm_wide_groups();
int st_gemm_can_fuse_merge(int M, int N, int K, int splits, int heads, int head_dim, int dtype);

int st_attn_rows(void* out, float* part_o, float* part_lse, const void* q, int64_t q_stride,
                 const void* k_cache, const void* v_cache, int64_t page_stride,
                 const int* row_ids, const int* token_item, const int* positions,
                 const int* block_table, const float* head_slopes,
                 int max_pages, int page_size, int num_tokens, int num_q_heads,
                 int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                 int num_waves, int dtype, hipStream_t stream);

// No counterpart in the reference.  For callers that cannot allocate (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc): st_attn_rows with the key
// split's partial results kept in a static device array of the library (4 MiB per GPU, held
// until the process ends) instead of a workspace argument.  Calls no hipMalloc/hipFree.  Refuses
// num_tokens * num_q_heads * num_splits * (head_dim + 1) floats beyond that size.  Calls that
// overlap on one GPU share the array and race.  st_attn_rows_static_init() resolves the array's
// address on the current device ahead of the first call (the first call does it otherwise).
int st_attn_rows_static_init();
size_t st_attn_rows_static_capacity();
int st_attn_rows_static(void* out, const void* q, int64_t q_stride,
                        const void* k_cache, const void* v_cache, int64_t page_stride,
                        const int* row_ids, const int* token_item, const int* positions,
                        const int* block_table, const float* head_slopes,
                        int max_pages, int page_size, int num_tokens, int num_q_heads,
                        int num_kv_heads, int head_dim, float scale, int window, int num_splits,
                        int num_waves, int dtype, hipStream_t stream);

int st_attn_prefill(void* out, const void* q, int64_t q_stride,
                    const void* k_cache, const void* v_cache, int64_t page_stride,
                    const int* tile_item, const int* tile_q0, int num_tiles,
                    const int* item_tok_off, const int* item_start, const int* item_len,
                    const int* block_table, const float* head_slopes, int max_pages, int page_size,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, int window,
                    int key_split, int tile_rows, int algo, int dtype, hipStream_t stream);

int st_has_attn_prefill();
int st_attn_prefill_tile_rows(int head_dim, int page_size, int max_pages, int num_q_heads, int num_rows, int dtype);

int st_gemm_library_init();
int st_gemm_library_tuning(int on);
int st_gemm_library_allow_workspace(int on);

int st_sample(int* out, const float* logits, int num_rows, int vocab, const float* temperature,
              const uint32_t* seeds, const uint32_t* draws, hipStream_t stream);

float st_hash_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t draw, uint32_t v);

// Measurement kernels (csrc/probe.hip): a plain streaming read, and a kernel without work.
int st_probe_read(const void* src, int64_t bytes, void* sink, int workgroups, int pattern, hipStream_t stream);
int st_probe_empty(void* sink, hipStream_t stream);
int st_probe_fill(const void* src, int64_t region, void* sink, int workgroups, int turns, int to_lds,
                  hipStream_t stream);
int st_probe_mfma(void* sink, int workgroups, int rounds, int wide, hipStream_t stream);

}  // extern "C"
