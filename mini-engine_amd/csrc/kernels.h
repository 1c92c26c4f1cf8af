// The entry points of the kernels in this folder, for the native step program (host/program.cpp),
// which launches them without a round trip through Python. Every function returns 0 on success and
// leaves a message for me_last_error() otherwise; a refused size launches nothing.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

extern "C" {
const char* me_last_error();
int me_embed(void* x, const void* table, const int* ids, int num_tokens, int hidden, int vocab, float scale, int dtype,
             hipStream_t stream);
int me_embed_fed(void* x, const void* table, const int* ids, const int* fed_rows, const int* fed_tokens, int num_tokens,
                 int hidden, int vocab, float scale, int dtype, hipStream_t stream);
int me_scale_f32(float* x, float scale, long long count, hipStream_t stream);
int me_add_rmsnorm(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, const float* w,
                   void* h, const int* rows, int num_rows, int dim, float eps, int write_x, int dtype, hipStream_t stream);
int me_residual_add(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, int num_rows, int dim,
                    int dtype, hipStream_t stream);
int me_rmsnorm(const void* in, const float* w, void* out, int num_rows, int dim, float eps, int dtype, hipStream_t stream);
int me_swiglu(const void* gu, void* act, int num_tokens, int inter, int gate, int dtype, hipStream_t stream);
int me_qk_norm_rope_scatter(const void* qkv, const float* q_w, const float* k_w, const float* rope_table,
                            const int* positions, const int* token_item, const int* block_table, int table_width,
                            void* q_out, void* k_cache, void* v_cache, int num_tokens, int nh, int nkv, int d, int rd, int bs,
                            float eps, int write_kv, int dtype, const int* item_start, int num_items, int num_segments,
                            hipStream_t stream);
int me_attention_general(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                         const int* token_item, const int* block_table, int table_width, void* out, int num_tokens, int nh,
                         int nkv, int d, int bs, int window, float scale, int dtype, int items, hipStream_t stream);
int me_attention_mfma_supported(int d, int bs);
int me_attention_decode_fused_supported(int d, int bs, int rotary_dim, int group);
int me_attention_prefill_columns(int wide);
int me_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                             const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                             int nh, int nkv, int d, int bs, int window, float scale, int split_keys, int num_splits,
                             int max_ctx, const int* live_items, int full_splits, int waves_wanted, const int* step_flags,
                             hipStream_t stream);
int me_attention_decode_fused_bf16(const void* qkv, const float* q_w, const float* k_w, const float* rope_table,
                                   int rotary_dim, float eps, int write_kv, void* k_cache, void* v_cache, const int* item_ctx,
                                   const int* block_table, int table_width, void* out, float* part_o, float* part_ml,
                                   int items, int nh, int nkv, int d, int bs, int window, float scale, int split_keys,
                                   int num_splits, int max_ctx, const int* live_items, int full_splits, int waves_wanted,
                                   const int* step_flags, hipStream_t stream);
// Decode steps of very few items: the launch leaves its splits' partial results (out == nullptr) and the output
// projection adds them up itself.
int me_attention_decode_leaves_parts(int items, int nh, int nkv, int d, int num_splits);
int me_attention_out_product_runs(int nh);
int me_attention_out_product_supported(int items, int nh, int d, int n, int num_splits);
int me_attention_out_product_bf16(const float* part_o, const float* part_ml, int num_splits, const void* W, float* parts,
                                  int items, int nh, int d, int n, hipStream_t stream);
int me_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, int num_items, const int* block_table,
                              int table_width, void* out, const int* work, const int* bundle_first, int num_bundles,
                              float* part_o, float* part_ml, const int* token_chunks, int max_chunks, int num_tokens, int nh,
                              int nkv, int d, int bs, int window, float scale, int columns, hipStream_t stream);
int me_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, hipStream_t stream);
int me_gemm_plain(const void* A, const void* W, void* C, int M, int N, int K, int in_dtype, int out_dtype, hipStream_t stream);
int me_gemm_bf16_small(const void* X, const float* x_in, const void* delta, const float* w_norm, float eps, float* x_out,
                       const void* W, void* C, int M, int N, int K, int norm, int swiglu, int out_dtype, int k_splits,
                       hipStream_t stream);
int me_gemm_bf16_stream_splits(int M, int N, int K, int compute_units);
void me_gemm_bf16_stream_plan(int M, int N, int K, int gated, int k_splits, int compute_units, int* out);
int me_gemm_bf16_stream(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype, int k_splits,
                        int compute_units, hipStream_t stream);
int me_gemm_bf16_stream_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                               int compute_units, const float* row_ss, int ss_blocks, int ss_dim, float eps, hipStream_t stream);
int me_gemm_bf16_stream_carry_blocks(int M, int N, int K, int compute_units);
int me_gemm_bf16_stream_carry(const void* X, const void* W, float* x, void* h, float* ss, const float* w_norm, int M, int N, int K,
                              int compute_units, hipStream_t stream);
int me_gemm_bf16_small_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                              const float* row_ss, int ss_blocks, int ss_dim, float eps, hipStream_t stream);
int me_gemm_bf16_stream_norm_fits(int M, int K);
int me_gemm_bf16_stream_norm(const float* x_in, const void* delta, const float* parts, int num_parts, long long part_stride,
                             const float* w_norm, float eps, float* x_out, const void* W, void* C, int M, int N, int K,
                             int swiglu, int out_dtype, int compute_units, hipStream_t stream);
int me_gemm_bf16_tiled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype, int shape,
                       hipStream_t stream);
int me_gemm_bf16_library(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype, hipStream_t stream);
int me_gemm_bf16_library_add(const void* X, const void* W, float* C, int M, int N, int K, hipStream_t stream);
int me_sample_chunks(int vocab);
int me_sample(const float* logits, int num_rows, int vocab, const float* temperatures, const uint64_t* keys, int* out,
              void* workspace, hipStream_t stream);
}
