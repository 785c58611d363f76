// The C entry points of the kernel libraries (csrc/kernels/*.hip), declared in one place for the
// native engine. Every launcher returns 0, a positive HIP error code, or a negative code when it
// refuses the sizes; none of them allocates.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>

extern "C" {

// elementwise.hip
int mllm_embed(const int* ids, const int* pos, const void* wte, const void* wpe, float* x, int T, int D,
               int dtype, const int* src, const int* prev, int n_prev, hipStream_t stream);
int mllm_select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream);
int mllm_reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int B,
                     hipStream_t stream);
int mllm_layernorm(const float* x, const int* rows, const float* gamma, const float* beta, void* y, int n,
                   int D, float eps, int out_dtype, hipStream_t stream);
int mllm_kv_append(const void* src, int src_stride, int k_col, int v_col, void* k_pages, void* v_pages,
                   int kv_dim, const int* slots, int T, int dtype, hipStream_t stream);

// gemm_f32.hip, gemm_bf16.hip
int mllm_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, void* C, int ldc,
                  int M, int N, int K, int mode, hipStream_t stream);
int mllm_gemm_bf16(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                   int M, int N, int K, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream);
int mllm_gemm_bf16_kv(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                      int M, int N, int K, const int* slots, void* k_pages, void* v_pages, int q_cols, int kv_dim,
                      hipStream_t stream);
int mllm_gemm_bf16_merged(const float* split_o, const float* split_ml, int n_splits, int n_heads, int head_dim,
                          const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int mode,
                          hipStream_t stream);
int mllm_ln_gemm_bf16(const float* x, int ldx, const int* rows, const float* gamma, const float* beta, float eps,
                      const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int K, int mode,
                      hipStream_t stream);

// attention.hip, attention_decode.hip, attention_prefill.hip
int mllm_paged_attention_generic(const void* q, int q_stride, int q_col, const void* k_pages,
                                 const void* v_pages, int kv_dim, const int* block_tables, int max_blocks,
                                 const int* token_seq, const int* positions, int n_tokens, int n_heads,
                                 int n_kv_heads, int head_dim, int page_size, float scale, int window,
                                 void* out, int out_stride, int dtype, hipStream_t stream);
int mllm_paged_attention_tiled(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                               int kv_dim, const int* block_tables, int max_blocks, const int* cu_q, const int* ctx_len,
                               int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads, int head_dim, int page_size,
                               float scale, int window, void* out, int out_stride, int dtype, hipStream_t stream);
int mllm_decode_attention(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                          int kv_dim, const int* block_tables, int max_blocks, const int* token_seq,
                          const int* positions, int n_q, int n_heads, int n_kv_heads, int head_dim,
                          int page_size, float scale, int window, int nsplit, int waves, void* out,
                          int out_stride, float* ws, int* counters, int k_col, int v_col, const int* slots,
                          int partial_out, int dtype, hipStream_t stream);
int mllm_merge_attention_splits(const float* ws, int n_q, int n_heads, int head_dim, int nsplit, void* out,
                                int out_stride, int dtype, hipStream_t stream);
int mllm_prefill_attention_bf16(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                                int kv_dim, const int* block_tables, int max_blocks, const int* cu_q,
                                const int* ctx_len, int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads,
                                int head_dim, int page_size, float scale, int window, void* out, int out_stride,
                                hipStream_t stream);

// sampling.hip
int mllm_argmax_chunks(int V);
int mllm_argmax_mirrored(const float* logits, int ld, int n, int V, int* out, int* mirror, float* part_val, int* part_idx,
                hipStream_t stream);
int mllm_sample_mirrored(const float* logits, int ld, int n, int V, const float* temperature, const float* u, int* out, int* mirror,
                hipStream_t stream);

}  // extern "C"
