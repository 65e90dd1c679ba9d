// Prototypes of the kernel libraries' entry points that the executor calls (defined in the .hip files one folder up;
// the host library is linked against both kernel libraries).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

extern "C" {
// ---- plain
int apc_embed_rows(const void* table, int table_dtype, const int* tokens, void* out, int out_dtype, int n_tok, int dim,
                   int ldo, hipStream_t stream);
int apc_embed_rows_tiled(const void* table, int chunks, const int* tokens, void* out, int out_dtype, int n_tok, int dim,
                         int ldo, hipStream_t stream);
int apc_rmsnorm_rows(const void* x, int x_dtype, int ldx, const int* rows, const float* w, float eps, void* out,
                     int out_dtype, int ldo, int n_rows, int dim, hipStream_t stream);
int apc_silu_mul(const void* gu, int in_dtype, int ldg, void* out, int out_dtype, int ldo, int n_rows, int F,
                 hipStream_t stream);
int apc_rope_kv_write(void* qkv, int dtype, int ld, int q_off, int k_off, int v_off, int n_tok, int H, int Hk, int d,
                      int rot, const float* cos_sin, const int* positions, const int* row_seg, const int* block_table,
                      int max_blocks, void* cache, int cache_dtype, int page_tokens, hipStream_t stream);
int apc_gemm_plain(const void* A, int a_dtype, int lda, const void* W, int w_dtype, int ldw, void* C, int c_dtype,
                   int ldc, int M, int N, int K, int mode, hipStream_t stream);
int apc_paged_attention_plain(const void* q, int q_dtype, int ldq, int q_off, void* out, int out_dtype, int ldo,
                              int n_rows, int H, int Hk, int d, const void* cache, int cache_dtype, int page_tokens,
                              const int* block_table, int max_blocks, const int* positions, const int* row_seg,
                              int window, float scale, hipStream_t stream);
// ---- tuned
int apc_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K, int mode,
                  hipStream_t stream);
int apc_gemm_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, void* C, int ldc, int M, int F, int K,
                         hipStream_t stream);
int apc_gemm_pre_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps, const void* W, const void* Wu,
                      void* C, int ldc, int M, int N, int K, int mode, hipStream_t stream);
int apc_gemm_splitk_bf16(const void* A, int lda, const void* W, const void* Wu, void* C, int ldc, int M, int N, int K,
                         int mode, int k_split, float* workspace, hipStream_t stream);
int apc_gemm_splitk_emit_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K, int k_split,
                              float* workspace, const float* g, void* raw, int ld_raw, float* ss, hipStream_t stream);
int apc_gemm_splitk_pre_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps, const void* W,
                             const void* Wu, void* C, int ldc, int M, int N, int K, int mode, int k_split,
                             float* workspace, hipStream_t stream);
int apc_gemm_splitk_qkv_rope_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps, const void* W,
                                  void* q_out, int ldq, int M, int K, int H, int Hk, int d, const float* cos_sin,
                                  const int* positions, const int* row_seg, const int* block_table, int max_blocks,
                                  void* cache, int page_tokens, int k_split, float* workspace, hipStream_t stream);
int apc_gemm_direct_k_split(int M, int N, int K);
int apc_gemm_direct_emit_parts(const void* A, int lda, const void* residual, int ldc, int M, int N, int K);
int apc_gemm_direct_emit_bf16(const void* A, int lda, const void* W, float* residual, int ldc, int M, int N, int K,
                              const float* g, void* raw, int ldr, float* ss, int parts, float* workspace,
                              hipStream_t stream);
int apc_skinny_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K, int mode,
                         hipStream_t stream);
int apc_skinny_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, void* C, int ldc, int M, int F, int K,
                           hipStream_t stream);
int apc_skinny_gemm_emit_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                              const float* g, void* raw, int ld_raw, float* ss, hipStream_t stream);
int apc_skinny_gemm_pre_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* W, void* C,
                             int ldc, int M, int N, int K, int mode, hipStream_t stream);
int apc_skinny_swiglu_pre_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* Wg,
                               const void* Wu, void* C, int ldc, int M, int F, int K, hipStream_t stream);
int apc_skinny_qkv_rope_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* W, void* q_out,
                             int ldq, int M, int K, int H, int Hk, int d, const float* cos_sin, const int* positions,
                             const int* row_seg, const int* block_table, int max_blocks, void* cache, int page_tokens,
                             hipStream_t stream);
int apc_rope_kv_write_bf16(void* qkv, int ld, int q_off, int k_off, int v_off, int n_tok, int H, int Hk, int d, int rot,
                           const float* cos_sin, const int* positions, const int* row_seg, const int* block_table,
                           int max_blocks, void* cache, int page_tokens, hipStream_t stream);
int apc_attention_prefill_bf16(const void* q, int ldq, int q_off, void* out, int ldo, int H, int Hk, int d,
                               const void* cache, int page_tokens, const int* block_table, int max_blocks,
                               const int* positions, const int* row_seg, const int* tile_row0, const int* tile_rows,
                               int n_tiles, int n_rows, int window, float scale, int n_splits, int part_rows,
                               float* parts, hipStream_t stream);
int apc_attention_decode_bf16(const void* q, int ldq, int q_off, void* out, int ldo, int n_rows, int H, int Hk, int d,
                              const void* cache, int page_tokens, const int* block_table, int max_blocks,
                              const int* positions, const int* row_seg, const int* rows, int window, float scale,
                              int keys_per_part, int n_parts, float* workspace, int* counters, hipStream_t stream);
int apc_attention_decode_last_fits(int H, int Hk, int d, int n_parts);
int apc_attention_decode_whole_fits(int H, int Hk, int d);
int apc_attention_prefill_tile_rows();
int apc_attention_prefill_wide_takes(int d, int page_tokens, int n_tiles, int n_rows);
}
