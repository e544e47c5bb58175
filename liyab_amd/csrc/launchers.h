// Declarations of the library's launchers, for code that calls them by name from inside the
// library (the replay of a recorded list of launches, replay.hip). Every .hip file that defines
// one includes this header, so that a declaration that does not match its definition is a
// compile error.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "epilogue.h"

extern "C" {

int liyab_fill(void* p, int elem_bytes, uint32_t bits, int64_t n, hipStream_t stream);
int liyab_add_into(float* y, const void* x, int dtype, int64_t n, hipStream_t stream);
int liyab_gather_rows(void* out, int out_dtype, const float* x, const int* rows, int n, int d, hipStream_t stream);
int liyab_scale(float* p, float scale, int64_t n, hipStream_t stream);
int liyab_embed(float* x, const void* tok, const void* pos, int dtype, const int* ids, const int* positions, int n, int d, float scale,
                const int* last_tokens, hipStream_t stream);
int liyab_add_rows(float* x, const void* table, int dtype, const int* rows, int n, int d, hipStream_t stream);
int liyab_kv_write(void* kc, void* vc, const void* src, int dtype, int64_t src_stride, int k_off, int v_off, const int* slots, int n,
                   int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);
int liyab_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                    hipStream_t stream);
int liyab_layernorm_parts(void* out, int out_dtype, const float* planes, int n_parts, int64_t part_stride, int x_rows, const float* w,
                          const float* b, const int* rows, int n, int d, float eps, hipStream_t stream);
int liyab_sum_parts(float* out, int x_rows, int d, const float* planes, int n_parts, int64_t part_stride, hipStream_t stream);
int liyab_gemm_simple(void* out, int out_dtype, int64_t ldo, const void* a, int64_t lda, const void* w, int dtype, const float* bias,
                      float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream);
int liyab_gemm_mfma(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile, const liyab::EpiParams* epi_in,
                    hipStream_t stream);
int liyab_gemm_mfma_dl(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile, const liyab::EpiParams* epi_in,
                       hipStream_t stream);
int liyab_gemm_mfma_dl_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts, int tile, float* parts,
                             int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                             hipStream_t stream);
int liyab_gemm_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit, int wide, int mtile,
                      const liyab::EpiParams* epi_in, hipStream_t stream);
int liyab_gemm_skinny_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts, int ksplit, float* parts,
                            int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                            hipStream_t stream);
int liyab_gemm_att_parts(const float* partials, int n_splits, int n_head, int hd, const void* w, int M, int N, int kparts, float* parts,
                         int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                         hipStream_t stream);
int liyab_gemm_skinny_ln(const float* planes, int n_planes, int64_t plane_stride, const float* ln_weight, const float* ln_bias,
                         float eps, const void* w, int M, int N, int K, int wide, const liyab::EpiParams* epi_in, hipStream_t stream);
int liyab_attention_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                            const int* block_tables, int max_blocks, const int* tok_seq, const int* tok_pos, int n, float scale,
                            int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);
int liyab_attention_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                           const int* block_tables, int max_blocks, const int* tok_list, const int* tok_seq, const int* tok_pos, int n,
                           float scale, int window, int n_head, int n_kv_head, int hd, int page_size, int n_splits, int chunk,
                           int waves, int rows_are_requests, float* partials, int leave_splits, int num_pages, hipStream_t stream);
int liyab_attention_merge(void* out, int out_dtype, int64_t out_stride, const float* partials, int n, int n_head, int hd, int n_splits,
                          hipStream_t stream);
int liyab_attention_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc,
                            const int* block_tables, int max_blocks, const int* work, int n_tiles, int tile, int ksplit, float scale,
                            int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);

}  // extern "C"
