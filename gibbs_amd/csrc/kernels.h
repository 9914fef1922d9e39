// Prototypes of the kernel entry points (each defined in the .hip file of its kernel), for host code
// inside the library that queues several of them: the native step (step_plan.hip).  Every entry point
// checks its operands, queues its kernels on `stream` and returns 0, or non-zero with the reason in
// gibbs_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include "attention_decode_api.h"

extern "C" {
int gibbs_embed(const void* table, int dtype, const int* ids, float* x, void* mirror, int n, int hidden, int vocab,
                hipStream_t stream);
int gibbs_add_rmsnorm(float* x, const void* delta, const float* gain, float eps, void* out, int dtype, const int* rows,
                      int n_out, int hidden, hipStream_t stream);
int gibbs_add_partials_rmsnorm(float* x, const float* partials, int n_partials, long partial_stride, const float* gain,
                               float eps, void* out, int dtype, const int* rows, int n_out, int hidden, hipStream_t stream);
int gibbs_residual_add(float* x, const void* delta, int dtype, int n_partials, long partial_stride, void* mirror,
                       long count, hipStream_t stream);
int gibbs_gemm_f32(const float* A, const float* W, float* C, int N, int O, int I, long lda, long ldw, long ldc,
                   hipStream_t stream);
int gibbs_gemm_bf16_plain(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda, long ldw,
                          long ldc, hipStream_t stream);
int gibbs_gemm_bf16(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda, long ldw,
                    long ldc, hipStream_t stream);
int gibbs_gemm_library_init();
int gibbs_gemm_library(const void* A, const void* W, void* C, int N, int O, int I, long lda, long ldw, long ldc,
                       hipStream_t stream);
int gibbs_gemm_skinny(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx, long ldw,
                      long ldy, int k_splits, hipStream_t stream);
int gibbs_skinny_store(const void* X, const void* W, void* Y, int N, int O, int I, long ldx, long ldw, long ldy, int rms,
                       float eps, hipStream_t stream);
int gibbs_skinny_residual(const void* X, const void* W, float* x, void* xb, int N, int O, int I, long ldx, long ldw,
                          hipStream_t stream);
int gibbs_skinny_glu(const void* X, const void* W, void* Y, int N, int F, int I, long ldx, long ldw, long ldy, int rms,
                     float eps, int act, hipStream_t stream);
int gibbs_skinny_conv(const void* X, const void* W, void* Y, int N, int C, int I, long ldx, long ldw, int rms, float eps,
                      const float* taps, const float* bias, float* state, long slot_stride, const int* slot,
                      const int* ctx, int K, hipStream_t stream);
int gibbs_glu(const void* gu, void* out, int dtype, int n, int F, int act, hipStream_t stream);
int gibbs_shortconv(const void* bcx, const float* taps, const float* bias, float* state, long slot_stride, const int* cu,
                    const int* ctx, const int* slot, void* y, int dtype, int n_rows, int n_req, int lead_single, int C, int K,
                    hipStream_t stream);
int gibbs_qk_rope_kv(void* qkv, void* kpages, void* vpages, int dtype, const float* q_gain, const float* k_gain, float eps,
                     const float* inv_freq, int rot, int variant, const float* cs_table, int table_len, const int* pos,
                     const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh,
                     int nkv, int hd, long ld, hipStream_t stream);
int gibbs_attention_plain(const void* q, const void* kpages, const void* vpages, void* out, int dtype, const int* pos,
                          const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows,
                          int nh, int nkv, int hd, long ldq, long ldo, float scale, int window, const float* slopes,
                          hipStream_t stream);
int gibbs_attention_prefill(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                            const int* cu, const int* ctx, const int* table, int n_req, int max_pages, int page_size,
                            int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale, int window,
                            int n_splits, int first_row, int heads_per_wg, hipStream_t stream);
int gibbs_attention_decode_fused(const void* qkv, void* kpages, void* vpages, void* out, float* partial,
                                 const float* q_gain, const float* k_gain, float eps, const float* inv_freq, int rot,
                                 int variant, const float* cs_table, int table_len, const int* pos, const int* row_req,
                                 const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                 int hd, long ld, long ldo, float scale, int window, int n_splits, int waves, int kind,
                                 int max_keys, hipStream_t stream);
int gibbs_argmax(const float* logits, int* out, int M, int V, long ld, hipStream_t stream);
int gibbs_sample(const float* logits, int* out, int M, int V, long ld, const float* temperature, const float* top_p,
                 const int* top_k, const float* u, hipStream_t stream);
int gibbs_decode_tail(const float* logits, int V, long ld, int* ids, int* pos, int* ctx, int* log, int* steps, int n,
                      int capacity, float* u, const float* u_all, const void* table, int table_dtype, int vocab, int hidden,
                      float* x, void* mirror, const int* live, hipStream_t stream);
}

// Inside the library only: gibbs_skinny_store with the output's type given (bfloat16 or float32); what
// gibbs_gemm_skinny hands whole sums of up to 16 rows to (gemm_skinny_fused.hip).
int gibbs_skinny_store_as(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx, long ldw,
                          long ldy, int rms, float eps, hipStream_t stream);
