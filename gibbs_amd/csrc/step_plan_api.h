// C interface of the native step (step_plan.hip): a model's step laid down once as a program of
// operations over parts, then run as one call per step.
//
// A plan holds parts (norms; bodies: what reads normed rows and gives a delta for the residual stream,
// a mixer or a feed-forward) and a program of operations over them.  The parts that the library brings
// are made by gibbs_plan_norm_rms / gibbs_plan_body_conv / _attention / _glu; a part from anywhere else
// is a function pointer with a user pointer (gibbs_plan_norm_host / gibbs_plan_body_host): code of
// another library, or a callback into an interpreter.  The program says how a layer arranges its parts;
// every function that appends to it returns the index of what it made, or -1 with the reason in
// gibbs_last_error().
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// One step's operands (the integer metadata lives on the device already).
struct GibbsStepArgs {
  const int* ids;          // [n_rows]
  const int* pos;          // [n_rows]
  const int* row_req;      // [n_rows]
  const int* cu;           // [n_req + 1]
  const int* ctx;          // [n_req]
  const int* slot;         // [n_req]
  const int* logit_rows;   // [n_logits]
  const int* const* tables;   // per cache group: [n_req, widths[g]] page ids
  const int* widths;
  int n_groups;
  int n_rows, n_req, n_logits, max_q, max_seq, lead_single;
  void* workspace;         // device memory for the step's activations (null: only count the bytes)
  long workspace_bytes;
  float* logits;           // [n_logits, vocab] float32 out
  hipStream_t stream;
  // A step that continues a captured decode loop: the rows' embeddings are there already (the end of the
  // previous step wrote them), as the float32 stream x_in [n_rows, hidden] and, for steps that take the fused
  // decode kernels, its bfloat16 mirror.  Null: the step embeds its ids itself.
  float* x_in;
  void* mirror_in;
  // The operations to run (n_ops 0: all of them, then the final norm and the head for the wanted rows), and
  // whether a delta that is still pending at the end is added into x (for a caller that reads x).
  int first_op, n_ops, settle;
};

// out [n_rows, hidden] (the run's activation type) = body(h [n_rows, hidden]); queued on step->stream.
typedef int (*GibbsHostBody)(void* user, const struct GibbsStepArgs* step, const void* h, void* out);
// x (+= delta, when all rows are normed: rows null); out [n_out, hidden] = norm of the rows (all, or `rows`).
// delta: null, [n_rows, hidden] in the activation type (delta_parts 1), or float32 [delta_parts, n_rows, hidden].
typedef int (*GibbsHostNorm)(void* user, const struct GibbsStepArgs* step, float* x, const void* delta, int delta_parts,
                             const int* rows, int n_out, void* out);
// q and k rows of a step, in place, after the q/k norm and before k is cached: qkv [n_rows, ld] in the activation type.
typedef int (*GibbsHostRows)(void* user, const struct GibbsStepArgs* step, void* qkv, long ld);

// dtype: GIBBS_F32 (0) or GIBBS_BF16 (1), of activations, matrices and cache pages.  table / head may be null
// for a plan that only runs parts (no embedding, no logits).
void* gibbs_plan_create(int dtype, int hidden, int vocab, const void* table, int table_dtype, const void* head,
                        const void* head_packed, int fused_rows, int own_gemm);
void gibbs_plan_destroy(void* plan);

// ---- parts
int gibbs_plan_norm_rms(void* plan, const float* gain, float eps);     // gain null: folded into the matrices that follow
int gibbs_plan_norm_host(void* plan, GibbsHostNorm fn, void* user);
int gibbs_plan_body_conv(void* plan, const void* w_in, const void* p_in3, const void* w_out, const void* p_out,
                         const float* taps, const float* bias, int C, int K, float* state, long slot_stride);
int gibbs_plan_body_attention(void* plan, const void* w_qkv, const void* p_qkv, const void* w_out, const void* p_out, int nh,
                              int nkv, int hd, float scale, int window, const float* q_gain, const float* k_gain,
                              float qk_eps, const float* inv_freq, int rot, int variant, const float* cos_sin,
                              int table_len, void* kpages, void* vpages, int num_pages, int page_size, int group,
                              int owns, const float* slopes, GibbsHostRows hook, void* hook_user);
int gibbs_plan_body_glu(void* plan, const void* w_gate_up, const void* p_gate_up2, const void* w_down, const void* p_down,
                        int F, int act);
int gibbs_plan_body_host(void* plan, GibbsHostBody fn, void* user, int group);   // group: the cache group it reads, or -1

// ---- the program (values are normed rows or deltas, named by the index their operation returns)
int gibbs_plan_op_half(void* plan, int norm, int body);       // x += body(norm(x)), in fused kernels where it can
int gibbs_plan_op_norm(void* plan, int norm);                 // -> value: norm(x + what is pending)
int gibbs_plan_op_body(void* plan, int body, int value);      // -> value: body(normed rows)
int gibbs_plan_op_add(void* plan, int value);                 // x += delta (lazily: it stays pending for the next norm)
int gibbs_plan_op_drop(void* plan, int value);                // the value is not read again
int gibbs_plan_tail(void* plan, int norm);                    // the norm in front of the head
int gibbs_plan_op_count(const void* plan);

// ---- running
long gibbs_plan_workspace(const void* plan, const struct GibbsStepArgs* args);   // bytes of workspace the step needs
int gibbs_plan_step(const void* plan, const struct GibbsStepArgs* args);
int gibbs_plan_last_fused(const void* plan);   // halves of the last step that ran as fused decode kernels
// One part alone.  args->workspace null: returns the bytes of workspace needed.  Else runs it and returns 0 (non-zero:
// failed), with the result at *out_offset bytes into the workspace: [parts, n_rows, hidden] float32 partial sums when
// *parts >= 2, else [n_rows, hidden] in the activation type.
long gibbs_plan_body_forward(const void* plan, int body, const struct GibbsStepArgs* args, const void* h, long* out_offset,
                             int* parts);
long gibbs_plan_norm_forward(const void* plan, int norm, const struct GibbsStepArgs* args, float* x, const void* delta,
                             int delta_parts, const int* rows, int n_out, long* out_offset);

// ---- the dispatch rules, for callers that run a kernel by itself
int gibbs_rule_skinny_splits(int n_out, int inner, int want_blocks, int features, int min_k);
void gibbs_rule_decode_splits(int n_rows, int nkv, int group, int max_seq, int hd, int page_size, int kind, int* n_splits,
                              int* waves);
long gibbs_rule_prefill_tiles(int rows, int reqs);            // query tiles that the rows of a ragged batch make
int gibbs_rule_prefill_splits(long n_tiles, int nh, int max_seq, int window);
int gibbs_rule_prefill_heads(int rows, int reqs, int nh, int nkv, int hd, int max_seq, int n_splits);   // query heads a workgroup
int gibbs_rule_fused_rows(void);                              // rows that the fused decode kernels take at most
// y = x W^T the way a step would run it.  gibbs_linear_splits: the float32 partial sums it would leave (1: the
// finished product [n, O]; s >= 2: [s, n, O] float32).  gibbs_linear: runs it into y (sized by that answer).
int gibbs_linear_splits(int dtype, int n, int O, int I, long ldx, const void* x, const void* w, int out_f32, int partial_ok,
                        int own_gemm);
int gibbs_linear(const void* x, long ldx, const void* w, const void* packed, void* y, int dtype, int n, int O, int I,
                 int out_f32, int partial_ok, int own_gemm, hipStream_t stream);
// x += y W^T, mirror = bfloat16(x), for up to 64 rows: floats of workspace that the route for these sizes needs (0:
// none), and the product itself (ldw 0: W in tile order).
long gibbs_skinny_residual_workspace(int n, int O, int I);
int gibbs_skinny_residual_routed(const void* y, const void* w, long ldw, float* x, void* mirror, int n, int O, int I,
                                 float* workspace, hipStream_t stream);

#ifdef __cplusplus
}
#endif
