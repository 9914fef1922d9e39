// C interface of the decode attention over prepared queries (attention_decode.hip).
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Floats of workspace that a call with n_splits > 1 key slices needs (0 for one slice).
long gibbs_attention_decode_workspace(int n_rows, int nh, int hd, int n_splits);

// q: [N, >= nh*hd] bfloat16 (row stride ldq); pages: [num_pages, nkv, page_size, hd] bfloat16;
// out: [N, nh*hd] bfloat16 (row stride ldo); partial: the workspace above, or null with n_splits 1.
// kind: 0 choose, 1 vector units, 2 matrix cores (+ 4: the key slices are merged by a second kernel, not by the
// slice that finishes last); max_keys: a bound on the keys of any row (0: the
// block table's width).  Returns 0, or non-zero with the reason in gibbs_last_error().
int gibbs_attention_decode(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                           const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                           int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale,
                           int window, int n_splits, int waves, int kind, int max_keys, hipStream_t stream);

// The same call for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
// runtime allocates its split-attention partials itself).  The partial results of the key slices go
// to an array that the library holds on every GPU it runs on until the process ends, of
// gibbs_attention_decode_static_capacity() floats; a call that needs more (see
// gibbs_attention_decode_workspace) is refused with an error, and so is everything that
// gibbs_attention_decode refuses.  The call allocates and frees nothing, on the host or the device.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race; calls in one stream are ordered and safe.  Nothing in the array has to start at
// zero: every slice writes its (maximum, sum, values) before the merge kernel reads them.
int gibbs_attention_decode_static(const void* q, const void* kpages, const void* vpages, void* out,
                                  const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                                  int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale,
                                  int window, int n_splits, int waves, int kind, int max_keys, hipStream_t stream);

// Floats of the per-GPU array behind gibbs_attention_decode_static (2 Mi floats = 8 MiB).
long gibbs_attention_decode_static_capacity(void);

#ifdef __cplusplus
}
#endif
