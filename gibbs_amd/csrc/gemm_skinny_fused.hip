// Decode-step matrix products with the neighbouring operations fused in, so that a layer is a
// handful of kernels instead of a dozen (no kernel on this chip is shorter than about 4 us, and
// a decode step at small batch is a chain of products that each stream a few megabytes).
//
//   Y = X W^T for at most 64 rows of X (bfloat16), W streamed once straight into the A operand of
//   v_mfma_f32_16x16x32_bf16, the workgroup's waves splitting k and meeting in LDS, as in
//   gemm_skinny.  On top of that:
//
//   packed W      W may come in MFMA-tile order (packed_layout.h: 16-row tiles, or 8-row tiles of two k tiles
//                  for matrices of few rows, zero-padded): a wave's load of an A operand is then 1 KB of
//                  consecutive memory, 8 requests of 128 bytes instead of 16 of 64, which is worth a fifth of
//                  the time of these products (the compute unit's memory pipe is bound by requests in flight,
//                  not by bytes).
//   8 features     Where 16 features per workgroup would leave compute units idle, a workgroup takes 8, and the
//                  other 8 rows of its A operands hold the same 8 features at the NEXT 32 values of k: the
//                  operand's product with X at k fills rows 0..7 of one accumulator, its product with X at
//                  k + 32 rows 8..15 of a second one, and the two halves are added at the end.  One load of
//                  1 KB then serves two MFMA steps, and it is consecutive memory in the pair layout (two
//                  workgroups that read alternate 128-byte pieces of the same tiles were measured a quarter
//                  slower than one that reads them whole).
//   prologue RMS   the rows of X are the bfloat16 mirror of the residual stream; the workgroup sums
//                  their squares from the B operands it loads anyway and scales its outputs by
//                  1/sqrt(mean(x^2) + eps).  The norm's gain is folded into W when weights are bound.
//   row groups     a workgroup computes the same ROWS features of up to 3 row ranges of W (offsets
//                  0, group_stride, 2 group_stride) so that an epilogue finds its operands in one lane:
//                  gate and up of a GLU; B, C, x of the short convolution.
//   epilogues      STORE     y = acc (bfloat16)
//                  RESIDUAL  x += acc (float32 stream, each element owned by one workgroup);
//                            xb = bfloat16(x), the mirror the next product reads
//                  GLU       out = act(gate) * up (activation.h)
//                  CONV      bx = B * x;  cv = bias + taps . [state, bx];  y = C * cv;  state shifts
//                            (every row is one decoded token of a different request)
#include "gemm_skinny_fused.h"

// (gemm_skinny_fused_rows.hip: the same kernels for a row-major W; `args` is a FusedArgs)
void gibbs_fused_rows(const void* args, int epilogue, int rms, hipStream_t stream);

// In all of these, ldw == 0 means that W is in tile order (packed_layout.h), each row group by itself.
//
// Y[n, o] = scale_n * sum_k X[n, k] W[o, k], bfloat16 out; scale_n = 1/sqrt(mean_k X[n,k]^2 + eps) if rms.
GIBBS_EXPORT int gibbs_skinny_store(const void* X, const void* W, void* Y, int N, int O, int I, long ldx, long ldw,
                                    long ldy, int rms, float eps, hipStream_t stream) {
  return gibbs_skinny_store_as(X, W, Y, GIBBS_BF16, N, O, I, ldx, ldw, ldy, rms, eps, stream);
}

// The same with the output's type given: bfloat16 or float32 (Y: [N, ldy] of that type, 16-byte aligned rows for
// the vector stores to be taken).
int gibbs_skinny_store_as(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx, long ldw,
                          long ldy, int rms, float eps, hipStream_t stream) {
  if (check_common("skinny_store", X, W, N, O, I, ldx, ldw)) return 1;
  GIBBS_REQUIRE(ldy >= O, "skinny_store: output rows shorter than %d", O);
  GIBBS_REQUIRE(out_dtype == GIBBS_BF16 || out_dtype == GIBBS_F32, "skinny_store: unknown output dtype %d", out_dtype);
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = O; a.I = I; a.ldw = ldw; a.ldx = ldx; a.eps = eps; note_layout(a);
  if (out_dtype == GIBBS_F32) a.Yf = (float*)Y;
  else a.Y = (bf16*)Y;
  a.ldy = ldy;
  a.y_vec = ((uintptr_t)Y % 16) == 0 && ldy % 4 == 0;   // float32 rows that take 16-byte stores
  if (a.packed) run_store<true>(a, rms != 0, stream);
  else gibbs_fused_rows(&a, EPI_STORE, rms, stream);
  GIBBS_LAUNCH_STATUS("skinny_store");
}

// x[n, o] += sum_k X[n, k] W[o, k];  xb[n, o] = bfloat16(x[n, o]).  x: [N, O] float32, xb: [N, O] bfloat16.
GIBBS_EXPORT int gibbs_skinny_residual(const void* X, const void* W, float* x, void* xb, int N, int O, int I, long ldx,
                                       long ldw, hipStream_t stream) {
  if (check_common("skinny_residual", X, W, N, O, I, ldx, ldw)) return 1;
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = O; a.I = I; a.ldw = ldw; a.ldx = ldx; note_layout(a);
  a.x = x; a.xb = (bf16*)xb;
  a.y_vec = O % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)xb % 8) == 0;
  if (a.packed) run_residual<true>(a, stream);
  else gibbs_fused_rows(&a, EPI_RESIDUAL, 0, stream);
  GIBBS_LAUNCH_STATUS("skinny_residual");
}

// out[n, f] = silu(s_n gate_f . X_n) * (s_n up_f . X_n); W = [gate rows (F); up rows (F)], rms prologue.
GIBBS_EXPORT int gibbs_skinny_glu(const void* X, const void* W, void* Y, int N, int F, int I, long ldx, long ldw,
                                  long ldy, int rms, float eps, int act, hipStream_t stream) {
  if (check_common("skinny_glu", X, W, N, F, I, ldx, ldw)) return 1;
  GIBBS_REQUIRE(ldy >= F, "skinny_glu: output rows shorter than %d", F);
  GIBBS_REQUIRE(act >= 0 && act < ACT_COUNT, "skinny_glu: unknown activation %d", act);
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = F; a.I = I; a.ldw = ldw; a.ldx = ldx; a.eps = eps; note_layout(a);
  a.group_stride = F; a.Y = (bf16*)Y; a.ldy = ldy; a.act = act;
  a.y_vec = ldy % 4 == 0 && ((uintptr_t)Y % 8) == 0;
  if (a.packed) run_glu<true>(a, rms != 0, stream);
  else gibbs_fused_rows(&a, EPI_GLU, rms, stream);
  GIBBS_LAUNCH_STATUS("skinny_glu");
}

// In-projection and gated short convolution of N decoded tokens of N different requests:
// W = [B rows (C); C rows (C); x rows (C)]; y[n, c] = Cg * (bias + taps . [state, B*x]); state shifts.
GIBBS_EXPORT int gibbs_skinny_conv(const void* X, const void* W, void* Y, int N, int C, int I, long ldx, long ldw,
                                   int rms, float eps, const float* taps, const float* bias, float* state,
                                   long slot_stride, const int* slot, const int* ctx, int K, hipStream_t stream) {
  if (check_common("skinny_conv", X, W, N, C, I, ldx, ldw)) return 1;
  GIBBS_REQUIRE(K >= 2 && K <= MAX_TAPS, "skinny_conv: kernel length %d outside 2..%d", K, MAX_TAPS);
  GIBBS_REQUIRE(slot_stride >= (long)(K - 1) * C, "skinny_conv: state slot stride %ld shorter than (K-1)*C", slot_stride);
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = C; a.I = I; a.ldw = ldw; a.ldx = ldx; a.eps = eps; note_layout(a);
  a.group_stride = C; a.Y = (bf16*)Y; a.ldy = C;
  a.taps = taps; a.bias = bias; a.state = state; a.slot_stride = slot_stride; a.slot = slot; a.ctx = ctx; a.K = K;
  a.y_vec = C % 4 == 0 && slot_stride % 4 == 0 && ((uintptr_t)Y % 8) == 0 && ((uintptr_t)state % 16) == 0;
  if (a.packed) run_conv<true>(a, rms != 0, stream);
  else gibbs_fused_rows(&a, EPI_CONV, rms, stream);
  GIBBS_LAUNCH_STATUS("skinny_conv");
}
