// Gated short convolution over a ragged batch, with its per-request state.
//
// Input bcx[N, 3C] holds the thirds [B | C | x] of the in-projection.  For request r with rows
// cu[r] .. cu[r+1]:   bx = B * x (float32);   window = state[slot[r]] (K-1 rows, oldest first)
// followed by bx;   cv[t] = bias + sum_j taps[c, j] * window[(K-1) + t - (K-1-j)];
// y[t] = C[t] * cv[t];   state <- last K-1 rows of the window.
// A history row at a negative absolute position (ctx[r] + t' < 0) counts as zero whatever the
// slot holds, so a slot needs no clearing when a new request takes it.
//
// One thread owns (request, tile of TL rows, channel).  Only the thread of tile 0 reads or
// writes the state of its (request, channel), after it has computed its rows, so no other
// thread can see a half-updated state.  Tap sums run in ascending j in every case, so a
// row's value does not depend on how the sequence was cut into steps.
#include "common.h"

namespace {
constexpr int TL = 32;  // rows per tile; K - 1 <= TL so that only tile 0 needs history

template <typename T>
__global__ __launch_bounds__(256) void shortconv_kernel(
    const T* __restrict__ bcx, const float* __restrict__ taps, const float* __restrict__ bias,
    float* __restrict__ state, long slot_stride, const int* __restrict__ cu, const int* __restrict__ ctx,
    const int* __restrict__ slot, T* __restrict__ y, int n_req, int C, int K) {
  int tile = blockIdx.y, r = 0, q = 0;
  for (; r < n_req; ++r) {
    q = cu[r + 1] - cu[r];
    const int t = (q + TL - 1) / TL;
    if (tile < t) break;
    tile -= t;
  }
  if (r >= n_req) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int row0 = cu[r], before = ctx[r];
  float* st = state + (size_t)slot[r] * slot_stride;  // [K-1, C]
  const float* w = taps + (size_t)c * K;
  const float b = bias ? bias[c] : 0.f;
  const size_t ld = (size_t)3 * C;

  auto bx_at = [&](int tp) -> float {  // tp: row index inside this step's chunk, may be negative
    if (tp >= 0) {
      const T* row = bcx + (size_t)(row0 + tp) * ld;
      return to_float(row[c]) * to_float(row[2 * C + c]);
    }
    return (before + tp >= 0) ? st[(size_t)(K - 1 + tp) * C + c] : 0.f;
  };

  const int t_end = min(q, (tile + 1) * TL);
  for (int t = tile * TL; t < t_end; ++t) {
    float acc = 0.f;
    for (int j = 0; j < K; ++j) acc = fmaf(w[j], bx_at(t - (K - 1 - j)), acc);
    acc += b;
    const size_t n = (size_t)(row0 + t);
    y[n * C + c] = from_float<T>(to_float(bcx[n * ld + C + c]) * acc);
  }
  if (tile == 0) {
    // new[s] = window[q + s]; it reads old[q + s] (an index above s), so ascending s is safe.
    for (int s = 0; s < K - 1; ++s) {
      const float v = bx_at(q - (K - 1) + s);
      st[(size_t)s * C + c] = v;
    }
  }
}
}  // namespace

GIBBS_EXPORT int gibbs_shortconv(const void* bcx, const float* taps, const float* bias, float* state,
                                 long slot_stride, const int* cu, const int* ctx, const int* slot, void* y,
                                 int dtype, int n_rows, int n_req, int C, int K, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && n_req >= 0 && C > 0, "shortconv: bad sizes rows=%d requests=%d width=%d", n_rows, n_req, C);
  GIBBS_REQUIRE(K >= 2 && K - 1 <= TL, "shortconv: kernel length %d outside 2..%d", K, TL + 1);
  GIBBS_REQUIRE(slot_stride >= (long)(K - 1) * C, "shortconv: state slot stride %ld shorter than (K-1)*C", slot_stride);
  if (n_rows == 0 || n_req == 0) return 0;
  dim3 grid(ceil_div(C, 256), ceil_div(n_rows, TL) + n_req);
  GIBBS_REQUIRE(grid.y <= 65535, "shortconv: too many row tiles (%d)", (int)grid.y);
  if (dtype == GIBBS_F32)
    shortconv_kernel<float><<<grid, 256, 0, stream>>>((const float*)bcx, taps, bias, state, slot_stride, cu, ctx,
                                                      slot, (float*)y, n_req, C, K);
  else if (dtype == GIBBS_BF16)
    shortconv_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)bcx, taps, bias, state, slot_stride, cu, ctx,
                                                     slot, (bf16*)y, n_req, C, K);
  else
    return gibbs_fail("shortconv: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("shortconv");
}
