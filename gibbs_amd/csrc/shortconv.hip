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
    const int* __restrict__ slot, T* __restrict__ y, int n_req, int C, int K, int lead_single) {
  // The first lead_single requests bring one row each (decoded tokens): tile i is request i.  Behind them a walk
  // over the requests finds the tile's request and rows.
  int tile = blockIdx.y, r = tile, q = 1;
  if (tile < lead_single) {
    tile = 0;
  } else {
    tile -= lead_single;
    for (r = lead_single; r < n_req; ++r) {
      q = cu[r + 1] - cu[r];
      const int t = (q + TL - 1) / TL;
      if (tile < t) break;
      tile -= t;
    }
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
// The same for bfloat16 with 8 channels (16 bytes) per thread and the window kept in registers:
// a prompt portion is a pass over 3 + 1 values per (row, channel), bound by memory traffic.
// K is a template parameter (2..4, what LFM2 checkpoints use); other lengths take the kernel above.
constexpr int TLV = 8;   // rows per tile (>= K - 1)
constexpr int RU = 4;    // rows whose loads are in flight together

__device__ __forceinline__ void unpack8(const uint4& raw, float* f) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

template <int K>
__global__ __launch_bounds__(64) void shortconv_bf16x8_kernel(
    const bf16* __restrict__ bcx, const float* __restrict__ taps, const float* __restrict__ bias,
    float* __restrict__ state, long slot_stride, const int* __restrict__ cu, const int* __restrict__ ctx,
    const int* __restrict__ slot, bf16* __restrict__ y, int n_req, int C, int lead_single) {
  // (the first lead_single requests bring one row each: tile i is request i, and there is no walk)
  int tile = blockIdx.y, r = tile, q = 1;
  if (tile < lead_single) {
    tile = 0;
  } else {
    tile -= lead_single;
    for (r = lead_single; r < n_req; ++r) {
      q = cu[r + 1] - cu[r];
      const int t = (q + TLV - 1) / TLV;
      if (tile < t) break;
      tile -= t;
    }
  }
  if (r >= n_req) return;
  const int c0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c0 >= C) return;
  const int row0 = cu[r], before = ctx[r];
  float* st = state + (size_t)slot[r] * slot_stride;
  const size_t ld = (size_t)3 * C;
  float w[8][K], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    b[i] = bias ? bias[c0 + i] : 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) w[i][j] = taps[(size_t)(c0 + i) * K + j];
  }
  // B * x of row tp of this step's chunk (tp may be negative: the request's state, or zero before its start)
  auto bx_at = [&](int tp, float* out) {
    if (tp >= 0) {
      const bf16* row = bcx + (size_t)(row0 + tp) * ld + c0;
      float bv[8], xv[8];
      unpack8(*(const uint4*)row, bv);
      unpack8(*(const uint4*)(row + 2 * C), xv);
#pragma unroll
      for (int i = 0; i < 8; ++i) out[i] = bv[i] * xv[i];
    } else {
      const bool have = before + tp >= 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) out[i] = have ? st[(size_t)(K - 1 + tp) * C + c0 + i] : 0.f;
    }
  };
  const int t0 = tile * TLV, t_end = min(q, t0 + TLV);
  float win[K][8];  // win[j]: B * x of row t - (K-1) + j
#pragma unroll
  for (int j = 0; j < K - 1; ++j) bx_at(t0 - (K - 1) + j, win[j + 1]);
  for (int tg = t0; tg < t_end; tg += RU) {
    // the loads of RU rows first, then their arithmetic: a wave is alone with its rows' latency
    uint4 rb[RU], rx[RU], rc[RU];
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      rb[u] = rx[u] = rc[u] = make_uint4(0, 0, 0, 0);
      if (tg + u < t_end) {
        const bf16* row = bcx + (size_t)(row0 + tg + u) * ld + c0;
        rb[u] = *(const uint4*)row;
        rc[u] = *(const uint4*)(row + C);
        rx[u] = *(const uint4*)(row + 2 * C);
      }
    }
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int t = tg + u;
      if (t >= t_end) break;
#pragma unroll
      for (int j = 0; j < K - 1; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) win[j][i] = win[j + 1][i];
      float bv[8], xv[8], cg[8];
      unpack8(rb[u], bv);
      unpack8(rx[u], xv);
      unpack8(rc[u], cg);
#pragma unroll
      for (int i = 0; i < 8; ++i) win[K - 1][i] = bv[i] * xv[i];
      uint32_t ow[4];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < K; ++j) acc = fmaf(w[i][j], win[j][i], acc);
        acc += b[i];
        const uint32_t bits = (uint32_t)__builtin_bit_cast(unsigned short, (bf16)(cg[i] * acc));
        if (i % 2 == 0) ow[i / 2] = bits;
        else ow[i / 2] |= bits << 16;
      }
      *(uint4*)(y + (size_t)(row0 + t) * C + c0) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
  if (tile == 0) {
    // new[s] = window[q + s] reads old[q + s] (an index above s), so ascending s is safe
    for (int s2 = 0; s2 < K - 1; ++s2) {
      float v[8];
      bx_at(q - (K - 1) + s2, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) st[(size_t)s2 * C + c0 + i] = v[i];
    }
  }
}
}  // namespace

// lead_single: how many requests at the head of the batch bring exactly one row each (decoded tokens; 0 if unknown).
GIBBS_EXPORT int gibbs_shortconv(const void* bcx, const float* taps, const float* bias, float* state,
                                 long slot_stride, const int* cu, const int* ctx, const int* slot, void* y,
                                 int dtype, int n_rows, int n_req, int lead_single, int C, int K, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && n_req >= 0 && C > 0, "shortconv: bad sizes rows=%d requests=%d width=%d", n_rows, n_req, C);
  GIBBS_REQUIRE(K >= 2 && K - 1 <= TL, "shortconv: kernel length %d outside 2..%d", K, TL + 1);
  GIBBS_REQUIRE(slot_stride >= (long)(K - 1) * C, "shortconv: state slot stride %ld shorter than (K-1)*C", slot_stride);
  GIBBS_REQUIRE(lead_single >= 0 && lead_single <= n_req && lead_single <= n_rows, "shortconv: %d leading single rows among %d requests, %d rows", lead_single, n_req, n_rows);
  if (n_rows == 0 || n_req == 0) return 0;
  // tiles: one per leading single row; behind them at most ceil(rows / tile) + requests
  const int rest_rows = n_rows - lead_single, rest_req = n_req - lead_single;
  auto tiles = [&](int per) { return lead_single + (rest_req > 0 ? ceil_div(rest_rows, per) + rest_req : 0); };
  dim3 grid(ceil_div(C, 256), tiles(TL));
  GIBBS_REQUIRE(grid.y <= 65535, "shortconv: too many row tiles (%d)", (int)grid.y);
  if (dtype == GIBBS_F32)
    shortconv_kernel<float><<<grid, 256, 0, stream>>>((const float*)bcx, taps, bias, state, slot_stride, cu, ctx,
                                                      slot, (float*)y, n_req, C, K, lead_single);
  else if (dtype == GIBBS_BF16 && C % 8 == 0 && K >= 2 && K <= 4 && ((uintptr_t)bcx % 16) == 0 && ((uintptr_t)y % 16) == 0) {
    dim3 vgrid(ceil_div(C, 8 * 64), tiles(TLV));
    GIBBS_REQUIRE(vgrid.y <= 65535, "shortconv: too many row tiles (%d)", (int)vgrid.y);
    const bf16* in = (const bf16*)bcx;
    bf16* out = (bf16*)y;
    if (K == 2) shortconv_bf16x8_kernel<2><<<vgrid, 64, 0, stream>>>(in, taps, bias, state, slot_stride, cu, ctx, slot, out, n_req, C, lead_single);
    else if (K == 3) shortconv_bf16x8_kernel<3><<<vgrid, 64, 0, stream>>>(in, taps, bias, state, slot_stride, cu, ctx, slot, out, n_req, C, lead_single);
    else shortconv_bf16x8_kernel<4><<<vgrid, 64, 0, stream>>>(in, taps, bias, state, slot_stride, cu, ctx, slot, out, n_req, C, lead_single);
  } else if (dtype == GIBBS_BF16)
    shortconv_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)bcx, taps, bias, state, slot_stride, cu, ctx,
                                                     slot, (bf16*)y, n_req, C, K, lead_single);
  else
    return gibbs_fail("shortconv: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("shortconv");
}
