// Matrix product for few rows (decode: one row per live request, up to 64):
//   Y[n, o] = sum_k X[n, k] * W[o, k],  bfloat16 operands, float32 accumulation.
// The work is reading W once, so the layout serves that: a workgroup owns 16 output features and a
// range of k (or 4 such tiles at once, for many rows of X); its 8 waves split the range, each streaming its part of the 16 rows of W straight
// from memory into the A operand of v_mfma_f32_16x16x32_bf16 (a lane holds 8 consecutive k of one
// row, so no LDS staging is needed), with X (small, cache resident) as the B operand: 16 rows of
// X per MFMA, NT such tiles for up to 64 rows.  The waves' sums meet in LDS.  When 16-feature
// blocks alone cannot fill the chip, k is also split over workgroups (`k_splits`), each writing
// its float32 partial Y[s] for the consumer to add in a fixed order.
#include "common.h"
#include "packed_layout.h"
#include "kernels.h"
#include <type_traits>

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

enum { OUT_BF16 = 0, OUT_F32 = 1 };
constexpr int WAVES = 8;

// FT: tiles of 16 features per workgroup, computed from the same B operands (for more than 32 rows
// of X: every workgroup re-reads X from L2, so it should use each B operand for more of W).
template <int NT, int FT, int OUT>
__global__ __launch_bounds__(WAVES * WAVE) void gemm_skinny_kernel(const bf16* __restrict__ W, const bf16* __restrict__ X,
                                                          void* __restrict__ Yv, int N, int O, int I, long ldw,
                                                          long ldx, long ldy, int k_per_block, long split_stride, bool pair) {
  static_assert(FT <= WAVES, "wave f finishes tile f");
  // More than 16 rows of X: a wave brings its part of X in through LDS (its own region: no barrier),
  // 128 contiguous bytes or more of a row per request instead of the 64 that a lane group of an MFMA
  // operand covers; see gemm_skinny_fused.
  constexpr bool STAGE = NT >= 2;
  constexpr int U = FT * NT >= 8 ? 2 : 4;     // MFMA steps per iteration: U * FT loads of W in flight per lane
  constexpr int CH = 4 * U;                   // 16-byte chunks of a row per iteration
  constexpr int RED_BYTES = WAVES * FT * NT * WAVE * 16;
  constexpr int STAGE_BYTES = STAGE ? WAVES * NT * 16 * CH * 16 : 0;
  __shared__ __attribute__((aligned(16))) char smem[RED_BYTES > STAGE_BYTES ? RED_BYTES : STAGE_BYTES];
  floatx4 (*red)[FT][NT][WAVE] = reinterpret_cast<floatx4 (*)[FT][NT][WAVE]>(smem);
  bf16x8* stage = reinterpret_cast<bf16x8*>(smem) + (size_t)(threadIdx.x / WAVE) * NT * 16 * CH;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int r = lane % 16, g = lane / 16;
  const int o0 = blockIdx.x * 16 * FT;
  const int kb0 = blockIdx.y * k_per_block;
  const int kb1 = min(I, kb0 + k_per_block);
  // the wave's share of the block's range, in whole MFMA steps of 32
  const int steps = (kb1 - kb0 + 31) / 32;
  const int per_wave = (steps + WAVES - 1) / WAVES;
  const int k_begin = kb0 + wave * per_wave * 32;
  const int k_end = min(kb1, k_begin + per_wave * 32);

  // ldw == 0: W is in tile order (packed_layout.h; which of the two orders follows from O), a wave's A
  // operand 1 KB of consecutive memory (pair layout read here by 16 features: 8 pieces of 128 bytes)
  const bool packed = ldw == 0;
  const bool pairs = packed && pair;
  const int ktiles = pairs ? (I + 63) / 64 : (I + 31) / 32;
  bool row_ok[FT];
  const bf16* wrow[FT];
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    row_ok[f] = o0 + f * 16 + r < O;
    const size_t tile = min(o0 / 16 + f, (O + 15) / 16 - 1);   // (a tile beyond the last one: rows nobody stores)
    wrow[f] = pairs    ? W + ((2 * tile + r / 8) * ktiles) * 512 + (g * 16 + r % 8) * 8
              : packed ? W + (tile * ktiles) * 512 + lane * 8
                       : W + (size_t)(row_ok[f] ? o0 + f * 16 + r : 0) * ldw + g * 8;
  }
  const int koff = packed ? 0 : g * 8;
  // elements from wrow to the lane's A operand of 32-k tile j, clamped into the wave's range (so that every load
  // is unconditional; see gemm_skinny_fused.hip): packed, tile min(j, last tile); row-major, element
  // min(32 j + koff, I - 8) of the row
  const int a_limit = packed ? (k_end - 1) / 32 : I - 8;
  auto a_off = [&](int j) -> long {
    const int c = min(packed ? j : j * 32 + koff, a_limit);
    return pairs ? (long)(c >> 1) * 512 + (c & 1) * 64 : (packed ? (long)c * 512 : (long)c - koff);
  };
  const bf16* xrow[NT];
  bool x_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    x_ok[t] = t * 16 + r < N;
    xrow[t] = X + (size_t)(x_ok[t] ? t * 16 + r : 0) * ldx + g * 8;
  }
  floatx4 acc[FT][NT];
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[f][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int RPI = WAVE / CH;              // rows per staging load
  constexpr int LPT = 16 / RPI;               // staging loads per tile of 16 rows
  const bf16* srow[NT][LPT];
  bool s_ok[NT][LPT];
  int s_chunk[LPT];
  int read_slot[U];
  if (STAGE) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int row = i * RPI + lane / CH;
      s_chunk[i] = (lane % CH + row * U / 4) % CH;   // rotated so that the operand reads do not collide
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        s_ok[t][i] = t * 16 + row < N;
        srow[t][i] = X + (size_t)(s_ok[t][i] ? t * 16 + row : 0) * ldx + s_chunk[i] * 8;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) read_slot[u] = r * CH + ((u * 4 + g - r * U / 4) & (CH - 1));
  }
  // every workgroup of a k slice reads the same rows of X: workgroup b starts b iterations into its
  // waves' ranges and wraps around, so that they do not ask the same L2 channels at the same time
  const int n_iter = (k_end - k_begin + 32 * U - 1) / (32 * U);
  const int first_iter = (STAGE && n_iter > 0) ? (int)(blockIdx.x % n_iter) : 0;
  auto k_of = [&](int it) { return k_begin + ((it + first_iter) % n_iter) * 32 * U; };
  // Loads are unconditional and roll, as in gemm_skinny_fused.hip: as soon as a step's operands have been used
  // their registers are asked for the next stretch of k; rows of X beyond N give columns nobody stores, and
  // where k runs beyond the wave's range the rows of X are made zero before they are used.
  bf16x8 av[U][FT], bv[U][NT], sv[NT][LPT];
  auto load_a = [&](int k, int u) {
    const long off = a_off(k / 32 + u);
#pragma unroll
    for (int f = 0; f < FT; ++f) av[u][f] = *(const bf16x8*)(wrow[f] + off);
  };
  auto load_b = [&](int k, int u) {
    const int kc = min(k + u * 32 + g * 8, I - 8) - g * 8;
#pragma unroll
    for (int t = 0; t < NT; ++t) bv[u][t] = *(const bf16x8*)(xrow[t] + kc);
  };
  auto load_s = [&](int k) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int kc = min(k + s_chunk[i] * 8, I - 8) - s_chunk[i] * 8;
#pragma unroll
      for (int t = 0; t < NT; ++t) sv[t][i] = *(const bf16x8*)(srow[t][i] + kc);
    }
  };
  auto iteration = [&](int k, int k_next, auto more) {
    if (STAGE) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        const bool k_ok = k + s_chunk[i] * 8 < k_end;
#pragma unroll
        for (int t = 0; t < NT; ++t) stage[(t * LPT + i) * WAVE + lane] = k_ok ? sv[t][i] : zero;
      }
      if (more) load_s(k_next);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) bv[u][t] = stage[t * 16 * CH + read_slot[u]];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        bf16x8 b = bv[u][t];
        if (!STAGE && !(k + u * 32 + g * 8 < k_end)) b = zero;
#pragma unroll
        for (int f = 0; f < FT; ++f) acc[f][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u][f], b, acc[f][t], 0, 0, 0);
      }
      if (more) {
        load_a(k_next, u);
        if (!STAGE) load_b(k_next, u);
      }
    }
  };
  if (n_iter > 0) {
    int k = k_of(0);
    if (STAGE) load_s(k);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      load_a(k, u);
      if (!STAGE) load_b(k, u);
    }
    for (int it = 0; it + 1 < n_iter; ++it) {
      const int k_next = k_of(it + 1);
      iteration(k, k_next, std::true_type{});
      k = k_next;
    }
    iteration(k, 0, std::false_type{});
  }
  if (STAGE) __syncthreads();  // the staging regions become the reduction buffer

  // the waves' sums meet in LDS; the tiles of the result (FT of features by NT of rows) go round the waves, each
  // adding its tiles' parts in the order of the waves
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int t = 0; t < NT; ++t) red[wave][f][t][lane] = acc[f][t];
  __syncthreads();
  for (int unit = wave; unit < FT * NT; unit += WAVES) {
    const int tile = unit / NT, t = unit % NT;
    floatx4 sum = red[0][tile][t][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][tile][t][lane];
    // D[feature (lane/16)*4 + i][row lane%16]: 4 consecutive features of one row of Y
    const int n = t * 16 + r, o = o0 + tile * 16 + g * 4;
    if (n >= N) continue;
    if (OUT == OUT_BF16) {
      bf16* y = (bf16*)Yv + (size_t)n * ldy + o;
      if (o + 3 < O && (ldy % 4 == 0)) {
        typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
        bf16x4 v = {(bf16)sum[0], (bf16)sum[1], (bf16)sum[2], (bf16)sum[3]};
        *(bf16x4*)y = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (o + i < O) y[i] = (bf16)sum[i];
      }
    } else {
      float* y = (float*)Yv + (size_t)blockIdx.y * split_stride + (size_t)n * ldy + o;
      if (o + 3 < O && (ldy % 4 == 0)) {
        *(floatx4*)y = sum;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (o + i < O) y[i] = sum[i];
      }
    }
  }
}

template <int NT>
void launch(int out, int ft, int n_out, int k_splits, hipStream_t s, const bf16* W, const bf16* X, void* Y, int N, int O, int I,
            long ldw, long ldx, long ldy, int kpb, long ss) {
  if constexpr (NT >= 3) {
    if (ft == 4) {
      dim3 grid(ceil_div(n_out, 64), k_splits);
      if (out == OUT_BF16)
        gemm_skinny_kernel<NT, 4, OUT_BF16><<<grid, WAVES * WAVE, 0, s>>>(W, X, Y, N, O, I, ldw, ldx, ldy, kpb, ss, ldw == 0 && pair_layout(O));
      else
        gemm_skinny_kernel<NT, 4, OUT_F32><<<grid, WAVES * WAVE, 0, s>>>(W, X, Y, N, O, I, ldw, ldx, ldy, kpb, ss, ldw == 0 && pair_layout(O));
      return;
    }
  }
  dim3 grid(ceil_div(n_out, 16), k_splits);
  if (out == OUT_BF16)
    gemm_skinny_kernel<NT, 1, OUT_BF16><<<grid, WAVES * WAVE, 0, s>>>(W, X, Y, N, O, I, ldw, ldx, ldy, kpb, ss, ldw == 0 && pair_layout(O));
  else
    gemm_skinny_kernel<NT, 1, OUT_F32><<<grid, WAVES * WAVE, 0, s>>>(W, X, Y, N, O, I, ldw, ldx, ldy, kpb, ss, ldw == 0 && pair_layout(O));
}
}  // namespace

// X: [N <= 64, I], W: [O, I] bfloat16 (ldw == 0: in tile order, see the kernel).  k_splits == 1: Y [N, O] bfloat16 (out_dtype 1) or float32 (0).
// k_splits > 1: Y is float32 [k_splits, N, O] (split stride N * ldy): partial sums over k ranges.
GIBBS_EXPORT int gibbs_gemm_skinny(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx,
                                   long ldw, long ldy, int k_splits, hipStream_t stream) {
  GIBBS_REQUIRE(N > 0 && N <= 64 && O > 0 && I > 0, "gemm_skinny: bad sizes N=%d O=%d I=%d (N up to 64)", N, O, I);
  GIBBS_REQUIRE(I % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: inner size %d and row strides (%ld, %ld) must be multiples of 8", I, ldx, ldw);
  GIBBS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_skinny: operands must be 16-byte aligned");
  GIBBS_REQUIRE(ldx >= I && (ldw == 0 || ldw >= I) && ldy >= O, "gemm_skinny: row strides shorter than rows");
  GIBBS_REQUIRE(k_splits >= 1 && k_splits <= 1024, "gemm_skinny: %d k splits", k_splits);
  GIBBS_REQUIRE(k_splits == 1 || out_dtype == GIBBS_F32, "gemm_skinny: partial sums are float32");
  GIBBS_REQUIRE(out_dtype == GIBBS_F32 || out_dtype == GIBBS_BF16, "gemm_skinny: unknown output dtype %d", out_dtype);
  // up to three tiles of rows and whole sums: the kernel of the fused products (gemm_skinny_fused.hip) does the same
  // faster (measured on the head matrix: 17 to 48 rows; at 64 rows the tiled product is ahead)
  if (k_splits == 1 && N <= 48) return gibbs_skinny_store_as(X, W, Y, out_dtype, N, O, I, ldx, ldw, ldy, 0, 0.f, stream);
  // each block's k range is a whole number of 128-element steps (what one wave does per iteration)
  int kpb = ceil_div(ceil_div(I, k_splits), 128) * 128;
  const int used = ceil_div(I, kpb);
  GIBBS_REQUIRE(used == k_splits, "gemm_skinny: %d k splits leave some empty for inner size %d (use %d)", k_splits, I, used);
  const int out = out_dtype == GIBBS_BF16 ? OUT_BF16 : OUT_F32;
  // more than 32 rows of X: 4 tiles of 16 features per workgroup where that leaves enough workgroups
  const int ft = (N > 32 && (long)ceil_div(O, 64) * k_splits >= 128) ? 4 : 1;
  const long ss = (long)N * ldy;
  const bf16 *w = (const bf16*)W, *x = (const bf16*)X;
  const int nt = ceil_div(N, 16);
  if (nt == 1) launch<1>(out, ft, O, k_splits, stream, w, x, Y, N, O, I, ldw, ldx, ldy, kpb, ss);
  else if (nt == 2) launch<2>(out, ft, O, k_splits, stream, w, x, Y, N, O, I, ldw, ldx, ldy, kpb, ss);
  else if (nt == 3) launch<3>(out, ft, O, k_splits, stream, w, x, Y, N, O, I, ldw, ldx, ldy, kpb, ss);
  else launch<4>(out, ft, O, k_splits, stream, w, x, Y, N, O, I, ldw, ldx, ldy, kpb, ss);
  GIBBS_LAUNCH_STATUS("gemm_skinny");
}
