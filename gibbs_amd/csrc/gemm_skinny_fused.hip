// Decode-step matrix products with the neighbouring operations fused in, so that a layer is a
// handful of kernels instead of a dozen (no kernel on this chip is shorter than about 4 us, and
// a decode step at small batch is a chain of products that each stream a few megabytes).
//
//   Y = X W^T for at most 64 rows of X (bfloat16), W streamed once straight into the A operand of
//   v_mfma_f32_16x16x32_bf16, the workgroup's waves splitting k and meeting in LDS, as in
//   gemm_skinny.  On top of that:
//
//   packed W      W may come in MFMA-tile order (`pack_weight`: [row group][16-row tile][32-k tile][lane][8],
//                  zero-padded): a wave's load of an A operand is then 1 KB of consecutive memory, 8 requests
//                  of 128 bytes instead of 16 of 64, which is worth a fifth of the time of these products
//                  (the compute unit's memory pipe is bound by requests in flight, not by bytes).
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
#include "activation.h"
#include <stdlib.h>

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_GLU = 2, EPI_CONV = 3 };
constexpr int MAX_TAPS = 8;

struct FusedArgs {
  int rotate;     // 1: workgroups start at different k (see the kernel)
  const bf16* W;
  int packed;        // W is in tile order
  int ktiles;        // packed: 32-k tiles per 16-row tile
  long group_tiles;  // packed: 16-row tiles per row group
  const bf16* X;   // [N, I] bfloat16 (the mirror of the residual stream when rms)
  int N, O, I;     // O: features per row group
  long ldw, ldx;
  long group_stride;  // rows of W between row groups
  float eps;          // rms prologue
  // STORE / GLU / CONV: bfloat16 output [N, ldy]
  bf16* Y;
  long ldy;
  // RESIDUAL
  float* x;   // [N, O] float32, updated in place
  bf16* xb;   // [N, O] mirror
  // CONV
  const float* taps;  // [O, K]
  const float* bias;  // [O] or null
  float* state;       // [slots, K-1, O]
  long slot_stride;
  const int* slot;  // [N]
  const int* ctx;   // [N] cached length of each row's request (history rows before position 0 are zero)
  int K;
  int act;  // GLU: the activation's code
};

// KC: the convolution's kernel length when it is 2..4 (its operands are then asked for before the
// product), 0 for any other length or epilogue.
// FT: tiles of ROWS features that a workgroup computes from the same B operands (more rows of X
// than one or two MFMA tiles: X is re-read from L2 by every workgroup, so a workgroup should use
// each B operand for more of W).  Wave f sums tile f over the waves and runs its epilogue.
template <int NT, int RG, int ROWS, int FT, int WAVES, bool RMS, int EPI, int KC>
__global__ __launch_bounds__(WAVES * WAVE) void gemm_skinny_fused_kernel(FusedArgs a) {
  static_assert(FT <= WAVES && (FT == 1 || EPI == EPI_STORE || EPI == EPI_GLU), "several tiles: store and GLU only");
  // More than 16 rows of X: a wave brings its part of X in through LDS, 128 contiguous bytes or more of
  // a row per request instead of the 64 that a lane group of an MFMA operand covers (the memory pipe
  // of a compute unit is bound by requests in flight).  The wave's region is its own: no barrier.
  constexpr bool STAGE = NT >= 2;
  constexpr int U = (FT * RG * NT >= 6) ? 2 : (FT * RG * NT == 1 ? 8 : 4);  // MFMA steps per iteration
  constexpr int CH = 4 * U;                    // 16-byte chunks of a row per iteration
  constexpr int RED_BYTES = WAVES * FT * RG * NT * WAVE * 16;
  constexpr int STAGE_BYTES = STAGE ? WAVES * NT * 16 * CH * 16 : 0;
  __shared__ __attribute__((aligned(16))) char smem[RED_BYTES > STAGE_BYTES ? RED_BYTES : STAGE_BYTES];
  floatx4 (*red)[FT][RG][NT][WAVE] = reinterpret_cast<floatx4 (*)[FT][RG][NT][WAVE]>(smem);
  bf16x8* stage = reinterpret_cast<bf16x8*>(smem) + (size_t)(threadIdx.x / WAVE) * NT * 16 * CH;
  __shared__ float red_ss[WAVES][NT][16];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int r = lane % 16, g = lane / 16;
  const int o0 = blockIdx.x * ROWS * FT;
  // the wave's share of k, in whole MFMA steps of 32
  const int steps = (a.I + 31) / 32;
  const int per_wave = (steps + WAVES - 1) / WAVES;
  const int k_begin = wave * per_wave * 32;
  const int k_end = min(a.I, k_begin + per_wave * 32);

  bool row_ok[FT];
  const bf16* wrow[FT][RG];
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    row_ok[f] = r < ROWS && o0 + f * ROWS + r < a.O;
#pragma unroll
    for (int q = 0; q < RG; ++q)
      if (a.packed) {
        // 16-row tile of the feature tile, and this lane's place in it (8-row workgroups take half a tile)
        const int o_tile = (o0 + f * ROWS) / 16;
        const int in_tile = ROWS == 16 ? lane : g * 16 + ((o0 / 8) % 2) * 8 + (r % 8);
        wrow[f][q] = a.W + (((size_t)q * a.group_tiles + o_tile) * a.ktiles) * 512 + in_tile * 8;
      } else {
        wrow[f][q] = a.W + ((size_t)q * a.group_stride + (row_ok[f] ? o0 + f * ROWS + r : 0)) * a.ldw + g * 8;
      }
  }
  const int kstride = a.packed ? 512 : 32;  // elements between a lane's A operands of consecutive MFMA steps
  const int koff = a.packed ? 0 : g * 8;    // packed tiles are whole (zero-padded)
  const bf16* xrow[NT];
  bool x_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    x_ok[t] = t * 16 + r < a.N;
    xrow[t] = a.X + (size_t)(x_ok[t] ? t * 16 + r : 0) * a.ldx + g * 8;
  }
  // What the epilogue reads besides the product is asked for now: the product hides the latency
  // (the state row hangs on a slot index, two dependent loads).  Wave 0 writes the outputs; its lane
  // holds features o_epi .. +3 of row t*16 + r.
  constexpr int KH = KC > 1 ? KC - 1 : 1;
  const int o_epi = o0 + g * 4;
  const bool epi_lane = wave == 0 && g * 4 < ROWS && o_epi < a.O;
  float pre_x[NT][4];          // RESIDUAL: the stream; CONV: unused
  float pre_hist[NT][KH][4];   // CONV: the state rows
  float pre_taps[KC > 1 ? KC : 1][4], pre_bias[4];
  if (EPI == EPI_RESIDUAL) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = t * 16 + r;
#pragma unroll
      for (int i = 0; i < 4; ++i) pre_x[t][i] = (epi_lane && n < a.N && o_epi + i < a.O) ? a.x[(size_t)n * a.O + o_epi + i] : 0.f;
    }
  }
  if (EPI == EPI_CONV && KC > 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = epi_lane && o_epi + i < a.O;
#pragma unroll
      for (int j = 0; j < KC; ++j) pre_taps[j][i] = ok ? a.taps[(size_t)(o_epi + i) * KC + j] : 0.f;
      pre_bias[i] = (ok && a.bias) ? a.bias[o_epi + i] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = t * 16 + r;
      const bool row = epi_lane && n < a.N;
      const float* st = a.state + (size_t)(row ? a.slot[n] : 0) * a.slot_stride;
      const int before = row ? a.ctx[n] : 0;
#pragma unroll
      for (int j = 0; j < KH; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          pre_hist[t][j][i] = (row && o_epi + i < a.O && before - (KC - 1) + j >= 0) ? st[(size_t)j * a.O + o_epi + i] : 0.f;
    }
  }

  floatx4 acc[FT][RG][NT];
  float ss[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    ss[t] = 0.f;
#pragma unroll
    for (int f = 0; f < FT; ++f)
#pragma unroll
      for (int q = 0; q < RG; ++q) acc[f][q][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // staging: lane l of load instruction i brings chunk (l % CH + rot) % CH of row i * (64 / CH) + l / CH to
  // slot i * 64 + l; rot(row) = row * U / 4 makes the operand reads below free of bank conflicts
  constexpr int RPI = WAVE / CH;               // rows per load instruction
  constexpr int LPT = 16 / RPI;                // load instructions per tile of 16 rows
  const bf16* srow[NT][LPT];
  bool s_ok[NT][LPT];
  int s_chunk[LPT];
  int read_slot[U];
  if (STAGE) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int row = i * RPI + lane / CH;
      s_chunk[i] = (lane % CH + row * U / 4) % CH;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        s_ok[t][i] = t * 16 + row < a.N;
        srow[t][i] = a.X + (size_t)(s_ok[t][i] ? t * 16 + row : 0) * a.ldx + s_chunk[i] * 8;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) read_slot[u] = r * CH + ((u * 4 + g - r * U / 4) & (CH - 1));
  }
  // Every workgroup reads the same rows of X: started at the same k, all of them would ask the same L2
  // channels for the same lines at the same time.  Workgroup b starts b iterations into its waves'
  // ranges and wraps around (the order of a feature's additions is fixed by its workgroup).
  const int n_iter = (k_end - k_begin + 32 * U - 1) / (32 * U);
  const int first_iter = (STAGE && n_iter > 0 && a.rotate) ? (int)(blockIdx.x % n_iter) : 0;
  for (int it = 0; it < n_iter; ++it) {
    const int k = k_begin + ((it + first_iter) % n_iter) * 32 * U;
    bf16x8 av[U][FT][RG], bv[U][NT];
    if (STAGE) {
      bf16x8 sv[NT][LPT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < LPT; ++i)
          sv[t][i] = (s_ok[t][i] && k + s_chunk[i] * 8 < k_end) ? *(const bf16x8*)(srow[t][i] + k) : zero;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kk = k + u * 32;
#pragma unroll
        for (int f = 0; f < FT; ++f)
#pragma unroll
          for (int q = 0; q < RG; ++q)
            av[u][f][q] = (row_ok[f] && kk + koff < k_end) ? *(const bf16x8*)(wrow[f][q] + (size_t)(kk / 32) * kstride) : zero;
      }
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < LPT; ++i) stage[(t * LPT + i) * WAVE + lane] = sv[t][i];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) bv[u][t] = stage[t * 16 * CH + read_slot[u]];
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kk = k + u * 32;
        const bool k_ok = kk + g * 8 < k_end;
#pragma unroll
        for (int f = 0; f < FT; ++f)
#pragma unroll
          for (int q = 0; q < RG; ++q)
            av[u][f][q] = (row_ok[f] && kk + koff < k_end) ? *(const bf16x8*)(wrow[f][q] + (size_t)(kk / 32) * kstride) : zero;
#pragma unroll
        for (int t = 0; t < NT; ++t) bv[u][t] = (x_ok[t] && k_ok) ? *(const bf16x8*)(xrow[t] + kk) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (RMS) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float v = (float)bv[u][t][e];
            ss[t] = fmaf(v, v, ss[t]);
          }
        }
#pragma unroll
        for (int f = 0; f < FT; ++f)
#pragma unroll
          for (int q = 0; q < RG; ++q)
            acc[f][q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u][f][q], bv[u][t], acc[f][q][t], 0, 0, 0);
      }
  }
  if (STAGE) __syncthreads();  // the staging regions become the reduction buffer

  // sum of squares of row n = t*16 + r: over the 4 lane groups, then over the waves
  if (RMS) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      ss[t] += __shfl_xor(ss[t], 16, WAVE);
      ss[t] += __shfl_xor(ss[t], 32, WAVE);
      if (g == 0) red_ss[wave][t][r] = ss[t];
    }
  }
  // the waves' partial products meet in LDS; wave f adds those of tile f in the order of the waves
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int q = 0; q < RG; ++q)
#pragma unroll
      for (int t = 0; t < NT; ++t) red[wave][f][q][t][lane] = acc[f][q][t];
  __syncthreads();
  if (wave >= FT) return;
  const int tile = wave;
  floatx4 sum[RG][NT];
#pragma unroll
  for (int q = 0; q < RG; ++q)
#pragma unroll
    for (int t = 0; t < NT; ++t) sum[q][t] = red[0][tile][q][t][lane];
#pragma unroll(RG * NT <= 2 ? WAVES : 1)
  for (int w = 1; w < WAVES; ++w)
#pragma unroll
    for (int q = 0; q < RG; ++q)
#pragma unroll
      for (int t = 0; t < NT; ++t) sum[q][t] += red[w][tile][q][t][lane];

  // D[feature g*4 + i][row r] of tile t: lane holds 4 consecutive features of one row
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = t * 16 + r;
    const int o = o0 + tile * ROWS + g * 4;
    if (n >= a.N || g * 4 >= ROWS || o >= a.O) continue;
    float scale = 1.f;
    if (RMS) {
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) tot += red_ss[w][t][r];
      scale = 1.0f / sqrtf(tot / (float)a.I + a.eps);
    }
    const bool full = o + 3 < a.O;
    if (EPI == EPI_STORE) {
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      if (full && a.ldy % 4 == 0) {
        *(bf16x4*)y = bf16x4{(bf16)(sum[0][t][0] * scale), (bf16)(sum[0][t][1] * scale), (bf16)(sum[0][t][2] * scale),
                             (bf16)(sum[0][t][3] * scale)};
      } else {
        for (int i = 0; i < 4 && o + i < a.O; ++i) y[i] = (bf16)(sum[0][t][i] * scale);
      }
    } else if (EPI == EPI_RESIDUAL) {
      float* xp = a.x + (size_t)n * a.O + o;
      bf16* bp = a.xb + (size_t)n * a.O + o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (o + i >= a.O) break;
        const float v = pre_x[t][i] + sum[0][t][i] * scale;
        xp[i] = v;
        bp[i] = (bf16)v;
      }
    } else if (EPI == EPI_GLU) {
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      for (int i = 0; i < 4 && o + i < a.O; ++i) {
        const float gt = sum[0][t][i] * scale, up = sum[RG > 1 ? 1 : 0][t][i] * scale;
        y[i] = (bf16)(activate(gt, a.act) * up);
      }
    } else if (KC > 1) {  // EPI_CONV, operands at hand
      float* st = a.state + (size_t)a.slot[n] * a.slot_stride;
      bf16* y = a.Y + (size_t)n * a.ldy + o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (o + i >= a.O) break;
        const int c = o + i;
        const float bx = (sum[0][t][i] * scale) * (sum[RG > 2 ? 2 : 0][t][i] * scale);
        const float cg = sum[RG > 1 ? 1 : 0][t][i] * scale;
        float cv = 0.f;
#pragma unroll
        for (int j = 0; j < KC - 1; ++j) cv = fmaf(pre_taps[j][i], pre_hist[t][j][i], cv);
        cv = fmaf(pre_taps[KC - 1][i], bx, cv);
        if (a.bias) cv += pre_bias[i];
        y[i] = (bf16)(cg * cv);
#pragma unroll
        for (int j = 0; j + 1 < KC - 1; ++j) st[(size_t)j * a.O + c] = pre_hist[t][j + 1][i];
        st[(size_t)(KC - 2) * a.O + c] = bx;
      }
    } else {  // EPI_CONV, any kernel length
      const int K = a.K;
      float* st = a.state + (size_t)a.slot[n] * a.slot_stride;
      const int before = a.ctx[n];
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      for (int i = 0; i < 4 && o + i < a.O; ++i) {
        const int c = o + i;
        const float bx = (sum[0][t][i] * scale) * (sum[RG > 2 ? 2 : 0][t][i] * scale);
        const float cg = sum[RG > 1 ? 1 : 0][t][i] * scale;
        float hist[MAX_TAPS - 1];
        float cv = 0.f;
#pragma unroll
        for (int j = 0; j < MAX_TAPS - 1; ++j) {
          hist[j] = 0.f;
          if (j < K - 1) {
            // history row j is position before - (K-1) + j; rows before the sequence start are zero
            if (before - (K - 1) + j >= 0) hist[j] = st[(size_t)j * a.O + c];
            cv = fmaf(a.taps[(size_t)c * K + j], hist[j], cv);
          }
        }
        cv = fmaf(a.taps[(size_t)c * K + K - 1], bx, cv);
        if (a.bias) cv += a.bias[c];
        y[i] = (bf16)(cg * cv);
#pragma unroll
        for (int j = 0; j < MAX_TAPS - 2; ++j)
          if (j + 1 < K - 1) st[(size_t)j * a.O + c] = hist[j + 1];
        st[(size_t)(K - 2) * a.O + c] = bx;
      }
    }
  }
}

template <int NT, int RG, bool RMS, int EPI, int KC>
void launch_rows(const FusedArgs& a, hipStream_t s) {
  constexpr int rows8_below = 256;   // tiles of 16 features below which a workgroup takes 8 (one per compute unit)
  constexpr int tiles2_from = 192;   // pairs of tiles from which a workgroup takes two (measured at 33 to 64 rows)
  if constexpr (NT >= 3 && (EPI == EPI_STORE || EPI == EPI_GLU)) {
    // many rows of X: two tiles of 16 features per workgroup where that still leaves enough workgroups
    if (a.O / 32 >= tiles2_from) {
      gemm_skinny_fused_kernel<NT, RG, 16, 2, 8, RMS, EPI, KC><<<ceil_div(a.O, 32), 8 * WAVE, 0, s>>>(a);
      return;
    }
  }
  // few features: halve the rows per workgroup so that every compute unit gets one
  if ((NT <= 2 || EPI == EPI_CONV) && a.O / 16 < rows8_below) {
    gemm_skinny_fused_kernel<NT, RG, 8, 1, 8, RMS, EPI, KC><<<ceil_div(a.O, 8), 8 * WAVE, 0, s>>>(a);
  } else {
    gemm_skinny_fused_kernel<NT, RG, 16, 1, 8, RMS, EPI, KC><<<ceil_div(a.O, 16), 8 * WAVE, 0, s>>>(a);
  }
}

template <int RG, bool RMS, int EPI, int KC = 0>
void launch_nt(const FusedArgs& a, hipStream_t s) {
  const int nt = ceil_div(a.N, 16);
  if (nt == 1) launch_rows<1, RG, RMS, EPI, KC>(a, s);
  else if (nt == 2) launch_rows<2, RG, RMS, EPI, KC>(a, s);
  else if (nt == 3) launch_rows<3, RG, RMS, EPI, KC>(a, s);
  else launch_rows<4, RG, RMS, EPI, KC>(a, s);
}

template <bool RMS>
void launch_conv(const FusedArgs& a, hipStream_t s) {
  switch (a.K) {
    case 2: launch_nt<3, RMS, EPI_CONV, 2>(a, s); break;
    case 3: launch_nt<3, RMS, EPI_CONV, 3>(a, s); break;
    case 4: launch_nt<3, RMS, EPI_CONV, 4>(a, s); break;
    default: launch_nt<3, RMS, EPI_CONV, 0>(a, s); break;
  }
}

int check_common(const char* what, const void* X, const void* W, int N, int O, int I, long ldx, long ldw) {
  GIBBS_REQUIRE(N > 0 && N <= 64 && O > 0 && I > 0, "%s: bad sizes N=%d O=%d I=%d (N up to 64)", what, N, O, I);
  GIBBS_REQUIRE(I % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "%s: inner size %d and row strides (%ld, %ld) must be multiples of 8", what, I, ldx, ldw);
  GIBBS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: operands must be 16-byte aligned", what);
  GIBBS_REQUIRE(ldx >= I && (ldw == 0 || ldw >= I), "%s: row strides shorter than rows", what);
  return 0;
}

// A row stride of 0 says that W is in tile order (pack_weight).
void note_layout(FusedArgs& a) {
  a.rotate = 1;
  if (a.ldw != 0) return;
  a.packed = 1;
  a.ktiles = ceil_div(a.I, 32);
  a.group_tiles = ceil_div(a.O, 16);
}
}  // namespace

// In all of these, ldw == 0 means that W is in tile order: [row group][ceil(O/16)][ceil(I/32)][64 lanes][8],
// lane (r, g) of a tile holding W[tile row * 16 + r][k tile * 32 + g * 8 .. + 8], zeros beyond O and I.
//
// Y[n, o] = scale_n * sum_k X[n, k] W[o, k], bfloat16 out; scale_n = 1/sqrt(mean_k X[n,k]^2 + eps) if rms.
GIBBS_EXPORT int gibbs_skinny_store(const void* X, const void* W, void* Y, int N, int O, int I, long ldx, long ldw,
                                    long ldy, int rms, float eps, hipStream_t stream) {
  if (check_common("skinny_store", X, W, N, O, I, ldx, ldw)) return 1;
  GIBBS_REQUIRE(ldy >= O, "skinny_store: output rows shorter than %d", O);
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = O; a.I = I; a.ldw = ldw; a.ldx = ldx; a.eps = eps; note_layout(a);
  a.Y = (bf16*)Y; a.ldy = ldy;
  if (rms) launch_nt<1, true, EPI_STORE>(a, stream);
  else launch_nt<1, false, EPI_STORE>(a, stream);
  GIBBS_LAUNCH_STATUS("skinny_store");
}

// x[n, o] += sum_k X[n, k] W[o, k];  xb[n, o] = bfloat16(x[n, o]).  x: [N, O] float32, xb: [N, O] bfloat16.
GIBBS_EXPORT int gibbs_skinny_residual(const void* X, const void* W, float* x, void* xb, int N, int O, int I, long ldx,
                                       long ldw, hipStream_t stream) {
  if (check_common("skinny_residual", X, W, N, O, I, ldx, ldw)) return 1;
  FusedArgs a{};
  a.W = (const bf16*)W; a.X = (const bf16*)X; a.N = N; a.O = O; a.I = I; a.ldw = ldw; a.ldx = ldx; note_layout(a);
  a.x = x; a.xb = (bf16*)xb;
  launch_nt<1, false, EPI_RESIDUAL>(a, stream);
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
  if (rms) launch_nt<2, true, EPI_GLU>(a, stream);
  else launch_nt<2, false, EPI_GLU>(a, stream);
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
  if (rms) launch_conv<true>(a, stream);
  else launch_conv<false>(a, stream);
  GIBBS_LAUNCH_STATUS("skinny_conv");
}
