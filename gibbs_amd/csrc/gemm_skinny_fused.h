// The kernel of the fused few-row products and its launchers (see gemm_skinny_fused.hip for what they compute).
// Two translation units instantiate it: gemm_skinny_fused.hip for matrices in tile order, which is what a model's
// bound weights are, and gemm_skinny_fused_rows.hip for row-major ones (the instantiations are a large share of the
// library's compile time, and a kernel that knows its layout has less in front of its first loads).
#pragma once
#include "common.h"
#include "activation.h"
#include "packed_layout.h"
#include "kernels.h"
#include <stdlib.h>
#include <type_traits>

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_GLU = 2, EPI_CONV = 3 };

// The operand with lanes r and r ^ 8 of every 16 exchanged (a rotation by 8 within the row of lanes).
__device__ __forceinline__ bf16x8 swap_halves16(bf16x8 v) {
  typedef int int4v __attribute__((ext_vector_type(4)));
  int4v w = __builtin_bit_cast(int4v, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = __builtin_amdgcn_update_dpp(0, w[i], 0x128 /* row_ror:8 */, 0xf, 0xf, false);
  return __builtin_bit_cast(bf16x8, w);
}
constexpr int MAX_TAPS = 8;

struct FusedArgs {
  int rotate;     // 1: workgroups start at different k (see the kernel)
  const bf16* W;
  int packed;        // W is in tile order: 1 = 16-row tiles, 2 = 8-row tiles of two k tiles (packed_layout.h)
  int ktiles;        // packed: 32-k tiles per 16-row tile (pair layout: 64-k pairs per 8-row tile)
  long group_tiles;  // packed: 16-row tiles per row group
  const bf16* X;   // [N, I] bfloat16 (the mirror of the residual stream when rms)
  int N, O, I;     // O: features per row group
  long ldw, ldx;
  long group_stride;  // rows of W between row groups
  float eps;          // rms prologue
  float inv_I;        // 1 / I
  // STORE / GLU / CONV: bfloat16 output [N, ldy] (STORE: or float32, Yf)
  bf16* Y;
  float* Yf;
  int y_vec;   // a lane's four features take one store (rows and pointers are aligned for it)
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
// each B operand for more of W).  Wave f * NT + t sums tile f of features and tile t of rows over the waves
// and runs its epilogue.
template <bool TILED, int NT, int RG, int ROWS, int FT, int WAVES, bool RMS, int EPI, int KC, bool STAGE, bool BP = false>
__global__ __launch_bounds__(WAVES * WAVE) void gemm_skinny_fused_kernel(const bf16* W, const bf16* X, int N, int O, int I, int packed,
                                                                         int ktiles, int rotate, long group_tiles, long ldx,
                                                                         long ldw, FusedArgs rest) {
  // What the first loads need comes as scalar arguments, the first 14 dwords of which arrive in registers with
  // the wave (all but ldw, the row stride of a matrix that is not in tile order); the rest of the arguments is a
  // struct, which the kernel loads as it needs it.
  FusedArgs a = rest;
  a.W = W; a.X = X; a.N = N; a.O = O; a.I = I; a.packed = packed; a.ktiles = ktiles; a.rotate = rotate;
  a.group_tiles = group_tiles; a.ldw = ldw; a.ldx = ldx;
  // TILED: W is in tile order (pairs for workgroups of 8 features, else whichever the matrix has); not TILED:
  // row-major.  Known at compile time, the other layouts' address arithmetic is not in the way of the first loads.
  a.packed = TILED ? (ROWS == 8 ? 2 : (packed == 2 ? 2 : 1)) : 0;
  static_assert(FT * NT <= WAVES && (FT == 1 || EPI == EPI_STORE || EPI == EPI_GLU), "several tiles: store and GLU only; a wave per tile of the result");
  // STAGE (more than a few rows of X): a wave brings its part of X in through LDS, 128 contiguous bytes or
  // more of a row per request instead of the 64 that a lane group of an MFMA operand covers (the memory
  // pipe of a compute unit is bound by requests in flight, and from 8 rows on X is as many requests as W
  // for a workgroup of 8 features).  The wave's region is its own: no barrier.
  static_assert(STAGE || NT == 1 || BP, "more than 16 rows of X are staged");
  // MFMA steps per iteration (8 features and one tile of rows: an A operand serves two steps, so 8 steps are 4 loads a row group)
  constexpr int U = (ROWS == 8 && (NT == 1 || BP)) ? 8 : (FT * RG * NT >= 6) ? 2 : (FT * RG * NT == 1 ? 8 : 4);
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
  // the wave's share of k, in whole MFMA steps of 32 (workgroups of 8 features: in pairs of steps)
  constexpr bool PAIR = ROWS == 8;
  constexpr int KU = PAIR ? 64 : 32;
  static_assert(!PAIR || FT == 1, "8 features: one tile per workgroup");
  // BP (at most 16 rows of X, not staged): the B operands are pairs as well, rows 8..15 holding the same 8 rows
  // of X at the next 32 values of k, and a tile of rows is 8 rows of X (NT of them).  One MFMA then does two
  // steps: the upper left 8 x 8 block of its result is the product at k, the lower right one the product at
  // k + 32 (the other two blocks mix the two and are dropped).  A load of X is 8 requests of 128 bytes instead
  // of two loads of 8 requests of 64.
  // With 16 features the A operands are single steps: the step at k takes the pair as it is (columns 0..7 of the
  // result are the rows of X), the step at k + 32 takes it with the halves of every 16 lanes exchanged.
  static_assert(!BP || (NT <= 2 && !STAGE && FT == 1), "paired B operands: two tiles of 8 rows at most, one of features, not staged");
  constexpr int TILE_ROWS = BP ? 8 : 16;   // rows of X in a tile of rows
  const int steps = (a.I + KU - 1) / KU;
  const int per_wave = (steps + WAVES - 1) / WAVES;
  const int k_begin = wave * per_wave * KU;
  const int k_end = min(a.I, k_begin + per_wave * KU);

  // Where a lane's A operands lie: wrow + a_off(step), the step being the number of the 32-k tile (pairs: of
  // the 64-k pair) from the start of k.  One expression for all layouts, so that no branch stands between loads:
  //   j = min(step * a_unit + koff, a_limit);  offset = (j >> a_sh) * a_mul + (j & a_sh) * 64 - koff
  //   16-row tiles: tile j, 512 elements each.  Pair layout read by 16 features: pair j / 2, half j % 2.
  //   Row-major: element j of the row (a_unit elements per step).
  bool row_ok[FT];
  const bf16* wrow[FT][RG];
  int koff = 0, a_unit = 1, a_sh = 0, a_mul = 512;
  int a_limit = (k_end - 1) / KU;
  const int r8 = r % 8, half = r / 8;
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    row_ok[f] = r < ROWS && o0 + f * ROWS + r < a.O;
#pragma unroll
    for (int q = 0; q < RG; ++q) {
      if (a.packed == 2) {
        // 8-row tiles of two k tiles: [row group][8-row tile][pair][g][half][r8][8]
        const size_t tiles8 = 2 * a.group_tiles;
        if (PAIR) {
          wrow[f][q] = a.W + ((q * tiles8 + o0 / 8) * a.ktiles) * 512 + lane * 8;
        } else {
          const size_t o8 = min((size_t)(o0 + f * ROWS) / 8 + half, tiles8 - 1);   // (beyond the last tile: unused rows)
          wrow[f][q] = a.W + ((q * tiles8 + o8) * a.ktiles) * 512 + (g * 16 + r8) * 8;
          a_sh = 1;
        }
      } else if (a.packed) {
        // 16-row tiles (never read by workgroups of 8 features: the layout follows the number of rows)
        const int o_tile = min((o0 + f * ROWS) / 16, (int)a.group_tiles - 1);   // (beyond the last tile: unused rows)
        wrow[f][q] = a.W + (((size_t)q * a.group_tiles + o_tile) * a.ktiles) * 512 + lane * 8;
      } else {
        const int row = PAIR ? (o0 + r8 < a.O ? o0 + r8 : 0) : (row_ok[f] ? o0 + f * ROWS + r : 0);
        koff = (PAIR ? half * 32 : 0) + g * 8;
        wrow[f][q] = a.W + ((size_t)q * a.group_stride + row) * a.ldw + koff;
        a_unit = KU; a_limit = a.I - 8; a_mul = 1;
      }
    }
  }
  auto a_off = [&](int step) {
    const int j = min(step * a_unit + koff, a_limit);
    return (long)(j >> a_sh) * a_mul + (j & a_sh) * 64 - koff;
  };
  const bf16* xrow[NT];
  bool x_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = BP ? t * 8 + r8 : t * 16 + r;
    x_ok[t] = n < a.N;
    xrow[t] = a.X + (size_t)(x_ok[t] ? n : 0) * a.ldx + (BP ? half * 32 : 0) + g * 8;
  }
  // What the epilogue reads besides the product is asked for behind the first loads of the operands: the
  // product hides the latency (the state row hangs on a slot index, two dependent loads, and wave 0 would
  // start its share of W that much later if they came first).  The tiles of the result are written by a wave
  // each: wave f * NT + t has tile f of the features and tile t of the rows (one wave alone spent as long
  // on four tiles of rows as the product itself took); its lane holds features o_epi .. +3 of row n_epi.
  constexpr int KH = KC > 1 ? KC - 1 : 1;
  const int f_epi = wave / NT, t_epi = wave % NT;
  const int o_epi = o0 + f_epi * ROWS + g * 4;
  const int n_epi = t_epi * TILE_ROWS + r;
  const bool epi_lane = wave < FT * NT && g * 4 < ROWS && r < TILE_ROWS && o_epi < a.O && n_epi < a.N;
  float pre_x[4];          // RESIDUAL: the stream; CONV: unused
  float pre_hist[KH][4];   // CONV: the state rows
  float pre_taps[KC > 1 ? KC : 1][4], pre_bias[4];
  floatx4 acc[FT][RG][NT];
  floatx4 acc_hi[PAIR ? RG : 1][NT];   // 8 features: the products with X at k + 32 (rows 8..15 hold the features)
  floatx4 gram[NT];   // RMS: X X^T of the tile's rows (its diagonal is the rows' sums of squares)
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    gram[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int f = 0; f < FT; ++f)
#pragma unroll
      for (int q = 0; q < RG; ++q) acc[f][q][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < (PAIR ? RG : 1); ++q) acc_hi[q][t] = floatx4{0.f, 0.f, 0.f, 0.f};
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
  auto k_of = [&](int it) { return k_begin + ((it + first_iter) % n_iter) * 32 * U; };

  // Operands live in registers for one iteration of U MFMA steps.  As soon as a step's operands have been
  // used, the same registers are asked for the next iteration's step: a wave keeps U steps of loads in
  // flight all the time instead of waiting for an iteration's loads, working on them and asking again.
  // Every load is unconditional and its value is used as it comes (a load under a branch of its own, or a
  // select right behind it, makes the wave wait for all its loads in flight at once): addresses are clamped
  // into the matrices.  Rows of X beyond N give columns of the product that nobody stores.  Where k is beyond
  // the wave's range, which only the last stretch of the range can be, the rows of X are made zero before
  // they are used, so that whatever W holds there adds nothing.
  constexpr int UA = PAIR ? U / 2 : U;   // A operands per iteration (8 features: one serves two MFMA steps)
  constexpr int UB = BP ? U / 2 : U;     // B operands per iteration
  static_assert(U % 2 == 0, "pairs of MFMA steps");
  const int xoff = (BP ? half * 32 : 0) + g * 8;   // a lane's k within a B operand
  // (three and four tiles of rows: the staged rows of X are asked for behind the iteration's products instead of
  // before them: their registers would cost a second resident workgroup, or spill)
  constexpr bool ROLL_S = NT <= 2;
  bf16x8 av[UA][FT][RG], bv[UB][NT], sv[NT][LPT];
  auto load_a = [&](int k, int u) {   // u: the iteration's A operand
    const long off = a_off(k / KU + u);
#pragma unroll
    for (int f = 0; f < FT; ++f)
#pragma unroll
      for (int q = 0; q < RG; ++q) av[u][f][q] = *(const bf16x8*)(wrow[f][q] + off);
  };
  auto load_b = [&](int k, int u) {
    const int kc = min(k + u * (BP ? 64 : 32) + xoff, a.I - 8) - xoff;
#pragma unroll
    for (int t = 0; t < NT; ++t) bv[u][t] = *(const bf16x8*)(xrow[t] + kc);
  };
  // (one or two tiles of rows: a load instruction whose rows of X are all beyond N is left out, 17 rows are not 32,
  // and its registers stay zero; 1.3 to 1.7 % of a step at 17 to 24 rows.  With three and four tiles the branches
  // cost more than the loads they save)
  if constexpr (STAGE && NT <= 2) {
#pragma unroll
    for (int i = 0; i < LPT; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t) sv[t][i] = zero;
  }
  auto load_s = [&](int k) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int kc = min(k + s_chunk[i] * 8, a.I - 8) - s_chunk[i] * 8;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (NT > 2 || t * 16 + i * RPI < a.N) sv[t][i] = *(const bf16x8*)(srow[t][i] + kc);
    }
  };
  // One iteration on the operands of stretch k; `more`: the next stretch k_next is asked for.  `ragged`: k may
  // run beyond the wave's range within this stretch.
  auto iteration = [&](int k, int k_next, auto more, auto ragged) {
    if (STAGE) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        const bool k_ok = !ragged || k + s_chunk[i] * 8 < k_end;
#pragma unroll
        for (int t = 0; t < NT; ++t) stage[(t * LPT + i) * WAVE + lane] = k_ok ? sv[t][i] : zero;
      }
      if (ROLL_S && more) load_s(k_next);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) bv[u][t] = stage[t * 16 * CH + read_slot[u]];
    }
    if constexpr (BP) {
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        bf16x8 b[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          b[t] = bv[u][t];
          if (ragged && !(k + u * 64 + xoff < k_end)) b[t] = zero;
          if (RMS) gram[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[t], b[t], gram[t], 0, 0, 0);
        }
        if constexpr (PAIR) {
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < RG; ++q) acc[0][q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u][0][q], b[t], acc[0][q][t], 0, 0, 0);
          if (more) load_a(k_next, u);
        } else {
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < RG; ++q) acc[0][q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[2 * u][0][q], b[t], acc[0][q][t], 0, 0, 0);
          if (more) load_a(k_next, 2 * u);
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const bf16x8 b2 = swap_halves16(b[t]);
#pragma unroll
            for (int q = 0; q < RG; ++q) acc[0][q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[2 * u + 1][0][q], b2, acc[0][q][t], 0, 0, 0);
          }
          if (more) load_a(k_next, 2 * u + 1);
        }
        if (more) load_b(k_next, u);
      }
    } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        bf16x8 b = bv[u][t];
        if (!STAGE && ragged && !(k + u * 32 + g * 8 < k_end)) b = zero;
        if (RMS) gram[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, b, gram[t], 0, 0, 0);
#pragma unroll
        for (int f = 0; f < FT; ++f)
#pragma unroll
          for (int q = 0; q < RG; ++q) {
            if (PAIR && u % 2 == 1)
              acc_hi[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u / 2][f][q], b, acc_hi[q][t], 0, 0, 0);
            else
              acc[f][q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[PAIR ? u / 2 : u][f][q], b, acc[f][q][t], 0, 0, 0);
          }
      }
      if (more) {
        if (!PAIR) load_a(k_next, u);
        else if (u % 2 == 1) load_a(k_next, u / 2);
        if (!STAGE) load_b(k_next, u);
      }
    }
    }
    if (STAGE && !ROLL_S && more) load_s(k_next);
  };
  if (n_iter > 0) {
    const int k = k_of(0);
    if (STAGE) load_s(k);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (u < UA) load_a(k, u);
      if (!STAGE && u < UB) load_b(k, u);
    }
  }
  if (EPI == EPI_RESIDUAL) {
#pragma unroll
    for (int i = 0; i < 4; ++i) pre_x[i] = (epi_lane && o_epi + i < a.O) ? a.x[(size_t)n_epi * a.O + o_epi + i] : 0.f;
  }
  if (EPI == EPI_CONV && KC > 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = epi_lane && o_epi + i < a.O;
#pragma unroll
      for (int j = 0; j < KC; ++j) pre_taps[j][i] = ok ? a.taps[(size_t)(o_epi + i) * KC + j] : 0.f;
      pre_bias[i] = (ok && a.bias) ? a.bias[o_epi + i] : 0.f;
    }
    const float* st = a.state + (size_t)(epi_lane ? a.slot[n_epi] : 0) * a.slot_stride;
    const int before = epi_lane ? a.ctx[n_epi] : 0;
#pragma unroll
    for (int j = 0; j < KH; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        pre_hist[j][i] = (epi_lane && o_epi + i < a.O && before - (KC - 1) + j >= 0) ? st[(size_t)j * a.O + o_epi + i] : 0.f;
  }

  if (n_iter > 0) {
    int k = k_of(0);
    // (with the rotated start of the staged variant the range's last stretch may come at any iteration)
    for (int it = 0; it + 1 < n_iter; ++it) {
      const int k_next = k_of(it + 1);
      if (STAGE) iteration(k, k_next, std::true_type{}, std::true_type{});
      else iteration(k, k_next, std::true_type{}, std::false_type{});
      k = k_next;
    }
    iteration(k, 0, std::false_type{}, std::true_type{});
  }
  if (STAGE) __syncthreads();  // the staging regions become the reduction buffer

  // sum of squares of row n = t*16 + r: element (r, r) of the Gram matrix, which lane (r, r / 4) holds as its
  // element r % 4 (a lane holds rows g*4 .. g*4+3 of column r); then over the waves
  if (RMS) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int i = r % 4;
      const float d = i == 0 ? gram[t][0] : (i == 1 ? gram[t][1] : (i == 2 ? gram[t][2] : gram[t][3]));
      if (g == r / 4) red_ss[wave][t][r] = d;   // (paired B operands: rows 8..15 are rows 0..7 at k + 32)
    }
  }
  // the waves' partial products meet in LDS; wave f * NT + t adds those of its tile in the order of the waves
  // (8 features: lanes g < 2 hold them in the first accumulator, lanes g >= 2 in the second; lane l < 32 then
  // adds what lane l + 32 left)
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int q = 0; q < RG; ++q)
#pragma unroll
      for (int t = 0; t < NT; ++t) red[wave][f][q][t][lane] = (PAIR && !BP && g >= 2) ? acc_hi[PAIR ? q : 0][t] : acc[f][q][t];
  __syncthreads();
  if (wave >= FT * NT) return;
  // (paired B operands: the second half of feature (g, i) and row r is at rows + 8, columns + 8 of the tile)
  const int partner = BP ? (lane + 40) & 63 : (lane & 31) + 32;   // (8 features only)
  floatx4 sum[RG];
#pragma unroll
  for (int q = 0; q < RG; ++q) {
    sum[q] = red[0][f_epi][q][t_epi][lane];
    if (PAIR) sum[q] += red[0][f_epi][q][t_epi][partner];
  }
#pragma unroll
  for (int w = 1; w < WAVES; ++w)
#pragma unroll
    for (int q = 0; q < RG; ++q) {
      sum[q] += red[w][f_epi][q][t_epi][lane];
      if (PAIR) sum[q] += red[w][f_epi][q][t_epi][partner];
    }

  // D[feature g*4 + i][row r] of the tile: lane holds 4 consecutive features of one row
  {
    const int t = t_epi;
    const int n = n_epi;
    const int o = o_epi;
    if (n >= a.N || r >= TILE_ROWS || g * 4 >= ROWS || o >= a.O) return;
    float scale = 1.f;
    if (RMS) {
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) tot += red_ss[w][t][r] + (BP ? red_ss[w][t][(r + 8) & 15] : 0.f);
      scale = __builtin_amdgcn_rsqf(tot * a.inv_I + a.eps);   // (1 ulp: the outputs are rounded to bfloat16, or added to a stream that is)
    }
    const bool full = o + 3 < a.O;
    if (EPI == EPI_STORE && a.Yf) {
      float* y = a.Yf + (size_t)n * a.ldy + o;
      if (full && a.y_vec) {
        *(floatx4*)y = floatx4{sum[0][0] * scale, sum[0][1] * scale, sum[0][2] * scale, sum[0][3] * scale};
      } else {
        for (int i = 0; i < 4 && o + i < a.O; ++i) y[i] = sum[0][i] * scale;
      }
    } else if (EPI == EPI_STORE) {
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      if (full && a.ldy % 4 == 0) {
        *(bf16x4*)y = bf16x4{(bf16)(sum[0][0] * scale), (bf16)(sum[0][1] * scale), (bf16)(sum[0][2] * scale),
                             (bf16)(sum[0][3] * scale)};
      } else {
        for (int i = 0; i < 4 && o + i < a.O; ++i) y[i] = (bf16)(sum[0][i] * scale);
      }
    } else if (EPI == EPI_RESIDUAL) {
      float* xp = a.x + (size_t)n * a.O + o;
      bf16* bp = a.xb + (size_t)n * a.O + o;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = pre_x[i] + sum[0][i] * scale;
      if (full && a.y_vec) {   // (a lane's four features in one store each)
        *(floatx4*)xp = floatx4{v[0], v[1], v[2], v[3]};
        *(bf16x4*)bp = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
      } else {
        for (int i = 0; i < 4 && o + i < a.O; ++i) { xp[i] = v[i]; bp[i] = (bf16)v[i]; }
      }
    } else if (EPI == EPI_GLU) {
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      bf16 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gt = sum[0][i] * scale, up = sum[RG > 1 ? 1 : 0][i] * scale;
        v[i] = (bf16)(activate_to_bf16(gt, a.act) * up);
      }
      if (full && a.y_vec) *(bf16x4*)y = bf16x4{v[0], v[1], v[2], v[3]};
      else for (int i = 0; i < 4 && o + i < a.O; ++i) y[i] = v[i];
    } else if (KC > 1) {  // EPI_CONV, operands at hand
      float* st = a.state + (size_t)a.slot[n] * a.slot_stride;
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      float bx[4];
      bf16 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bx[i] = (sum[0][i] * scale) * (sum[RG > 2 ? 2 : 0][i] * scale);
        const float cg = sum[RG > 1 ? 1 : 0][i] * scale;
        float cv = 0.f;
#pragma unroll
        for (int j = 0; j < KC - 1; ++j) cv = fmaf(pre_taps[j][i], pre_hist[j][i], cv);
        cv = fmaf(pre_taps[KC - 1][i], bx[i], cv);
        if (a.bias) cv += pre_bias[i];
        v[i] = (bf16)(cg * cv);
      }
      if (full && a.y_vec) {
        *(bf16x4*)y = bf16x4{v[0], v[1], v[2], v[3]};
#pragma unroll
        for (int j = 0; j + 1 < KC - 1; ++j)
          *(floatx4*)(st + (size_t)j * a.O + o) = floatx4{pre_hist[j + 1][0], pre_hist[j + 1][1], pre_hist[j + 1][2], pre_hist[j + 1][3]};
        *(floatx4*)(st + (size_t)(KC - 2) * a.O + o) = floatx4{bx[0], bx[1], bx[2], bx[3]};
      } else {
        for (int i = 0; i < 4 && o + i < a.O; ++i) {
          const int c = o + i;
          y[i] = v[i];
#pragma unroll
          for (int j = 0; j + 1 < KC - 1; ++j) st[(size_t)j * a.O + c] = pre_hist[j + 1][i];
          st[(size_t)(KC - 2) * a.O + c] = bx[i];
        }
      }
    } else {  // EPI_CONV, any kernel length
      const int K = a.K;
      float* st = a.state + (size_t)a.slot[n] * a.slot_stride;
      const int before = a.ctx[n];
      bf16* y = a.Y + (size_t)n * a.ldy + o;
      for (int i = 0; i < 4 && o + i < a.O; ++i) {
        const int c = o + i;
        const float bx = (sum[0][i] * scale) * (sum[RG > 2 ? 2 : 0][i] * scale);
        const float cg = sum[RG > 1 ? 1 : 0][i] * scale;
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

#define FUSED_KERNEL_ARGS(a) (a).W, (a).X, (a).N, (a).O, (a).I, (a).packed, (a).ktiles, (a).rotate, (a).group_tiles, (a).ldx, (a).ldw, (a)

template <bool TILED, int NT, bool ST, int RG, bool RMS, int EPI, int KC>
void launch_rows(const FusedArgs& a, hipStream_t s) {
  constexpr int tiles2_from = 192;   // pairs of tiles from which a workgroup takes two (measured at 33 to 64 rows)
  if constexpr (NT >= 2 && (EPI == EPI_STORE || EPI == EPI_GLU)) {
    // many rows of X: two tiles of 16 features per workgroup where that still leaves enough workgroups
    // (also where single tiles would need a second round of workgroups that pairs do not: 257 to 383 tiles)
    if (a.O / 32 >= tiles2_from || (ceil_div(a.O, 16) > 256 && a.O / 32 >= 128)) {
      gemm_skinny_fused_kernel<TILED, NT, RG, 16, 2, 8, RMS, EPI, KC, ST><<<ceil_div(a.O, 32), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
      return;
    }
  }
  // few features: halve the rows per workgroup so that every compute unit gets one
  if ((NT <= 2 || EPI == EPI_CONV) && pair_layout(a.O)) {
    if constexpr (NT == 1 && !ST) {   // paired B operands: one tile of 8 rows of X, or two
      if (a.N <= 8) gemm_skinny_fused_kernel<TILED, 1, RG, 8, 1, 8, RMS, EPI, KC, ST, true><<<ceil_div(a.O, 8), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
      else gemm_skinny_fused_kernel<TILED, 2, RG, 8, 1, 8, RMS, EPI, KC, ST, true><<<ceil_div(a.O, 8), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
    } else {
      gemm_skinny_fused_kernel<TILED, NT, RG, 8, 1, 8, RMS, EPI, KC, ST><<<ceil_div(a.O, 8), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
    }
  } else {
    if constexpr (NT == 1 && !ST) {
      if (a.N <= 8) gemm_skinny_fused_kernel<TILED, 1, RG, 16, 1, 8, RMS, EPI, KC, ST, true><<<ceil_div(a.O, 16), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
      else gemm_skinny_fused_kernel<TILED, 2, RG, 16, 1, 8, RMS, EPI, KC, ST, true><<<ceil_div(a.O, 16), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
    } else {
      gemm_skinny_fused_kernel<TILED, NT, RG, 16, 1, 8, RMS, EPI, KC, ST><<<ceil_div(a.O, 16), 8 * WAVE, 0, s>>>(FUSED_KERNEL_ARGS(a));
    }
  }
}

template <bool TILED, int RG, bool RMS, int EPI, int KC = 0>
void launch_nt(const FusedArgs& a, hipStream_t s) {
  // Up to 16 rows of X come straight into paired B operands, except 9 to 16 rows where the product has no more
  // workgroups than the chip has compute units: those come through LDS.  Measured over whole decode steps of
  // three model shapes (hidden sizes 1024, 2048 and 2048 with wider feed-forwards): products of up to 2048
  // features (256 workgroups of 8) are 1 to 5 % of a step faster staged from 9 rows on and slower staged at 8
  // and below; products of 3072 features and more are faster unstaged through 16 rows (2 to 3 % of a step at 13
  // to 16 rows, the gate and up products most of all).
  constexpr int one_round = 256;   // workgroups of 8 features that get a compute unit each
  const bool staged = a.N > 8 && ceil_div(a.O, 8) <= one_round;
  const int nt = ceil_div(a.N, 16);
  if (nt == 1 && !staged) launch_rows<TILED, 1, false, RG, RMS, EPI, KC>(a, s);
  else if (nt == 1) launch_rows<TILED, 1, true, RG, RMS, EPI, KC>(a, s);
  else if (nt == 2) launch_rows<TILED, 2, true, RG, RMS, EPI, KC>(a, s);
  else if (nt == 3) launch_rows<TILED, 3, true, RG, RMS, EPI, KC>(a, s);
  else launch_rows<TILED, 4, true, RG, RMS, EPI, KC>(a, s);
}

template <bool TILED, bool RMS>
void launch_conv(const FusedArgs& a, hipStream_t s) {
  switch (a.K) {
    case 2: launch_nt<TILED, 3, RMS, EPI_CONV, 2>(a, s); break;
    case 3: launch_nt<TILED, 3, RMS, EPI_CONV, 3>(a, s); break;
    case 4: launch_nt<TILED, 3, RMS, EPI_CONV, 4>(a, s); break;
    default: launch_nt<TILED, 3, RMS, EPI_CONV, 0>(a, s); break;
  }
}

int check_common(const char* what, const void* X, const void* W, int N, int O, int I, long ldx, long ldw) {
  GIBBS_REQUIRE(N > 0 && N <= 64 && O > 0 && I > 0, "%s: bad sizes N=%d O=%d I=%d (N up to 64)", what, N, O, I);
  GIBBS_REQUIRE(I % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "%s: inner size %d and row strides (%ld, %ld) must be multiples of 8", what, I, ldx, ldw);
  GIBBS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: operands must be 16-byte aligned", what);
  GIBBS_REQUIRE(ldx >= I && (ldw == 0 || ldw >= I), "%s: row strides shorter than rows", what);
  return 0;
}

// A row stride of 0 says that W is in tile order; which of the two follows from the rows of a group (packed_layout.h).
void note_layout(FusedArgs& a) {
  a.rotate = 1;
  a.inv_I = 1.0f / (float)a.I;
  a.group_tiles = ceil_div(a.O, 16);
  if (a.ldw != 0) return;
  a.packed = pair_layout(a.O) ? 2 : 1;
  a.ktiles = a.packed == 2 ? ceil_div(a.I, 64) : ceil_div(a.I, 32);
}

// The four products on arguments that an entry point has filled in and checked.
template <bool TILED>
void run_store(const FusedArgs& a, bool rms, hipStream_t s) {
  if (rms) launch_nt<TILED, 1, true, EPI_STORE>(a, s);
  else launch_nt<TILED, 1, false, EPI_STORE>(a, s);
}
template <bool TILED>
void run_residual(const FusedArgs& a, hipStream_t s) { launch_nt<TILED, 1, false, EPI_RESIDUAL>(a, s); }
template <bool TILED>
void run_glu(const FusedArgs& a, bool rms, hipStream_t s) {
  if (rms) launch_nt<TILED, 2, true, EPI_GLU>(a, s);
  else launch_nt<TILED, 2, false, EPI_GLU>(a, s);
}
template <bool TILED>
void run_conv(const FusedArgs& a, bool rms, hipStream_t s) {
  if (rms) launch_conv<TILED, true>(a, s);
  else launch_conv<TILED, false>(a, s);
}
}  // namespace
