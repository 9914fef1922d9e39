// bfloat16 matrix product on the gfx950 matrix cores:  C[n, o] = sum_k A[n, k] * W[o, k],
// float32 accumulation, output bfloat16 or float32 (logits).
//
// Both operands are contiguous along k, which is the layout v_mfma_f32_32x32x16_bf16 wants for
// both of its inputs: a lane holds 8 consecutive k of one row.  A workgroup of 4 waves computes a
// 128 x 128 tile; each wave owns 64 x 64 of it as 2 x 2 MFMA tiles of 32 x 32.  Tiles of 64 k are
// staged through LDS (rows padded by 16 bytes against bank conflicts), double-buffered so that
// the next tile's global loads are in flight while the matrix cores work on the current one.
// Rows beyond N or O and k beyond I are read as zero.  I and the row strides must be multiples
// of 8 elements (16-byte loads).
#include "common.h"

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_LD = BK + 8;  // padded row, in elements

struct Tile {
  bf16 a[BM][LDS_LD];
  bf16 w[BN][LDS_LD];
};

template <typename OutT>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                        OutT* __restrict__ C, int N, int O, int I, long lda, long ldw,
                                                        long ldc) {
  __shared__ Tile tiles[2];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
  const int wr = (wave / 2) * 64, wc = (wave % 2) * 64;

  // each thread moves 4 chunks of 16 bytes per operand and tile
  uint4 ra[4], rw[4];
#define LOAD_GLOBAL(k0)                                                                   \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                         \
    const int c = tid + i * 256, r = c / 8, gk = (k0) + (c % 8) * 8;                      \
    ra[i] = make_uint4(0, 0, 0, 0);                                                       \
    rw[i] = make_uint4(0, 0, 0, 0);                                                       \
    if (row0 + r < N && gk < I) ra[i] = *(const uint4*)(A + (size_t)(row0 + r) * lda + gk); \
    if (col0 + r < O && gk < I) rw[i] = *(const uint4*)(W + (size_t)(col0 + r) * ldw + gk); \
  }
#define STORE_LDS(t)                                                \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) {                   \
    const int c = tid + i * 256, r = c / 8, kc = (c % 8) * 8;       \
    *(uint4*)&(t).a[r][kc] = ra[i];                                 \
    *(uint4*)&(t).w[r][kc] = rw[i];                                 \
  }

  floatx16 acc[2][2];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.f;

  const int n_tiles = (I + BK - 1) / BK;
  LOAD_GLOBAL(0)
  STORE_LDS(tiles[0])
  __syncthreads();
  for (int t = 0; t < n_tiles; ++t) {
    const Tile& cur = tiles[t & 1];
    if (t + 1 < n_tiles) { LOAD_GLOBAL((t + 1) * BK) }
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[2], fw[2];
      const int k = kk * 16 + (lane / 32) * 8;
#pragma unroll
      for (int m = 0; m < 2; ++m) fa[m] = *(const bf16x8*)&cur.a[wr + m * 32 + lane % 32][k];
#pragma unroll
      for (int n = 0; n < 2; ++n) fw[n] = *(const bf16x8*)&cur.w[wc + n * 32 + lane % 32][k];
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
          acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[m], fw[n], acc[m][n], 0, 0, 0);
    }
    if (t + 1 < n_tiles) {
      STORE_LDS(tiles[(t + 1) & 1])  // the other buffer: nobody reads it during this iteration
      __syncthreads();
    }
  }

  // D[row][col]: lane holds col = lane % 32 and rows (i / 4) * 8 + (lane / 32) * 4 + i % 4.
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int col = col0 + wc + n * 32 + lane % 32;
      if (col >= O) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = row0 + wr + m * 32 + (i / 4) * 8 + (lane / 32) * 4 + i % 4;
        if (row < N) C[(size_t)row * ldc + col] = from_float<OutT>(acc[m][n][i]);
      }
    }
}
#undef LOAD_GLOBAL
#undef STORE_LDS
}  // namespace

// A: [N, I] bfloat16, W: [O, I] bfloat16, C: [N, O] bfloat16 (out_dtype 1) or float32 (0).
GIBBS_EXPORT int gibbs_gemm_bf16(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda,
                                 long ldw, long ldc, hipStream_t stream) {
  GIBBS_REQUIRE(N >= 0 && O > 0 && I > 0, "gemm_bf16: bad sizes N=%d O=%d I=%d", N, O, I);
  GIBBS_REQUIRE(I % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: inner size %d and row strides (%ld, %ld) must be multiples of 8", I, lda, ldw);
  GIBBS_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_bf16: operands must be 16-byte aligned");
  GIBBS_REQUIRE(lda >= I && ldw >= I && ldc >= O, "gemm_bf16: row strides shorter than rows");
  if (N == 0) return 0;
  dim3 grid(ceil_div(O, BN), ceil_div(N, BM));
  GIBBS_REQUIRE(grid.y <= 65535, "gemm_bf16: too many rows (%d)", N);
  if (out_dtype == GIBBS_BF16)
    gemm_bf16_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, N, O, I, lda, ldw, ldc);
  else if (out_dtype == GIBBS_F32)
    gemm_bf16_kernel<float><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, N, O, I, lda, ldw, ldc);
  else
    return gibbs_fail("gemm_bf16: unknown output dtype %d", out_dtype);
  GIBBS_LAUNCH_STATUS("gemm_bf16");
}
