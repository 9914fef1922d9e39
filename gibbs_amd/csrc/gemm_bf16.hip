// bfloat16 matrix product on the gfx950 matrix cores:  C[n, o] = sum_k A[n, k] * W[o, k],
// float32 accumulation, output bfloat16 or float32 (logits).
//
// Both operands are contiguous along k, which is the layout v_mfma_f32_32x32x16_bf16 wants for
// both of its inputs: a lane holds 8 consecutive k of one row.  A workgroup of 4 waves computes a
// 128 x 128 tile; each wave owns 64 x 64 of it as 2 x 2 MFMA tiles of 32 x 32.  Tiles of 64 k are
// staged through LDS (rows padded by 16 bytes against bank conflicts), double-buffered so that
// the next tile's global loads are in flight while the matrix cores work on the current one.
// Rows beyond N or O and k beyond I are read as zero.  I and the row strides must be multiples
// of 8 elements (16-byte loads).  Large aligned shapes take a 256 x 256 kernel (below).
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

// The same product for large aligned shapes (N and O multiples of 256, I of 64): a workgroup of 8 waves
// computes 256 x 256, each wave 128 tokens x 64 features as 4 x 2 MFMA tiles (two waves per SIMD), and
// asks LDS for fewer operand bytes per product than the 128 x 128 kernel.  Tiles of 64 k travel
// global -> LDS without passing through registers (global_load_lds, 16 bytes a lane; a wave's
// instruction covers 8 whole rows of 128 bytes).  LDS holds three tiles of A and two of W (160 KB): W
// is asked for one tile ahead and A two, so that loads stay in flight across the tile's barrier.  The
// loads are issued one after every four products: issued together they block the wave for as long as
// the memory pipe takes to accept them (measured: 1,500 cycles a tile with idle matrix cores).  A tile
// in LDS is [256 rows][64 k] with the 16-byte chunk c of row r at position c ^ ((r >> 1) & 7): the lane
// that fills slot (r, p) loads chunk p ^ ((r >> 1) & 7) from memory, and the operand reads
// (ds_read_b128, 32 rows x one chunk per instruction) are free of bank conflicts (measured: none).
// The product is computed transposed (features x tokens), so a lane's results are 4 consecutive
// features of one row.  Workgroups are numbered so that the 32 that an XCD runs at a time share 8
// tiles of W and 4 of A.
constexpr int TM = 256, TN = 256, TK = 64, TILE_ELEMS = 256 * TK;
__device__ __forceinline__ int swizzled(int row, int chunk) { return row * TK + ((chunk ^ ((row >> 1) & 7)) << 3); }

template <typename OutT>
__global__ __launch_bounds__(512) void gemm_bf16_256_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                            OutT* __restrict__ C, int I, long lda, long ldw, long ldc,
                                                            int tiles_n, int tiles_o) {
  extern __shared__ __attribute__((aligned(16))) bf16 lds_tiles[];
  bf16* sA = lds_tiles;                     // [3][TILE_ELEMS]
  bf16* sB = lds_tiles + 3 * TILE_ELEMS;    // [2][TILE_ELEMS]
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int total = tiles_n * tiles_o;
  int tn, to;
  if (total % 8 == 0 && (total / 8) % tiles_n == 0) {
    // workgroup b runs on XCD b % 8: each XCD takes a contiguous range of W tiles, W varying fastest
    const int b = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
    const int per = total / 8, i = b % per, x = b / per, wt = per / tiles_n;
    to = x * wt + i % wt;
    tn = i / wt;
  } else {
    tn = blockIdx.x % tiles_n;
    to = blockIdx.x / tiles_n;
  }
  const int row0 = tn * TM, col0 = to * TN;
  const int wm = wave / 4, wn = wave % 4;
  const int lp = tid % 8, lr = tid / 8;
  // instruction i (0..3) of a tile's loads: this thread fills slot (row lr + 64 i, position lp)
  auto load_one = [&](const bf16* G, long ld, int g0, int k0, bf16* dst, int i) {
    const int r = lr + 64 * i;
    const int c = lp ^ ((r >> 1) & 7);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(G + (size_t)(g0 + r) * ld + k0 + c * 8),
                                     (__attribute__((address_space(3))) void*)(dst + (wave * 64 + i * 512) * 8), 16, 0, 0);
  };
  floatx16 acc[2][4];   // [feature tile][token tile]
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[n][m][i] = 0.f;

  const int nt = I / TK;
  // A(0), W(0), A(1) before the loop (a tile beyond the last is the last once more: harmless, and the
  // count of loads in flight stays the same in every iteration)
#pragma unroll
  for (int i = 0; i < 4; ++i) load_one(A, lda, row0, 0, sA, i);
#pragma unroll
  for (int i = 0; i < 4; ++i) load_one(W, ldw, col0, 0, sB, i);
#pragma unroll
  for (int i = 0; i < 4; ++i) load_one(A, lda, row0, min(1, nt - 1) * TK, sA + TILE_ELEMS, i);
  const int r32 = lane % 32, h = lane / 32;
  for (int t = 0; t < nt; ++t) {
    // A(t) and W(t) have landed (this thread's part; the barrier covers the others'); the four loads of
    // A(t+1) may still be on their way
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    // (the bare barrier: __syncthreads() carries a fence, for which the compiler waits until no load is in flight;
    // a tile's operands were read from LDS into registers before its products, which stand before this barrier)
    __builtin_amdgcn_s_barrier();
    const int kb = min(t + 1, nt - 1) * TK, ka = min(t + 2, nt - 1) * TK;
    bf16* dB = sB + ((t + 1) & 1) * TILE_ELEMS;
    bf16* dA = sA + ((t + 2) % 3) * TILE_ELEMS;
    const bf16* cA = sA + (t % 3) * TILE_ELEMS;
    const bf16* cB = sB + (t & 1) * TILE_ELEMS;
#pragma unroll
    for (int kk = 0; kk < TK / 16; ++kk) {
      bf16x8 fa[4], fb[2];
      const int chunk = kk * 2 + h;
#pragma unroll
      for (int m = 0; m < 4; ++m) fa[m] = *(const bf16x8*)(cA + swizzled(wm * 128 + m * 32 + r32, chunk));
#pragma unroll
      for (int n = 0; n < 2; ++n) fb[n] = *(const bf16x8*)(cB + swizzled(wn * 64 + n * 32 + r32, chunk));
#pragma unroll
      for (int n = 0; n < 2; ++n) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
          acc[n][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[n], fa[m], acc[n][m], 0, 0, 0);
        // one load of the tiles to come after every four products: W(t+1) first (it has to be through at
        // the next barrier), then A(t+2)
        const int j = kk * 2 + n;
        if (j < 4) load_one(W, ldw, col0, kb, dB, j);
        else load_one(A, lda, row0, ka, dA, j - 4);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be writing LDS when the workgroup ends
  // D[feature i][token j]: lane holds token j = lane % 32 and features (v / 4) * 8 + (lane / 32) * 4 + v % 4
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      OutT* out = C + (size_t)(row0 + wm * 128 + m * 32 + r32) * ldc + col0 + wn * 64 + n * 32 + h * 4;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) out[q * 8 + e] = from_float<OutT>(acc[n][m][q * 4 + e]);
    }
}

template <typename OutT>
int launch_256(const bf16* A, const bf16* W, OutT* C, int N, int O, int I, long lda, long ldw, long ldc, hipStream_t stream) {
  constexpr int LDS_BYTES = 5 * TILE_ELEMS * (int)sizeof(bf16);   // three tiles of A, two of W
  static bool prepared = false;    // (per output type: the template makes one flag each)
  if (!prepared) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_256_kernel<OutT>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return gibbs_fail("gemm_bf16: %s", hipGetErrorString(e));
    prepared = true;
  }
  const int tiles_n = N / TM, tiles_o = O / TN;
  gemm_bf16_256_kernel<OutT><<<tiles_n * tiles_o, 512, LDS_BYTES, stream>>>(A, W, C, I, lda, ldw, ldc, tiles_n, tiles_o);
  GIBBS_LAUNCH_STATUS("gemm_bf16");
}

// Large aligned shapes that fill the chip with 256 x 256 tiles take the kernel above.
bool takes_256(int N, int O, int I, long ldc) {
  return N % TM == 0 && O % TN == 0 && I % TK == 0 && ldc % 4 == 0 && (long)(N / TM) * (O / TN) >= 192;
}
}  // namespace

// A: [N, I] bfloat16, W: [O, I] bfloat16, C: [N, O] bfloat16 (out_dtype 1) or float32 (0).
GIBBS_EXPORT int gibbs_gemm_bf16(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda,
                                 long ldw, long ldc, hipStream_t stream) {
  GIBBS_REQUIRE(N >= 0 && O > 0 && I > 0, "gemm_bf16: bad sizes N=%d O=%d I=%d", N, O, I);
  GIBBS_REQUIRE(I % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: inner size %d and row strides (%ld, %ld) must be multiples of 8", I, lda, ldw);
  GIBBS_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_bf16: operands must be 16-byte aligned");
  GIBBS_REQUIRE(lda >= I && ldw >= I && ldc >= O, "gemm_bf16: row strides shorter than rows");
  if (N == 0) return 0;
  if (takes_256(N, O, I, ldc)) {
    if (out_dtype == GIBBS_BF16) return launch_256((const bf16*)A, (const bf16*)W, (bf16*)C, N, O, I, lda, ldw, ldc, stream);
    if (out_dtype == GIBBS_F32) return launch_256((const bf16*)A, (const bf16*)W, (float*)C, N, O, I, lda, ldw, ldc, stream);
  }
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
