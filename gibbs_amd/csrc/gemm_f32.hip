// True 32-bit matrix product for the float32 path:  C[n, o] = sum_k A[n, k] * W[o, k].
// Plain FMA on the vector units (no matrix-core mode of reduced precision).  Every output
// element adds its products in ascending k, whatever tile it falls in, so a row's result
// does not depend on how many other rows the call holds.
// The same kernel with bfloat16 operands (float32 accumulation) takes the shapes that the
// matrix-core kernels refuse: inner sizes or row strides that are no multiple of 8.
#include "common.h"

namespace {
constexpr int TM = 64, TN = 64, TK = 16;

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                         OutT* __restrict__ C, int N, int O, int I, long lda,
                                                         long ldw, long ldc) {
  __shared__ float sa[TK][TM + 4];
  __shared__ float sw[TK][TN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int row0 = blockIdx.y * TM, col0 = blockIdx.x * TN;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < I; k0 += TK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;
      const int r = e / TK, k = e % TK;
      const int gr = row0 + r, gc = col0 + r, gk = k0 + k;
      sa[k][r] = (gr < N && gk < I) ? to_float(A[(size_t)gr * lda + gk]) : 0.f;
      sw[k][r] = (gc < O && gk < I) ? to_float(W[(size_t)gc * ldw + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sa[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = sw[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = row0 + ty * 4 + i;
    if (gr >= N) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = col0 + tx * 4 + j;
      if (gc < O) C[(size_t)gr * ldc + gc] = from_float<OutT>(acc[i][j]);
    }
  }
}
}  // namespace

// A: [N, I] (row stride lda), W: [O, I] (row stride ldw), C: [N, O] (row stride ldc), all float32.
GIBBS_EXPORT int gibbs_gemm_f32(const float* A, const float* W, float* C, int N, int O, int I, long lda,
                                long ldw, long ldc, hipStream_t stream) {
  GIBBS_REQUIRE(N >= 0 && O > 0 && I > 0, "gemm_f32: bad sizes N=%d O=%d I=%d", N, O, I);
  GIBBS_REQUIRE(lda >= I && ldw >= I && ldc >= O, "gemm_f32: row strides shorter than rows");
  if (N == 0) return 0;
  dim3 grid(ceil_div(O, TN), ceil_div(N, TM));
  GIBBS_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows (%d)", N);
  gemm_plain_kernel<float, float><<<grid, 256, 0, stream>>>(A, W, C, N, O, I, lda, ldw, ldc);
  GIBBS_LAUNCH_STATUS("gemm_f32");
}

// A: [N, I], W: [O, I] bfloat16 with any sizes and strides; C: [N, O] bfloat16 (out_dtype 1) or float32 (0).
GIBBS_EXPORT int gibbs_gemm_bf16_plain(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I,
                                       long lda, long ldw, long ldc, hipStream_t stream) {
  GIBBS_REQUIRE(N >= 0 && O > 0 && I > 0, "gemm_bf16_plain: bad sizes N=%d O=%d I=%d", N, O, I);
  GIBBS_REQUIRE(lda >= I && ldw >= I && ldc >= O, "gemm_bf16_plain: row strides shorter than rows");
  if (N == 0) return 0;
  dim3 grid(ceil_div(O, TN), ceil_div(N, TM));
  GIBBS_REQUIRE(grid.y <= 65535, "gemm_bf16_plain: too many rows (%d)", N);
  if (out_dtype == GIBBS_BF16)
    gemm_plain_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, N, O, I, lda, ldw, ldc);
  else if (out_dtype == GIBBS_F32)
    gemm_plain_kernel<bf16, float><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, N, O, I, lda, ldw, ldc);
  else
    return gibbs_fail("gemm_bf16_plain: unknown output dtype %d", out_dtype);
  GIBBS_LAUNCH_STATUS("gemm_bf16_plain");
}
