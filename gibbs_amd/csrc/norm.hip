// RMSNorm over rows of the float32 residual stream, fused with the residual add that
// precedes it:  v = x[r] (+ delta[r]);  (x[r] = v);  out[m] = v * rsqrt(mean(v^2) + eps) * gain.
// Sums, the root and the gain product are float32; the output takes the activation type.
// `rows` (optional) selects which rows are normed: out[m] comes from row rows[m].
#include "common.h"

template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                   const float* __restrict__ gain, float eps, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const T* dr = delta ? delta + (size_t)r * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += to_float(dr[i]);
      if (write_x) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* o = out + (size_t)m * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (dr && !write_x) v += to_float(dr[i]);
    o[i] = from_float<T>(gain ? v * scale * gain[i] : v * scale);
  }
}

// Four consecutive elements as one access.
__device__ __forceinline__ float4 load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4(const bf16* p) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
  const bf16x4 v = *(const bf16x4*)p;
  return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
}
__device__ __forceinline__ void store4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
  *(bf16x4*)p = bf16x4{(bf16)v.x, (bf16)v.y, (bf16)v.z, (bf16)v.w};
}

// The same for hidden sizes in steps of 4 up to 4 * CHUNKS * blockDim: a thread keeps its elements in
// registers between the sum and the scaling (one pass over memory, 16-byte accesses of the stream).
template <typename T, int CHUNKS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                       const float* __restrict__ gain, float eps, T* __restrict__ out,
                                       const int* __restrict__ rows, int hidden, int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const T* dr = delta ? delta + (size_t)r * hidden : nullptr;
  float4 v[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < hidden) {
      v[c] = *(const float4*)(xr + i);
      if (dr) {
        const float4 d = load4(dr + i);
        v[c].x += d.x; v[c].y += d.y; v[c].z += d.z; v[c].w += d.w;
        if (write_x) *(float4*)(xr + i) = v[c];
      }
      ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
    }
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* o = out + (size_t)m * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    if (i < hidden) {
      float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
      if (gain) g = *(const float4*)(gain + i);
      store4(o + i, make_float4(v[c].x * scale * g.x, v[c].y * scale * g.y, v[c].z * scale * g.z, v[c].w * scale * g.w));
    }
  }
}

template <typename T>
bool launch_vec(float* x, const T* delta, const float* gain, float eps, T* out, const int* rows, int n_out, int hidden,
                int write_x, hipStream_t stream) {
  const uintptr_t vec = 4 * sizeof(T);
  if (hidden % 4 || ((uintptr_t)x % 16) || (gain && ((uintptr_t)gain % 16)) || ((uintptr_t)out % vec) ||
      (delta && ((uintptr_t)delta % vec)))
    return false;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int chunks = ceil_div(hidden, 4 * threads);
  if (chunks == 1) add_rmsnorm_vec_kernel<T, 1><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks == 2) add_rmsnorm_vec_kernel<T, 2><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks <= 4) add_rmsnorm_vec_kernel<T, 4><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks <= 8) add_rmsnorm_vec_kernel<T, 8><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else return false;
  return true;
}

// x: [n_x, hidden] float32 residual stream (updated in place when delta is given and rows is null);
// out: [n_out, hidden]; rows: n_out row indices into x, or null with n_out == n_x.
GIBBS_EXPORT int gibbs_add_rmsnorm(float* x, const void* delta, const float* gain, float eps, void* out,
                                   int dtype, const int* rows, int n_out, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(n_out >= 0 && hidden > 0, "rmsnorm: bad sizes n=%d hidden=%d", n_out, hidden);
  if (n_out == 0) return 0;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int write_x = rows == nullptr;
  if (dtype == GIBBS_F32) {
    if (!launch_vec<float>(x, (const float*)delta, gain, eps, (float*)out, rows, n_out, hidden, write_x, stream))
      add_rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(x, (const float*)delta, gain, eps, (float*)out, rows, hidden, write_x);
  } else if (dtype == GIBBS_BF16) {
    if (!launch_vec<bf16>(x, (const bf16*)delta, gain, eps, (bf16*)out, rows, n_out, hidden, write_x, stream))
      add_rmsnorm_kernel<bf16><<<n_out, threads, 0, stream>>>(x, (const bf16*)delta, gain, eps, (bf16*)out, rows, hidden, write_x);
  } else {
    return gibbs_fail("rmsnorm: unknown dtype %d", dtype);
  }
  GIBBS_LAUNCH_STATUS("rmsnorm");
}

// The same with the delta given as float32 partial sums of a product split over k:
// delta[r] = sum_s partials[s][r], added in ascending s.
template <typename T>
__global__ void add_partials_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ partials, int n_partials,
                                            long partial_stride, const float* __restrict__ gain, float eps,
                                            T* __restrict__ out, const int* __restrict__ rows, int hidden,
                                            int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const float* pr = partials + (size_t)r * hidden;
  T* o = out + (size_t)m * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float d = 0.f;
    for (int s = 0; s < n_partials; ++s) d += pr[(size_t)s * partial_stride + i];
    const float v = xr[i] + d;
    if (write_x) xr[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (!write_x) {
      float d = 0.f;
      for (int s = 0; s < n_partials; ++s) d += pr[(size_t)s * partial_stride + i];
      v += d;
    }
    o[i] = from_float<T>(gain ? v * scale * gain[i] : v * scale);
  }
}

// partials: [n_partials, n_x, hidden] float32 (stride between partials given in elements).
GIBBS_EXPORT int gibbs_add_partials_rmsnorm(float* x, const float* partials, int n_partials, long partial_stride,
                                            const float* gain, float eps, void* out, int dtype, const int* rows,
                                            int n_out, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(n_out >= 0 && hidden > 0 && n_partials >= 1, "rmsnorm: bad sizes n=%d hidden=%d partials=%d", n_out, hidden, n_partials);
  if (n_out == 0) return 0;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int write_x = rows == nullptr;
  if (dtype == GIBBS_F32)
    add_partials_rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(x, partials, n_partials, partial_stride, gain, eps, (float*)out, rows, hidden, write_x);
  else if (dtype == GIBBS_BF16)
    add_partials_rmsnorm_kernel<bf16><<<n_out, threads, 0, stream>>>(x, partials, n_partials, partial_stride, gain, eps, (bf16*)out, rows, hidden, write_x);
  else
    return gibbs_fail("rmsnorm: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("rmsnorm");
}

// x[r] += delta[r] alone (the last residual add of a model whose tail norms only some rows
// still has to leave x whole for callers that read it).  float32 delta may be `n_partials` partial
// sums, `partial_stride` elements apart, added in ascending order.
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ delta, int n_partials,
                                    size_t partial_stride, bf16* __restrict__ mirror, size_t count) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    float v = x[i];
    if (delta)
      for (int s = 0; s < n_partials; ++s) v += to_float(delta[s * partial_stride + i]);
    x[i] = v;
    if (mirror) mirror[i] = (bf16)v;
  }
}

// x += delta (delta may be null); mirror (optional) = bfloat16(x).
GIBBS_EXPORT int gibbs_residual_add(float* x, const void* delta, int dtype, int n_partials, long partial_stride,
                                    void* mirror, long count, hipStream_t stream) {
  GIBBS_REQUIRE(count >= 0 && n_partials >= 1 && (n_partials == 1 || (dtype == GIBBS_F32 && partial_stride >= count)),
                "residual_add: bad count %ld or partial sums (%d, stride %ld)", count, n_partials, partial_stride);
  if (count == 0) return 0;
  const int blocks = ceil_div(count, 256);
  if (dtype == GIBBS_F32)
    residual_add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, n_partials, (size_t)partial_stride, (bf16*)mirror, (size_t)count);
  else if (dtype == GIBBS_BF16)
    residual_add_kernel<bf16><<<blocks, 256, 0, stream>>>(x, (const bf16*)delta, 1, 0, (bf16*)mirror, (size_t)count);
  else
    return gibbs_fail("residual_add: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("residual_add");
}
