// A kernel that only reads: the sum of a buffer.  It is the yardstick that the weight-streaming kernels are held
// against (what a kernel of a given number of bytes can reach on this chip, inside a chain of dependent
// kernels), and serves measurement only: nothing on the product path calls it.
#include "common.h"

namespace {
__global__ void read_sum_kernel(const uint4* __restrict__ p, size_t n16, float* __restrict__ out) {
  __shared__ float red[16];
  float s = 0.f;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
    const uint4 v = p[i];
    s += __uint_as_float(v.x << 16) + __uint_as_float(v.y << 16) + __uint_as_float(v.z << 16) + __uint_as_float(v.w << 16);
  }
  for (int o = WAVE / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, WAVE);
  if (threadIdx.x % WAVE == 0) red[threadIdx.x / WAVE] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int w = 0; w < (int)blockDim.x / WAVE; ++w) t += red[w];
    out[blockIdx.x] = t;
  }
}
}  // namespace

// out: [grid] float32.  bytes: a multiple of 16, p 16-byte aligned; block: a multiple of 64 up to 1024.
GIBBS_EXPORT int gibbs_probe_read(const void* p, long bytes, float* out, int grid, int block, hipStream_t stream) {
  GIBBS_REQUIRE(bytes >= 0 && bytes % 16 == 0 && ((uintptr_t)p % 16) == 0, "probe_read: %ld bytes, 16-byte units", bytes);
  GIBBS_REQUIRE(grid > 0 && block >= WAVE && block <= 1024 && block % WAVE == 0, "probe_read: grid %d, block %d", grid, block);
  read_sum_kernel<<<grid, block, 0, stream>>>((const uint4*)p, (size_t)bytes / 16, out);
  GIBBS_LAUNCH_STATUS("probe_read");
}
