// Token embedding: x[n, :] = float(table[ids[n], :]).  The residual stream is float32
// whatever the table's type is.
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ x, bf16* __restrict__ mirror, int hidden, int vocab) {
  const int n = blockIdx.x;
  int id = ids[n];
  // The host checks ids it uploads; a sampled id is < vocab by construction.  Clamp so that
  // a bad id can never read outside the table.
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * hidden;
  float* out = x + (size_t)n * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_float(row[i]);
    out[i] = v;
    if (mirror) mirror[(size_t)n * hidden + i] = (bf16)v;
  }
}

// mirror (optional): the same rows rounded to bfloat16, [n, hidden].
GIBBS_EXPORT int gibbs_embed(const void* table, int dtype, const int* ids, float* x, void* mirror, int n,
                             int hidden, int vocab, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
  if (n == 0) return 0;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (dtype == GIBBS_F32)
    embed_kernel<float><<<n, threads, 0, stream>>>((const float*)table, ids, x, (bf16*)mirror, hidden, vocab);
  else if (dtype == GIBBS_BF16)
    embed_kernel<bf16><<<n, threads, 0, stream>>>((const bf16*)table, ids, x, (bf16*)mirror, hidden, vocab);
  else
    return gibbs_fail("embed: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("embed");
}
