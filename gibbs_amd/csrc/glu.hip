// Gated activation of a feed-forward:  out[n, f] = act(gu[n, f]) * gu[n, F + f], where the
// gate and up projections were computed as one product against [W_gate; W_up].
// silu(g) = g * 1 / (1 + exp(-g)), in float32.
#include "common.h"

enum { ACT_SILU = 0 };

template <typename T>
__global__ void glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int F, int act) {
  const int n = blockIdx.x;
  const int f = blockIdx.y * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = to_float(gu[(size_t)n * 2 * F + f]);
  const float u = to_float(gu[(size_t)n * 2 * F + F + f]);
  const float a = g * (1.0f / (1.0f + expf(-g)));
  out[(size_t)n * F + f] = from_float<T>(a * u);
}

GIBBS_EXPORT int gibbs_glu(const void* gu, void* out, int dtype, int n, int F, int act, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && F > 0, "glu: bad sizes n=%d F=%d", n, F);
  GIBBS_REQUIRE(act == ACT_SILU, "glu: unknown activation %d", act);
  GIBBS_REQUIRE(F <= 65535 * 256, "glu: width %d too large", F);
  if (n == 0) return 0;
  dim3 grid(n, ceil_div(F, 256));
  if (dtype == GIBBS_F32)
    glu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, F, act);
  else if (dtype == GIBBS_BF16)
    glu_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, F, act);
  else
    return gibbs_fail("glu: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("glu");
}
