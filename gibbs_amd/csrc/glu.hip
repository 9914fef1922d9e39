// Gated activation of a feed-forward:  out[n, f] = act(gu[n, f]) * gu[n, F + f], where the
// gate and up projections were computed as one product against [W_gate; W_up].
// The activation (activation.h: silu, two gelus, relu) is computed in float32.
#include "activation.h"

template <typename T>
__global__ void glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int F, int act) {
  const int n = blockIdx.x;
  const int f = blockIdx.y * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = to_float(gu[(size_t)n * 2 * F + f]);
  const float u = to_float(gu[(size_t)n * 2 * F + F + f]);
  out[(size_t)n * F + f] = from_float<T>(activate(g, act) * u);
}

// 8 elements (16 bytes of bfloat16) per thread: the pass is bound by memory traffic.
__global__ void glu_bf16x8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int F, int act) {
  const int n = blockIdx.x;
  const int f = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (f >= F) return;
  const uint4 gr = *(const uint4*)(gu + (size_t)n * 2 * F + f);
  const uint4 ur = *(const uint4*)(gu + (size_t)n * 2 * F + F + f);
  const uint32_t gw[4] = {gr.x, gr.y, gr.z, gr.w}, uw[4] = {ur.x, ur.y, ur.z, ur.w};
  uint32_t ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    const bf16 a0 = (bf16)(activate(g0, act) * u0);
    const bf16 a1 = (bf16)(activate(g1, act) * u1);
    ow[i] = (uint32_t)__builtin_bit_cast(unsigned short, a0) | ((uint32_t)__builtin_bit_cast(unsigned short, a1) << 16);
  }
  *(uint4*)(out + (size_t)n * F + f) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

GIBBS_EXPORT int gibbs_glu(const void* gu, void* out, int dtype, int n, int F, int act, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && F > 0, "glu: bad sizes n=%d F=%d", n, F);
  GIBBS_REQUIRE(act >= 0 && act < ACT_COUNT, "glu: unknown activation %d", act);
  GIBBS_REQUIRE(F <= 65535 * 256, "glu: width %d too large", F);
  if (n == 0) return 0;
  dim3 grid(n, ceil_div(F, 256));
  if (dtype == GIBBS_F32)
    glu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, F, act);
  else if (dtype == GIBBS_BF16 && F % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0)
    glu_bf16x8_kernel<<<dim3(n, ceil_div(F, 8 * 256)), 256, 0, stream>>>((const bf16*)gu, (bf16*)out, F, act);
  else if (dtype == GIBBS_BF16)
    glu_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, F, act);
  else
    return gibbs_fail("glu: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("glu");
}
