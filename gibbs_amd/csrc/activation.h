// The activations of a gated feed-forward, by the code that the host passes (one table for the
// stand-alone kernel and for the epilogue of the fused decode product).  All in float32.
#pragma once
#include "common.h"

enum { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_GELU = 2, ACT_RELU = 3, ACT_COUNT = 4 };

__device__ __forceinline__ float activate(float g, int act) {
  switch (act) {
    case ACT_GELU_TANH: {   // 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
      const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
      return 0.5f * g * (1.0f + tanhf(inner));
    }
    case ACT_GELU: return 0.5f * g * (1.0f + erff(g * 0.7071067811865476f));
    case ACT_RELU: return fmaxf(g, 0.0f);
    default: return g * (1.0f / (1.0f + expf(-g)));   // silu
  }
}

// The same for an epilogue whose result is rounded to bfloat16: silu by the hardware's exponential and reciprocal
// (a few units in the last place of float32), so that the serial tail of a product kernel stays short.
__device__ __forceinline__ float activate_to_bf16(float g, int act) {
  if (act == ACT_SILU) return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
  return activate(g, act);
}
