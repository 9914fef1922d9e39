// The kernel that merges the key slices of an attention call: every slice of a (row, head) left
// (max of the scaled scores, sum of exp(score - max), values weighted by exp(score - max)) as hd + 2
// floats at partial[((row * heads + head) * slices + slice) * (hd + 2)].
#pragma once
#include "common.h"

namespace {
// Merges the slices of one (row, head): out = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s.
// One wave per (row, head): lanes first fetch the slices' (max, sum) side by side, then each lane
// sums its elements over the slices, four loads in flight at a time.
__global__ void attention_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int nh, int hd,
                                       int n_splits, long ldo) {
  const int row = blockIdx.x, head = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (head >= nh) return;
  const size_t stride = hd + 2;
  const float* ps = partial + ((size_t)row * nh + head) * n_splits * stride;
  float M = -INFINITY;
  for (int s0 = 0; s0 < n_splits; s0 += WAVE) {
    const int s = s0 + lane;
    M = fmaxf(M, wave_max(s < n_splits ? ps[s * stride] : -INFINITY));
  }
  float L = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += WAVE) {
    const int s = s0 + lane;
    float term = 0.f;
    if (s < n_splits) {
      const float ms = ps[s * stride];
      if (ms != -INFINITY) term = __expf(ms - M) * ps[s * stride + 1];
    }
    L += wave_sum(term);
  }
  const float inv = 1.0f / L;
  for (int e = lane; e < hd; e += WAVE) {
    float v = 0.f;
    int s = 0;
    for (; s + 4 <= n_splits; s += 4) {
      float ms[4], av[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) { ms[j] = ps[(s + j) * stride]; av[j] = ps[(s + j) * stride + 2 + e]; }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (ms[j] != -INFINITY) v = fmaf(__expf(ms[j] - M), av[j], v);
    }
    for (; s < n_splits; ++s) {
      const float m1 = ps[s * stride];
      if (m1 != -INFINITY) v = fmaf(__expf(m1 - M), ps[s * stride + 2 + e], v);
    }
    out[(size_t)row * ldo + (size_t)head * hd + e] = (bf16)(v * inv);
  }
}
}  // namespace
