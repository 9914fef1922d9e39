// The kernel that merges the key slices of an attention call: every slice of a (row, head) left
// (max of the scaled scores, sum of exp(score - max), values weighted by exp(score - max)) as hd + 2
// floats at partial[((row * heads + head) * slices + slice) * (hd + 2)].
#pragma once
#include "common.h"

namespace {
// Merges the slices of one (row, head): out = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s.
// One wave per (row, head).  Up to 16 slices (what a decode step has): every lane asks for all the slices'
// (max, sum) and for its elements of all slices at once, one round trip to memory on the step's critical
// path, and does the whole arithmetic itself.  More slices: lanes first fetch the (max, sum) side by side,
// then each lane sums its elements over the slices, four loads in flight at a time.
// C: elements of a head per lane (head sizes up to 64 C); MERGE_AT_ONCE: slices merged with all loads at once.
template <int C, int MERGE_AT_ONCE>
__global__ void attention_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int nh, int hd,
                                       int n_splits, long ldo) {
  const int row = blockIdx.x, head = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (head >= nh) return;
  const size_t stride = hd + 2;
  const float* ps = partial + ((size_t)row * nh + head) * n_splits * stride;
  if (n_splits <= MERGE_AT_ONCE && hd <= C * WAVE) {
    float ms[MERGE_AT_ONCE], ls[MERGE_AT_ONCE], av[MERGE_AT_ONCE][C];
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j) {
      const int s = j < n_splits ? j : 0;      // (beyond the last slice: the first one again, weighted 0 below)
      ms[j] = ps[s * stride];
      ls[j] = ps[s * stride + 1];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const int e = lane + c * WAVE;
        av[j][c] = ps[s * stride + 2 + (e < hd ? e : 0)];
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // every load is asked for before the first value is used: one round trip
    float M = -INFINITY;
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j)
      if (j < n_splits) M = fmaxf(M, ms[j]);
    float L = 0.f, v[C];
#pragma unroll
    for (int c = 0; c < C; ++c) v[c] = 0.f;
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j) {
      const float w = (j < n_splits && ms[j] != -INFINITY) ? __expf(ms[j] - M) : 0.f;
      L = fmaf(w, ls[j], L);
#pragma unroll
      for (int c = 0; c < C; ++c) v[c] = fmaf(w, av[j][c], v[c]);
    }
    const float inv = 1.0f / L;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int e = lane + c * WAVE;
      if (e < hd) out[(size_t)row * ldo + (size_t)head * hd + e] = (bf16)(v[c] * inv);
    }
    return;
  }
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

// grid: (rows, ceil(heads / 4)), 4 waves a workgroup
inline void launch_attention_merge(dim3 grid, hipStream_t stream, const float* partial, bf16* out, int nh, int hd, int n_splits,
                                   long ldo) {
#define GIBBS_MERGE(C)                                                                                          \
  do {                                                                                                          \
    if (n_splits <= 4) attention_merge_kernel<C, 4><<<grid, 256, 0, stream>>>(partial, out, nh, hd, n_splits, ldo);      \
    else if (n_splits <= 8) attention_merge_kernel<C, 8><<<grid, 256, 0, stream>>>(partial, out, nh, hd, n_splits, ldo); \
    else attention_merge_kernel<C, 16><<<grid, 256, 0, stream>>>(partial, out, nh, hd, n_splits, ldo);                   \
  } while (0)
  if (hd <= WAVE) GIBBS_MERGE(1);
  else if (hd <= 2 * WAVE) GIBBS_MERGE(2);
  else GIBBS_MERGE(4);
#undef GIBBS_MERGE
}
}  // namespace
