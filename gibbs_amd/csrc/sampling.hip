// Sampling on the device from float32 logits [M, V], one workgroup per row.
//
// Greedy: the index of the first largest value; NaN never wins; 0 if nothing is above -inf.
// Sampled: candidates are the top k (<= 64) by (logit descending, id ascending); p_i =
// softmax(logit_i / T) over the candidates; the shortest prefix whose cumulative p reaches
// clamp(top_p, 0.01, 1) is kept; the draw r = u * sum(kept) picks the first candidate whose
// cumulative p reaches r.  u in [0, 1) comes from the host's counter-based generator, so a
// fixed seed reproduces the tokens.  Softmax and sums are float32.
#include "common.h"

namespace {
constexpr int MAX_K = 64;
constexpr int THREADS = 1024;

// Order of candidates: larger value first, then smaller index.  NaN ranks below everything.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  return v > bv || (v == bv && i < bi);
}

// Best (value, index) over the block under `better`; all threads get it.
__device__ __forceinline__ void block_best(float& v, int& i, float* sv, int* si) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, WAVE);
    const int oi = __shfl_xor(i, o, WAVE);
    if (better(ov, oi, v, i)) { v = ov; i = oi; }
  }
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  __syncthreads();
  if (lane == 0) { sv[wave] = v; si[wave] = i; }
  __syncthreads();
  v = sv[0]; i = si[0];
  for (int w = 1; w < THREADS / WAVE; ++w)
    if (better(sv[w], si[w], v, i)) { v = sv[w]; i = si[w]; }
}

__global__ __launch_bounds__(THREADS) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V,
                                                         long ld) {
  __shared__ float sv[THREADS / WAVE];
  __shared__ int si[THREADS / WAVE];
  const float* row = logits + (size_t)blockIdx.x * ld;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  // 16-byte loads over the aligned middle; NaN fails both comparisons in `better`
  const int head = min(V, (int)(((16 - ((uintptr_t)row & 15)) & 15) / 4));
  const int n4 = (V - head) / 4;
  for (int i = threadIdx.x; i < head; i += THREADS)
    if (better(row[i], i, bv, bi)) { bv = row[i]; bi = i; }
  const float4* row4 = (const float4*)(row + head);
  for (int j = threadIdx.x; j < n4; j += THREADS) {
    const float4 v = row4[j];
    const int i = head + 4 * j;
    if (better(v.x, i, bv, bi)) { bv = v.x; bi = i; }
    if (better(v.y, i + 1, bv, bi)) { bv = v.y; bi = i + 1; }
    if (better(v.z, i + 2, bv, bi)) { bv = v.z; bi = i + 2; }
    if (better(v.w, i + 3, bv, bi)) { bv = v.w; bi = i + 3; }
  }
  for (int i = head + 4 * n4 + threadIdx.x; i < V; i += THREADS)
    if (better(row[i], i, bv, bi)) { bv = row[i]; bi = i; }
  block_best(bv, bi, sv, si);
  if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

__global__ __launch_bounds__(THREADS) void sample_kernel(const float* __restrict__ logits, int* __restrict__ out, int V,
                                                         long ld, const float* __restrict__ temperature,
                                                         const float* __restrict__ top_p, const int* __restrict__ top_k,
                                                         const float* __restrict__ u) {
  __shared__ float sv[THREADS / WAVE];
  __shared__ int si[THREADS / WAVE];
  __shared__ float cand_v[MAX_K];
  __shared__ int cand_i[MAX_K];
  const int m = blockIdx.x;
  const float* row = logits + (size_t)m * ld;
  const float T = temperature[m];
  const bool greedy = T <= 1e-4f;
  int k = greedy ? 1 : top_k[m];
  k = k < 1 ? 1 : (k > MAX_K ? MAX_K : k);
  if (k > V) k = V;
  // Round c finds the best element strictly after the previous pick in candidate order.
  float pv = INFINITY;
  int pi = -1;
  int found = 0;
  for (int c = 0; c < k; ++c) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += THREADS) {
      const float v = row[i];
      const bool after = v < pv || (v == pv && i > pi);
      if (after && better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    block_best(bv, bi, sv, si);
    if (bi == 0x7fffffff) break;  // fewer than k finite candidates
    if (threadIdx.x == 0) { cand_v[c] = bv; cand_i[c] = bi; }
    pv = bv; pi = bi; found = c + 1;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  if (found == 0) { out[m] = 0; return; }
  if (greedy) { out[m] = cand_i[0]; return; }
  float probs[MAX_K];
  const float mx = cand_v[0] / T;
  float sum = 0.f;
  for (int c = 0; c < found; ++c) { probs[c] = expf(cand_v[c] / T - mx); sum += probs[c]; }
  const float denom = fmaxf(sum, 1e-12f);
  const float thresh = fminf(fmaxf(top_p[m], 0.01f), 1.0f);
  float cum = 0.f;
  int cut = found;
  for (int c = 0; c < found; ++c) {
    probs[c] /= denom;
    cum += probs[c];
    if (cum >= thresh) { cut = c + 1; break; }
  }
  float kept = 0.f;
  for (int c = 0; c < cut; ++c) kept += probs[c];
  const float r = u[m] * kept;
  cum = 0.f;
  int pick = cand_i[cut - 1];
  for (int c = 0; c < cut; ++c) {
    cum += probs[c];
    if (cum >= r) { pick = cand_i[c]; break; }
  }
  out[m] = pick;
}
}  // namespace

GIBBS_EXPORT int gibbs_argmax(const float* logits, int* out, int M, int V, long ld, hipStream_t stream) {
  GIBBS_REQUIRE(M >= 0 && V > 0 && ld >= V, "argmax: bad sizes M=%d V=%d ld=%ld", M, V, ld);
  if (M == 0) return 0;
  argmax_kernel<<<M, THREADS, 0, stream>>>(logits, out, V, ld);
  GIBBS_LAUNCH_STATUS("argmax");
}

// temperature, top_p, top_k, u: one value per row, on the device.
GIBBS_EXPORT int gibbs_sample(const float* logits, int* out, int M, int V, long ld, const float* temperature,
                              const float* top_p, const int* top_k, const float* u, hipStream_t stream) {
  GIBBS_REQUIRE(M >= 0 && V > 0 && ld >= V, "sample: bad sizes M=%d V=%d ld=%ld", M, V, ld);
  if (M == 0) return 0;
  sample_kernel<<<M, THREADS, 0, stream>>>(logits, out, V, ld, temperature, top_p, top_k, u);
  GIBBS_LAUNCH_STATUS("sample");
}
