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

// Calls fn(value, index) for the elements of a row that fall to this thread: 16-byte loads over the
// aligned middle of the row, single elements before and after it.  AHEAD: loads in flight per thread (a
// workgroup that walks a row alone, on the step's critical path, wants the whole row asked for at once).
template <int AHEAD = 4, typename F>
__device__ __forceinline__ void walk_row(const float* row, int V, F fn) {
  const int head = min(V, (int)(((16 - ((uintptr_t)row & 15)) & 15) / 4));
  const int n4 = (V - head) / 4;
  for (int i = threadIdx.x; i < head; i += THREADS) fn(row[i], i);
  const float4* row4 = (const float4*)(row + head);
  for (int j0 = threadIdx.x; j0 < n4; j0 += AHEAD * THREADS) {
    float4 v[AHEAD];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a)
      if (j0 + a * THREADS < n4) v[a] = row4[j0 + a * THREADS];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      const int j = j0 + a * THREADS;
      if (j >= n4) break;
      const int i = head + 4 * j;
      fn(v[a].x, i);
      fn(v[a].y, i + 1);
      fn(v[a].z, i + 2);
      fn(v[a].w, i + 3);
    }
  }
  for (int i = head + 4 * n4 + threadIdx.x; i < V; i += THREADS) fn(row[i], i);
}

__global__ __launch_bounds__(THREADS) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V,
                                                         long ld) {
  __shared__ float sv[THREADS / WAVE];
  __shared__ int si[THREADS / WAVE];
  const float* row = logits + (size_t)blockIdx.x * ld;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  // NaN fails both comparisons in `better`
  walk_row(row, V, [&](float v, int i) {
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  });
  block_best(bv, bi, sv, si);
  if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

// ---------------------------------------------------------------------------------------------- sampling
// A candidate as one number: larger is better.  High half: the value's bits made monotone (negative
// values flipped; -0 counted as +0, as the comparison of values does); low half: ~index, so that of
// equal values the smaller index wins.  0 stands for "none" (no value maps to it; NaN is never a
// candidate).
typedef unsigned long long key64;
constexpr int MAX_LIST = 2048;   // candidates above the threshold that are sorted exactly

__device__ __forceinline__ unsigned ordered_bits(float v) {
  const unsigned b = __float_as_uint(v == 0.f ? 0.f : v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ key64 make_key(float v, int i) {
  return v != v ? 0ull : ((key64)ordered_bits(v) << 32) | (key64)(0xffffffffu - (unsigned)i);
}
__device__ __forceinline__ float key_value(key64 k) {
  const unsigned o = (unsigned)(k >> 32);
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}
__device__ __forceinline__ int key_index(key64 k) { return (int)(0xffffffffu - (unsigned)k); }
// Lane c's value, for a c that is the same in every lane (a scalar read, not a trip through LDS).
__device__ __forceinline__ float lane_value(float v, int c) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), c));
}

// The k best candidates, one after the other: every round walks the whole row.  The way out when too
// many values tie at the threshold for the list below (a row of equal logits).
__device__ int top_k_by_rounds(const float* row, int V, int k, float* cand_v, int* cand_i, float* sv, int* si) {
  float pv = INFINITY;
  int pi = -1, found = 0;
  for (int c = 0; c < k; ++c) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += THREADS) {
      const float v = row[i];
      const bool after = v < pv || (v == pv && i > pi);
      if (after && better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    block_best(bv, bi, sv, si);
    if (bi == 0x7fffffff) break;  // fewer than k candidates
    if (threadIdx.x == 0) { cand_v[c] = bv; cand_i[c] = bi; }
    pv = bv; pi = bi; found = c + 1;
  }
  __syncthreads();
  return found;
}

// Two walks over the row instead of k.  First walk: every thread keeps the best of its elements.  The
// ceil(k / 16)-th best of those in every wave, and the smallest of these over the 16 waves, is a value
// that at least k elements of the row reach: a threshold at or below the k-th best value.  Second walk: the
// elements that reach it (a few hundred for logits of a model) go to a list, which is ranked exactly.
__global__ __launch_bounds__(THREADS) void sample_kernel(const float* __restrict__ logits, int* __restrict__ out, int V,
                                                         long ld, const float* __restrict__ temperature,
                                                         const float* __restrict__ top_p, const int* __restrict__ top_k,
                                                         const float* __restrict__ u) {
  constexpr int WAVES = THREADS / WAVE;
  __shared__ float sv[WAVES];
  __shared__ int si[WAVES];
  __shared__ float cand_v[MAX_K];
  __shared__ int cand_i[MAX_K];
  __shared__ unsigned wave_low[WAVES];
  __shared__ key64 list[MAX_LIST];
  __shared__ int s_count, s_valid;
  const int m = blockIdx.x;
  const float* row = logits + (size_t)m * ld;
  const float T = temperature[m];
  const bool greedy = T <= 1e-4f;
  int k = greedy ? 1 : top_k[m];
  k = k < 1 ? 1 : (k > MAX_K ? MAX_K : k);
  if (k > V) k = V;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  if (threadIdx.x == 0) { s_count = 0; s_valid = 0; }

  // first walk
  unsigned mine = 0;         // the largest value of this thread's elements, as ordered bits (0: none)
  int valid = 0;
  walk_row(row, V, [&](float v, int i) {
    const unsigned o = v != v ? 0u : ordered_bits(v);
    valid += o != 0;
    mine = max(mine, o);
  });
  // the ceil(k / 16)-th largest of the wave's threads, counting equal ones once (0: it has fewer): at
  // least that many threads of the wave hold an element that reaches it
  const int per_wave = (k + WAVES - 1) / WAVES;
  unsigned rest = mine, nth = 0;
  for (int c = 0; c < per_wave; ++c) {
    nth = rest;
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) nth = max(nth, (unsigned)__shfl_xor((int)nth, o, WAVE));
    if (rest == nth) rest = 0;
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) valid += __shfl_xor(valid, o, WAVE);
  __syncthreads();
  if (lane == 0) {
    wave_low[wave] = nth;
    atomicAdd(&s_valid, valid);
  }
  __syncthreads();
  unsigned threshold = wave_low[0];                       // 0: every candidate passes
  for (int w = 1; w < WAVES; ++w) threshold = min(threshold, wave_low[w]);
  const int n_valid = s_valid;
  int found = k < n_valid ? k : n_valid;
  if (found == 0) {
    if (threadIdx.x == 0) out[m] = 0;
    return;
  }

  // second walk: everything at or above the threshold
  walk_row(row, V, [&](float v, int i) {
    if (v == v && ordered_bits(v) >= threshold) {
      const int at = atomicAdd(&s_count, 1);
      if (at < MAX_LIST) list[at] = make_key(v, i);
    }
  });
  __syncthreads();
  const int n = s_count;
  if (n > MAX_LIST) {
    found = top_k_by_rounds(row, V, k, cand_v, cand_i, sv, si);
  } else {
    // rank of every listed candidate = how many are better; keys differ, so ranks do
    for (int j = threadIdx.x; j < n; j += THREADS) {
      const key64 key = list[j];
      int rank = 0;
      for (int o = 0; o < n; ++o) rank += list[o] > key;
      if (rank < found) {
        cand_v[rank] = key_value(key);
        cand_i[rank] = key_index(key);
      }
    }
    __syncthreads();
  }
  // The draw, by the first wave: lane c holds candidate c; the sums run over the candidates one after
  // the other (values passed from lane to lane), in the order a serial loop would add them.
  if (wave != 0) return;
  if (found == 0) {
    if (lane == 0) out[m] = 0;
    return;
  }
  if (greedy) {
    if (lane == 0) out[m] = cand_i[0];
    return;
  }
  const float mx = cand_v[0] / T;
  const float e = lane < found ? expf(cand_v[lane] / T - mx) : 0.f;
  float sum = 0.f;
  for (int c = 0; c < found; ++c) sum += lane_value(e, c);
  const float p = e / fmaxf(sum, 1e-12f);
  const float thresh = fminf(fmaxf(top_p[m], 0.01f), 1.0f);
  float cum = 0.f;
  int cut = found;
  for (int c = 0; c < found; ++c) {
    cum += lane_value(p, c);
    if (cum >= thresh) { cut = c + 1; break; }
  }
  float kept = 0.f;
  for (int c = 0; c < cut; ++c) kept += lane_value(p, c);
  const float r = u[m] * kept;
  cum = 0.f;
  int pick = cut - 1;
  for (int c = 0; c < cut; ++c) {
    cum += lane_value(p, c);
    if (cum >= r) { pick = c; break; }
  }
  if (lane == 0) out[m] = cand_i[pick];
}
}  // namespace

// Repetition penalty of the reference's sampler, applied to the logits in place before a row is
// sampled.  A token that occurs c times among the row's recent tokens (the reference passes the last
// 64 of prompt and output): greedy rows (src/runtime/lm.rs:1089-1105): c times
// v = v > 0 ? v / penalty : v * penalty, then v -= 1.5 c; sampled rows (:1176-1189): c times
// v = (v > 0 ? v / penalty : v * penalty) - 1.5.  Rows whose penalty is <= 1 are left alone (:1072,
// :1163).  One workgroup of R threads per row; the first thread that holds a token does its update.
__global__ void repetition_penalty_kernel(float* __restrict__ logits, long ld, int V, const int* __restrict__ recent,
                                          int R, const float* __restrict__ penalty,
                                          const float* __restrict__ temperature) {
  extern __shared__ int s_recent[];
  const int m = blockIdx.x, j = threadIdx.x;
  const float p = penalty[m];
  if (!(p > 1.0f)) return;
  const int t = recent[(size_t)m * R + j];
  s_recent[j] = t;
  __syncthreads();
  if (t < 0 || t >= V) return;
  int count = 0;
  for (int i = 0; i < R; ++i) {
    if (s_recent[i] == t) {
      if (i < j) return;          // an earlier thread holds this token
      count += 1;
    }
  }
  float v = logits[(size_t)m * ld + t];
  if (temperature[m] <= 1e-4f) {
    for (int c = 0; c < count; ++c) v = v > 0.f ? v / p : v * p;
    v -= 1.5f * (float)count;
  } else {
    for (int c = 0; c < count; ++c) v = (v > 0.f ? v / p : v * p) - 1.5f;
  }
  logits[(size_t)m * ld + t] = v;
}

// recent: [M, R] token ids (negative: none), R <= 1024; penalty, temperature: [M].
GIBBS_EXPORT int gibbs_repetition_penalty(float* logits, int M, int V, long ld, const int* recent, int R,
                                          const float* penalty, const float* temperature, hipStream_t stream) {
  GIBBS_REQUIRE(M >= 0 && V > 0 && ld >= V, "repetition_penalty: bad sizes M=%d V=%d ld=%ld", M, V, ld);
  GIBBS_REQUIRE(R >= 1 && R <= 1024, "repetition_penalty: %d recent tokens a row outside 1..1024", R);
  if (M == 0) return 0;
  repetition_penalty_kernel<<<M, R, R * sizeof(int), stream>>>(logits, ld, V, recent, R, penalty, temperature);
  GIBBS_LAUNCH_STATUS("repetition_penalty");
}

// The end of a decode step that runs as a captured graph, in one kernel (one workgroup per row): the row's
// next token (the first largest logit; or, with logits null, the token that a sampling kernel has put
// into ids already) is logged, the row's position and cached length move on by one, its next draw is
// loaded, and the token's embedding is written as the row of the next step's residual stream (and of its
// bfloat16 mirror), so that the next step starts at its first layer.
//   log[steps[i] * n + i] = ids[i];  pos[i] += 1;  ctx[i] += 1;  u[i] = u_all[(steps[i] + 1) * n + i];  steps[i] += 1
// A row with live[i] == 0 stands for no request (the padding of a loop made for more rows than are live):
// nothing of it is logged or moves on; it only gets the embedding of the token it holds again, so that its
// residual row, which the step updated in place, starts the next step from the same finite values.
template <typename T>
__global__ __launch_bounds__(THREADS) void decode_tail_kernel(const float* __restrict__ logits, int V, long ld,
                                                              int* __restrict__ ids, int* __restrict__ pos, int* __restrict__ ctx,
                                                              int* __restrict__ log, int* __restrict__ steps, int n, int capacity,
                                                              float* __restrict__ u, const float* __restrict__ u_all,
                                                              const T* __restrict__ table, int vocab, int hidden,
                                                              float* __restrict__ x, bf16* __restrict__ mirror,
                                                              const int* __restrict__ live) {
  __shared__ float sv[THREADS / WAVE];
  __shared__ int si[THREADS / WAVE];
  __shared__ int s_token;
  const int i = blockIdx.x;
  const bool padding = live && live[i] == 0;
  int token = 0;
  if (logits && !padding) {
    const float* row = logits + (size_t)i * ld;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    walk_row<16>(row, V, [&](float v, int j) {
      if (better(v, j, bv, bi)) { bv = v; bi = j; }
    });
    block_best(bv, bi, sv, si);
    token = (bi == 0x7fffffff) ? 0 : bi;
  }
  if (threadIdx.x == 0) {
    if (logits && !padding) ids[i] = token;
    else token = ids[i];
    if (!padding) {
      const int step = steps[i];
      if (step < capacity) log[(size_t)step * n + i] = token;
      pos[i] += 1;
      ctx[i] += 1;
      if (u && step + 1 < capacity) u[i] = u_all[(size_t)(step + 1) * n + i];
      steps[i] = step + 1;
    }
    s_token = token;
  }
  if (!x) return;
  __syncthreads();
  token = s_token;
  token = token < 0 ? 0 : (token >= vocab ? vocab - 1 : token);   // never read outside the table
  const T* src = table + (size_t)token * hidden;
  for (int e = threadIdx.x; e < hidden; e += THREADS) {
    const float v = to_float(src[e]);
    x[(size_t)i * hidden + e] = v;
    if (mirror) mirror[(size_t)i * hidden + e] = (bf16)v;
  }
}

// logits: [n, V] float32 (row stride ld) or null (ids hold the tokens); steps: [n] steps done per row; u, u_all:
// draws (or null); table: [vocab, hidden] in table_dtype; x: [n, hidden] float32 and mirror: [n, hidden]
// bfloat16 for the next step (or null: no embedding); live: [n], 0 for rows that stand for no request (or null: all do).
GIBBS_EXPORT int gibbs_decode_tail(const float* logits, int V, long ld, int* ids, int* pos, int* ctx, int* log, int* steps,
                                   int n, int capacity, float* u, const float* u_all, const void* table, int table_dtype,
                                   int vocab, int hidden, float* x, void* mirror, const int* live, hipStream_t stream) {
  GIBBS_REQUIRE(n > 0 && capacity > 0, "decode_tail: batch %d, log of %d steps", n, capacity);
  GIBBS_REQUIRE(!logits || (V > 0 && ld >= V), "decode_tail: bad logits V=%d ld=%ld", V, ld);
  GIBBS_REQUIRE(!x || (table && hidden > 0 && vocab > 0), "decode_tail: an embedding needs the token table");
  GIBBS_REQUIRE(!u || u_all, "decode_tail: draws without their table");
  if (table_dtype == GIBBS_F32)
    decode_tail_kernel<float><<<n, THREADS, 0, stream>>>(logits, V, ld, ids, pos, ctx, log, steps, n, capacity, u, u_all,
                                                         (const float*)table, vocab, hidden, x, (bf16*)mirror, live);
  else if (table_dtype == GIBBS_BF16)
    decode_tail_kernel<bf16><<<n, THREADS, 0, stream>>>(logits, V, ld, ids, pos, ctx, log, steps, n, capacity, u, u_all,
                                                        (const bf16*)table, vocab, hidden, x, (bf16*)mirror, live);
  else
    return gibbs_fail("decode_tail: unknown table dtype %d", table_dtype);
  GIBBS_LAUNCH_STATUS("decode_tail");
}

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
