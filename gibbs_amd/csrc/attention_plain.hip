// Plain paged attention: the reference twin of the fast kernels, and the kernel of the true
// 32-bit path.  It serves any mix of prompt portions and decoded tokens: every row carries its
// own absolute position and request.
//
//   row n, head h (kv head g = h / (nh / nkv)), position p = pos[n], request r = row_req[n]:
//   visible keys are lo .. p with lo = max(0, p - window + 1) (window 0: all keys);
//   s_k = (q . K[k]) * scale (+ slopes[h] * (k - p) when the position encoding is a linear bias over
//   the distance);  out = sum_k softmax(s)_k V[k], maxima and sums in float32.
// Key k of request r lives in page table[r][k / ps] at slot k % ps; pages are
// [page, kv head, slot in page, hd].  Visibility is by position only; what else a page holds is
// never read.  One wave per (row, head).  Keys are taken in blocks of 64 aligned to absolute key
// index, so the order of operations for a position is the same however the sequence was cut.
#include "common.h"

namespace {
constexpr int MAX_HD = 256;
constexpr int DPL = MAX_HD / WAVE;  // output elements per lane

struct AttnArgs {
  const int* pos;
  const int* row_req;
  const int* table;
  int max_pages, page_size, num_pages;
  int nh, nkv, hd;
  long ldq;  // row stride of q
  long ldo;  // row stride of out
  float scale;
  int window;
  const float* slopes;  // [nh] or null: s_k += slopes[h] * (k - p)
};

template <typename T>
__global__ __launch_bounds__(256) void attention_plain_kernel(const T* __restrict__ q, const T* __restrict__ kpages,
                                                              const T* __restrict__ vpages, T* __restrict__ out,
                                                              AttnArgs a) {
  __shared__ float sq[4][MAX_HD];
  const int n = blockIdx.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int h_raw = blockIdx.y * 4 + wave;
  const bool active = h_raw < a.nh;
  const int h = active ? h_raw : a.nh - 1;
  const int hd = a.hd;
  const int g = h / (a.nh / a.nkv);
  const int p = a.pos[n];
  const int* table = a.table + (size_t)a.row_req[n] * a.max_pages;
  const T* qv = q + (size_t)n * a.ldq + (size_t)h * hd;
  for (int e = lane; e < hd; e += WAVE) sq[wave][e] = to_float(qv[e]);
  __syncthreads();
  if (!active) return;

  const int hi = p;
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[DPL] = {};

  auto row_of = [&](const T* pages, int key) -> const T* {
    int page = table[key / a.page_size];
    page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // never read outside the pool
    return pages + (((size_t)page * a.nkv + g) * a.page_size + key % a.page_size) * hd;
  };

  for (int kb = lo / WAVE * WAVE; kb <= hi; kb += WAVE) {
    const int key = kb + lane;
    const bool valid = key >= lo && key <= hi;
    float s = -INFINITY;
    if (valid) {
      const T* kr = row_of(kpages, key);
      float dot = 0.f;
      for (int e = 0; e < hd; ++e) dot = fmaf(sq[wave][e], to_float(kr[e]), dot);
      s = dot * a.scale;
      if (a.slopes) s += a.slopes[h] * (float)(key - p);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float w = valid ? expf(s - m_new) : 0.f;
    const float keep = expf(m - m_new);  // 0 on the first block (m = -inf)
    l = l * keep + wave_sum(w);
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[i] *= keep;
    const int k_end = min(WAVE, hi - kb + 1);
    for (int kk = max(0, lo - kb); kk < k_end; ++kk) {
      const float wk = __shfl(w, kk, WAVE);
      const T* vr = row_of(vpages, kb + kk);
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int e = lane + i * WAVE;
        if (e < hd) acc[i] = fmaf(wk, to_float(vr[e]), acc[i]);
      }
    }
    m = m_new;
  }
  T* o = out + (size_t)n * a.ldo + (size_t)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int e = lane + i * WAVE;
    if (e < hd) o[e] = from_float<T>(acc[i] * inv);
  }
}
}  // namespace

GIBBS_EXPORT int gibbs_attention_plain(const void* q, const void* kpages, const void* vpages, void* out, int dtype,
                                       const int* pos, const int* row_req, const int* table, int max_pages,
                                       int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ldq,
                                       long ldo, float scale, int window, const float* slopes, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd <= MAX_HD, "attention: head size %d above %d", hd, MAX_HD);
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention: bad cache geometry");
  if (n_rows == 0) return 0;
  AttnArgs a{pos, row_req, table, max_pages, page_size, num_pages, nh, nkv, hd, ldq, ldo, scale, window, slopes};
  dim3 grid(n_rows, ceil_div(nh, 4));
  GIBBS_REQUIRE(grid.y <= 65535, "attention: too many heads (%d)", nh);
  if (dtype == GIBBS_F32)
    attention_plain_kernel<float><<<grid, 256, 0, stream>>>((const float*)q, (const float*)kpages, (const float*)vpages, (float*)out, a);
  else if (dtype == GIBBS_BF16)
    attention_plain_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)q, (const bf16*)kpages, (const bf16*)vpages, (bf16*)out, a);
  else
    return gibbs_fail("attention: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("attention");
}
