// Per-head q/k RMSNorm, rotary position encoding and the write of k, v into cache pages,
// in one pass over the fused projection qkv[N, (nh + 2 nkv) * hd].
//
//   q heads: (RMSNorm with a [hd] gain shared by all heads) -> rotation -> back in place
//   k heads: the same with the k gain -> page[table[req][pos / ps]][kv head][pos % ps]
//   v heads: copied to their page
// The norm comes before the rotation.  Rotation of pair (i0, i1) by angle = float(pos) * inv_freq[j]
// (a float32 product): half-split pairs (j, j + rot/2), interleaved pairs (2j, 2j+1); elements
// beyond rotary_dim pass through.  Sums, the root, angles, sine and cosine are float32.
// Pages are laid out [page, kv head, slot in page, hd].
//
// Cosines and sines come from a table [positions, rot/2] of (cos, sin) that `rope_table` fills once
// (accurate sinf/cosf cost more than everything else here together); positions beyond the table
// are computed in place with the same functions.
//
// Two kernels: the general one (any element type, any even rotary size; one wave per (row, head),
// element by element), and the bfloat16 one for head and rotary sizes in steps of 16 (a lane
// holds 8 elements, 16-byte loads and stores, four heads of a row per lane group).
#include "common.h"
#include "lane8.h"

namespace {
enum { ROPE_HALF_SPLIT = 0, ROPE_INTERLEAVED = 1 };

struct QkRopeArgs {
  const float* q_gain;  // [hd] or null: no q norm
  const float* k_gain;  // [hd] or null: no k norm
  float eps;
  const float* inv_freq;  // [rot / 2] or null: no rotation
  int rot, variant;
  const float2* cs_table;  // [table_len, rot / 2] or null
  int table_len;
  const int* pos;      // [N] absolute position of each row
  const int* row_req;  // [N] batch index of each row's request
  const int* table;    // [n_req, max_pages] page ids of the layer's cache group
  int max_pages, page_size, num_pages;
  int nh, nkv, hd;
  long ld;  // row stride of qkv
};

template <typename T>
__global__ __launch_bounds__(256) void qk_rope_kv_kernel(T* __restrict__ qkv, T* __restrict__ kpages,
                                                         T* __restrict__ vpages, QkRopeArgs a) {
  const int n = blockIdx.x;
  const int hs = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (hs >= a.nh + 2 * a.nkv) return;
  const int hd = a.hd;
  T* src = qkv + (size_t)n * a.ld + (size_t)hs * hd;
  const bool is_q = hs < a.nh, is_k = !is_q && hs < a.nh + a.nkv;
  const int p = a.pos[n];

  T* dst = src;  // q goes back in place
  if (!is_q) {
    if (!kpages) return;  // a layer that reads another layer's cache writes none
    const int r = a.row_req[n];
    const int page = a.table[(size_t)r * a.max_pages + p / a.page_size];
    if (page < 0 || page >= a.num_pages) return;  // the host never asks for this; never write outside
    const int g = is_k ? hs - a.nh : hs - a.nh - a.nkv;
    T* base = is_k ? kpages : vpages;
    dst = base + (((size_t)page * a.nkv + g) * a.page_size + p % a.page_size) * hd;
  }
  if (!is_q && !is_k) {
    for (int e = lane; e < hd; e += WAVE) dst[e] = src[e];
    return;
  }
  const float* gain = is_q ? a.q_gain : a.k_gain;
  float scale = 1.f;
  if (gain) {
    float ss = 0.f;
    for (int e = lane; e < hd; e += WAVE) {
      const float v = to_float(src[e]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    scale = 1.0f / sqrtf(ss / (float)hd + a.eps);
  }
  auto normed = [&](int e) -> float {
    const float v = to_float(src[e]);
    return gain ? v * scale * gain[e] : v;
  };
  const int half = a.inv_freq ? a.rot / 2 : 0;
  // Each lane reads both elements of its pairs before it writes either, so in-place is safe.
  for (int j = lane; j < half; j += WAVE) {
    const int i0 = a.variant == ROPE_HALF_SPLIT ? j : 2 * j;
    const int i1 = a.variant == ROPE_HALF_SPLIT ? j + half : 2 * j + 1;
    const float x0 = normed(i0), x1 = normed(i1);
    float c, s;
    if (a.cs_table && p < a.table_len) {
      const float2 cs = a.cs_table[(size_t)p * half + j];
      c = cs.x;
      s = cs.y;
    } else {
      rope_cos_sin((float)p * a.inv_freq[j], &c, &s);
    }
    dst[i0] = from_float<T>(x0 * c - x1 * s);
    dst[i1] = from_float<T>(x0 * s + x1 * c);
  }
  for (int e = 2 * half + lane; e < hd; e += WAVE) dst[e] = from_float<T>(normed(e));
}

// bfloat16, hd and rot multiples of 16: LPK lanes per (row, HPI consecutive heads), 64 / LPK such items per wave.
// A lane group takes several heads of its row, because what a head needs besides its own 16 bytes per lane (the
// position, the rotation factors, the gains, the page) is the same for all of them and four times as many bytes.
// (2,048 rows of 48 heads of 64: 16.0 -> 15.4 us, most of it from the 32-bit item numbers; without its stores and
// rotation factors the kernel still takes 11.7 us, a chain of loads that each hang on the one before.)
template <int LPK, int HPI>
__global__ __launch_bounds__(256) void qk_rope_kv_bf16x8_kernel(bf16* __restrict__ qkv, bf16* __restrict__ kpages,
                                                                bf16* __restrict__ vpages, QkRopeArgs a, int n_rows) {
  constexpr int IPW = WAVE / LPK;  // items per wave
  const int slots = a.nh + 2 * a.nkv;
  const int chunks = (slots + HPI - 1) / HPI;
  const int lane = threadIdx.x % WAVE;
  const int sub = lane % LPK, e0 = sub * EPL;
  // (32-bit item numbers: the launcher refuses more; a 64-bit division is a hundred instructions in front of the first load)
  const unsigned item = (blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE) * IPW + lane / LPK;
  const bool item_ok = item < (unsigned)n_rows * (unsigned)chunks;
  const int n = item_ok ? (int)(item / (unsigned)chunks) : 0;
  const int hs0 = item_ok ? (int)(item % (unsigned)chunks) * HPI : 0;
  const int hd = a.hd;
  const bool active = item_ok && e0 < hd;
  const int p = a.pos[n];
  bf16* row = qkv + (size_t)n * a.ld + e0;
  uint4 raw[HPI];
#pragma unroll
  for (int i = 0; i < HPI; ++i)
    raw[i] = (active && hs0 + i < slots) ? *(const uint4*)(row + (size_t)(hs0 + i) * hd) : make_uint4(0, 0, 0, 0);
  // the page of the row's position, if a head of this item goes there
  int page = -1;
  if (kpages && active && hs0 + HPI > a.nh) {
    page = a.table[(size_t)a.row_req[n] * a.max_pages + p / a.page_size];
    if (page >= a.num_pages) page = -1;  // the host never asks for another; never write outside
  }
  const Rot8 rt = rotation8(e0, a.inv_freq, a.rot, a.variant, p, a.cs_table, a.table_len);
  float q_gain8[EPL], k_gain8[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    q_gain8[i] = (a.q_gain && active) ? a.q_gain[e0 + i] : 1.f;
    k_gain8[i] = (a.k_gain && active) ? a.k_gain[e0 + i] : 1.f;
  }
#pragma unroll
  for (int i = 0; i < HPI; ++i) {
    const int hs = hs0 + i;
    if (!item_ok || hs >= slots) break;   // (whole lane groups leave: the sums below stay within a group)
    const bool is_q = hs < a.nh, is_k = !is_q && hs < a.nh + a.nkv;
    uint4 result = raw[i];                // value heads are copied
    if (is_q || is_k) {
      float v[EPL], gain8[EPL];
      unpack8(raw[i], v);
#pragma unroll
      for (int j = 0; j < EPL; ++j) gain8[j] = is_q ? q_gain8[j] : k_gain8[j];
      norm_rope8_with<LPK>(v, e0, hd, (is_q ? a.q_gain : a.k_gain) != nullptr, gain8, a.eps, a.inv_freq != nullptr, rt, a.rot,
                           a.variant, lane);
      result = pack8(v);
    }
    if (!active) continue;
    if (is_q) {
      *(uint4*)(row + (size_t)hs * hd) = result;
    } else if (page >= 0) {
      const int g = is_k ? hs - a.nh : hs - a.nh - a.nkv;
      bf16* dst = (is_k ? kpages : vpages) + (((size_t)page * a.nkv + g) * a.page_size + p % a.page_size) * hd + e0;
      *(uint4*)dst = result;
    }
  }
}

// (cos, sin) of float(pos) * inv_freq[j] for pos < n_pos, j < half.
__global__ __launch_bounds__(256) void rope_table_kernel(float2* __restrict__ table, const float* __restrict__ inv_freq,
                                                         int half, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int pos = (int)(i / half), j = (int)(i % half);
  float c, s;
  rope_cos_sin((float)pos * inv_freq[j], &c, &s);
  table[i] = make_float2(c, s);
}
}  // namespace

GIBBS_EXPORT int gibbs_rope_table(float* table, const float* inv_freq, int half, int n_pos, hipStream_t stream) {
  GIBBS_REQUIRE(half > 0 && n_pos > 0, "rope_table: bad sizes half=%d positions=%d", half, n_pos);
  const long total = (long)half * n_pos;
  rope_table_kernel<<<ceil_div(total, 256), 256, 0, stream>>>((float2*)table, inv_freq, half, total);
  GIBBS_LAUNCH_STATUS("rope_table");
}

GIBBS_EXPORT int gibbs_qk_rope_kv(void* qkv, void* kpages, void* vpages, int dtype, const float* q_gain,
                                  const float* k_gain, float eps, const float* inv_freq, int rot, int variant,
                                  const float* cs_table, int table_len, const int* pos, const int* row_req, const int* table, int max_pages,
                                  int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ld,
                                  hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv >= 0 && hd > 0, "qk_rope_kv: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(ld >= (long)(nh + 2 * nkv) * hd, "qk_rope_kv: row stride %ld shorter than (nh + 2 nkv) * hd", ld);
  GIBBS_REQUIRE(!inv_freq || (rot > 0 && rot % 2 == 0 && rot <= hd), "qk_rope_kv: rotary_dim %d must be even and <= head size %d", rot, hd);
  GIBBS_REQUIRE(variant == ROPE_HALF_SPLIT || variant == ROPE_INTERLEAVED, "qk_rope_kv: unknown rotation variant %d", variant);
  GIBBS_REQUIRE(!kpages || (vpages && table && page_size > 0 && max_pages > 0 && num_pages > 0), "qk_rope_kv: cache pages without a block table");
  if (n_rows == 0) return 0;
  QkRopeArgs a{q_gain, k_gain, eps, inv_freq, rot, variant, (const float2*)cs_table, cs_table ? table_len : 0, pos, row_req, table, max_pages, page_size, num_pages, nh, nkv, hd, ld};
  const int slots = nh + 2 * nkv;
  dim3 grid(n_rows, ceil_div(slots, 4));
  GIBBS_REQUIRE(grid.y <= 65535, "qk_rope_kv: too many heads (%d)", slots);
  const bool lanes8 = dtype == GIBBS_BF16 && hd % 16 == 0 && hd <= 256 && (!inv_freq || rot % 16 == 0) && ld % 8 == 0 &&
                      ((uintptr_t)qkv % 16) == 0;
  if (lanes8) {
    const int lanes = hd / EPL;
    const long items = (long)n_rows * ceil_div(slots, 4);   // a lane group takes four consecutive heads of a row
    GIBBS_REQUIRE(items < (1l << 31) - 64, "qk_rope_kv: %d rows of %d heads are more than the kernel numbers", n_rows, slots);
#define GIBBS_ROPE8(LPK)                                                                                   \
  qk_rope_kv_bf16x8_kernel<LPK, 4><<<ceil_div(items, 4 * (WAVE / LPK)), 256, 0, stream>>>((bf16*)qkv, (bf16*)kpages, \
                                                                                           (bf16*)vpages, a, n_rows)
    if (lanes <= 2) GIBBS_ROPE8(2);
    else if (lanes <= 4) GIBBS_ROPE8(4);
    else if (lanes <= 8) GIBBS_ROPE8(8);
    else if (lanes <= 16) GIBBS_ROPE8(16);
    else GIBBS_ROPE8(32);
#undef GIBBS_ROPE8
  } else if (dtype == GIBBS_F32)
    qk_rope_kv_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, (float*)kpages, (float*)vpages, a);
  else if (dtype == GIBBS_BF16)
    qk_rope_kv_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)qkv, (bf16*)kpages, (bf16*)vpages, a);
  else
    return gibbs_fail("qk_rope_kv: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("qk_rope_kv");
}
