// Paged attention for rows that each attend over a long cache with few queries: decoded tokens
// (and short prompt portions).  bfloat16 cache, float32 scores, maxima, sums and outputs.
//
// The work is bound by reading keys and values once, so it is split to fill the chip: one
// workgroup per (row, kv head [, chunk of the group's query heads], slice of the keys).  All query
// heads that share the kv head are served from the same loads.  Inside a workgroup every LPK
// neighbouring lanes own one key at a time (8 head-dim elements = 16 bytes per lane, so a wave
// reads 1 KB of contiguous cache per instruction) and keep an online-softmax stream of their own
// (max, sum, weighted values); the streams are merged at the end, first across the wave by
// shuffles, then across the 4 waves through LDS.  With more than one slice the workgroup writes a
// partial (max, sum, values) and a second kernel merges the slices.
//
// Visibility is by position only: row n sees keys lo .. pos[n] of its request
// (lo = max(0, pos - window + 1), window 0 = all).
#include "common.h"

namespace {
constexpr int EPL = 8;  // head-dim elements per lane (16 bytes of bfloat16)

struct DecodeArgs {
  const int* pos;
  const int* row_req;
  const int* table;
  int max_pages, page_size, num_pages;
  int nh, nkv, hd;
  long ldq, ldo;
  float scale;
  int window;
  int n_splits;
  int head_chunks;  // workgroups per kv head along the group's query heads
};

__device__ __forceinline__ void unpack8(const uint4& raw, float* f) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// Folds stream b (mb, lb, ab) into stream a.
template <int N>
__device__ __forceinline__ void fold(float& ma, float& la, float* aa, float mb, float lb, const float* ab) {
  const float m = fmaxf(ma, mb);
  const float sa = (ma == -INFINITY) ? 0.f : __expf(ma - m);
  const float sb = (mb == -INFINITY) ? 0.f : __expf(mb - m);
  la = la * sa + lb * sb;
#pragma unroll
  for (int i = 0; i < N; ++i) aa[i] = aa[i] * sa + ab[i] * sb;
  ma = m;
}

template <int LPK, int GT>
__global__ __launch_bounds__(256) void attention_decode_kernel(const bf16* __restrict__ q,
                                                               const bf16* __restrict__ kpages,
                                                               const bf16* __restrict__ vpages,
                                                               float* __restrict__ partial, bf16* __restrict__ out,
                                                               DecodeArgs a) {
  constexpr int KPW = WAVE / LPK;  // keys per wave and iteration
  constexpr int MAX_HD = LPK * EPL;
  __shared__ float s_ml[4][GT][2];
  __shared__ float s_acc[4][GT][MAX_HD];

  const int row = blockIdx.x;
  const int kvh = blockIdx.y / a.head_chunks, hc = blockIdx.y % a.head_chunks;
  const int split = blockIdx.z;
  const int G = a.nh / a.nkv;
  const int g0 = hc * GT;
  const int gcount = min(GT, G - g0);
  const int hd = a.hd;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int grp = lane / LPK, sub = lane % LPK;
  const int e0 = sub * EPL;
  const bool active = e0 < hd;

  const int p = a.pos[row];
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int len = p + 1 - lo;
  int per = (len + a.n_splits - 1) / a.n_splits;
  per = (per + 4 * KPW - 1) / (4 * KPW) * (4 * KPW);
  const int k0 = lo + split * per;
  const int k1 = min(k0 + per, p + 1);
  const int* table = a.table + (size_t)a.row_req[row] * a.max_pages;

  float qf[GT][EPL];
  float m[GT], l[GT], acc[GT][EPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) { acc[g][i] = 0.f; qf[g][i] = 0.f; }
    if (g < gcount && active) {
      const bf16* qp = q + (size_t)row * a.ldq + (size_t)(kvh * G + g0 + g) * hd + e0;
      unpack8(*(const uint4*)qp, qf[g]);
#pragma unroll
      for (int i = 0; i < EPL; ++i) qf[g][i] *= a.scale;
    }
  }

  for (int key = k0 + wave * KPW + grp; key < k1; key += 4 * KPW) {
    int page = table[key / a.page_size];
    page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // never read outside the pool
    const size_t off = (((size_t)page * a.nkv + kvh) * a.page_size + key % a.page_size) * hd + e0;
    float kf[EPL], vf[EPL];
    if (active) {
      unpack8(*(const uint4*)(kpages + off), kf);
      unpack8(*(const uint4*)(vpages + off), vf);
    } else {
#pragma unroll
      for (int i = 0; i < EPL; ++i) kf[i] = vf[i] = 0.f;
    }
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g >= gcount) break;
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < EPL; ++i) d = fmaf(qf[g][i], kf[i], d);
#pragma unroll
      for (int o = 1; o < LPK; o <<= 1) d += __shfl_xor(d, o, WAVE);
      const float m_new = fmaxf(m[g], d);
      const float keep = __expf(m[g] - m_new);  // 0 at the stream's first key
      const float w = __expf(d - m_new);
      l[g] = l[g] * keep + w;
#pragma unroll
      for (int i = 0; i < EPL; ++i) acc[g][i] = fmaf(w, vf[i], acc[g][i] * keep);
      m[g] = m_new;
    }
  }

  // merge the wave's streams (lanes that differ in the bits above LPK hold different keys)
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    if (g >= gcount) break;
#pragma unroll
    for (int o = LPK; o < WAVE; o <<= 1) {
      const float mb = __shfl_xor(m[g], o, WAVE), lb = __shfl_xor(l[g], o, WAVE);
      float ab[EPL];
#pragma unroll
      for (int i = 0; i < EPL; ++i) ab[i] = __shfl_xor(acc[g][i], o, WAVE);
      fold<EPL>(m[g], l[g], acc[g], mb, lb, ab);
    }
    if (grp == 0) {
      if (sub == 0) { s_ml[wave][g][0] = m[g]; s_ml[wave][g][1] = l[g]; }
#pragma unroll
      for (int i = 0; i < EPL; ++i) s_acc[wave][g][e0 + i] = acc[g][i];
    }
  }
  __syncthreads();
  // merge the 4 waves; wave 0's first LPK lanes write the result
  if (wave == 0 && grp == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g >= gcount) break;
      float mm = s_ml[0][g][0], ll = s_ml[0][g][1], aa[EPL];
#pragma unroll
      for (int i = 0; i < EPL; ++i) aa[i] = s_acc[0][g][e0 + i];
      for (int w = 1; w < 4; ++w) {
        float ab[EPL];
#pragma unroll
        for (int i = 0; i < EPL; ++i) ab[i] = s_acc[w][g][e0 + i];
        fold<EPL>(mm, ll, aa, s_ml[w][g][0], s_ml[w][g][1], ab);
      }
      const int head = kvh * G + g0 + g;
      if (a.n_splits == 1) {
        if (active) {
          const float inv = 1.0f / ll;
          bf16* o = out + (size_t)row * a.ldo + (size_t)head * hd + e0;
#pragma unroll
          for (int i = 0; i < EPL; ++i) o[i] = (bf16)(aa[i] * inv);
        }
      } else {
        float* ps = partial + (((size_t)row * a.nh + head) * a.n_splits + split) * (hd + 2);
        if (sub == 0) { ps[0] = mm; ps[1] = ll; }
        if (active) {
#pragma unroll
          for (int i = 0; i < EPL; ++i) ps[2 + e0 + i] = aa[i];
        }
      }
    }
  }
}

// Merges the slices of one (row, head): out = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s.
__global__ void attention_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int nh, int hd,
                                       int n_splits, long ldo) {
  const int row = blockIdx.x, head = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (head >= nh) return;
  const float* ps = partial + ((size_t)row * nh + head) * n_splits * (hd + 2);
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, ps[(size_t)s * (hd + 2)]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = ps[(size_t)s * (hd + 2)];
    if (ms != -INFINITY) L += __expf(ms - M) * ps[(size_t)s * (hd + 2) + 1];
  }
  const float inv = 1.0f / L;
  for (int e = lane; e < hd; e += WAVE) {
    float v = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float ms = ps[(size_t)s * (hd + 2)];
      if (ms != -INFINITY) v += __expf(ms - M) * ps[(size_t)s * (hd + 2) + 2 + e];
    }
    out[(size_t)row * ldo + (size_t)head * hd + e] = (bf16)(v * inv);
  }
}

template <int LPK>
int launch_decode(int gt, dim3 grid, hipStream_t stream, const bf16* q, const bf16* k, const bf16* v, float* partial,
                  bf16* out, const DecodeArgs& a) {
  switch (gt) {
    case 1: attention_decode_kernel<LPK, 1><<<grid, 256, 0, stream>>>(q, k, v, partial, out, a); break;
    case 2: attention_decode_kernel<LPK, 2><<<grid, 256, 0, stream>>>(q, k, v, partial, out, a); break;
    case 4: attention_decode_kernel<LPK, 4><<<grid, 256, 0, stream>>>(q, k, v, partial, out, a); break;
    default: attention_decode_kernel<LPK, 8><<<grid, 256, 0, stream>>>(q, k, v, partial, out, a); break;
  }
  return 0;
}
}  // namespace

// Floats of workspace that n_splits > 1 needs.
GIBBS_EXPORT long gibbs_attention_decode_workspace(int n_rows, int nh, int hd, int n_splits) {
  return n_splits > 1 ? (long)n_rows * nh * n_splits * (hd + 2) : 0;
}

// q: [N, >= nh*hd] bfloat16 (row stride ldq); pages: [num_pages, nkv, page_size, hd] bfloat16;
// out: [N, nh*hd] bfloat16 (row stride ldo); partial: workspace (see above) or null with n_splits 1.
GIBBS_EXPORT int gibbs_attention_decode(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                                        const int* pos, const int* row_req, const int* table, int max_pages,
                                        int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ldq,
                                        long ldo, float scale, int window, int n_splits, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_decode: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_decode: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 8 == 0 && hd <= 256, "attention_decode: head size %d must be a multiple of 8 up to 256", hd);
  GIBBS_REQUIRE(ldq % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_decode: q rows must be 16-byte aligned");
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention_decode: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode: bad cache geometry");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_decode: %d key slices need a workspace", n_splits);
  if (n_rows == 0) return 0;
  const int G = nh / nkv;
  const int gt = G >= 8 ? 8 : (G > 2 ? 4 : G);  // 1, 2, 4 or 8 query heads per workgroup
  const int head_chunks = ceil_div(G, gt);
  GIBBS_REQUIRE((long)nkv * head_chunks <= 65535, "attention_decode: too many heads");
  DecodeArgs a{pos, row_req, table, max_pages, page_size, num_pages, nh, nkv, hd, ldq, ldo, scale, window, n_splits, head_chunks};
  dim3 grid(n_rows, nkv * head_chunks, n_splits);
  const bf16 *qq = (const bf16*)q, *kk = (const bf16*)kpages, *vv = (const bf16*)vpages;
  const int lanes = hd / EPL;  // lanes that hold data; LPK is the next power of two
  if (lanes <= 2) launch_decode<2>(gt, grid, stream, qq, kk, vv, partial, (bf16*)out, a);
  else if (lanes <= 4) launch_decode<4>(gt, grid, stream, qq, kk, vv, partial, (bf16*)out, a);
  else if (lanes <= 8) launch_decode<8>(gt, grid, stream, qq, kk, vv, partial, (bf16*)out, a);
  else if (lanes <= 16) launch_decode<16>(gt, grid, stream, qq, kk, vv, partial, (bf16*)out, a);
  else launch_decode<32>(gt, grid, stream, qq, kk, vv, partial, (bf16*)out, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return gibbs_fail("attention_decode: %s", hipGetErrorString(e));
  if (n_splits > 1) {
    dim3 mgrid(n_rows, ceil_div(nh, 4));
    attention_merge_kernel<<<mgrid, 256, 0, stream>>>(partial, (bf16*)out, nh, hd, n_splits, ldo);
  }
  GIBBS_LAUNCH_STATUS("attention_decode");
}
