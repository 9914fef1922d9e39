// Paged attention for rows that each attend over a long cache with few queries: decoded tokens
// (and short prompt portions).  bfloat16 cache, float32 scores, maxima, sums and outputs.
//
// The work is reading keys and values once, so it is split to fill the chip: one workgroup of 4 or
// 8 waves per (row, kv head [, chunk of the group's query heads], slice of the keys).  All query
// heads that share the kv head are served from the same loads.  Inside a workgroup every LPK
// neighbouring lanes own one key at a time (8 head-dim elements = 16 bytes per lane, so a wave
// reads 1 KB of contiguous cache per instruction) and keep an online-softmax stream of their own
// (max, sum, weighted values); the streams are merged at the end, first across the wave by
// shuffles, then across the waves through LDS (wave g folds head g).  With more than one slice the workgroup writes a
// partial (max, sum, values) and a second kernel merges the slices.  The slice's page ids are
// staged in LDS, and the loads of the next two keys are in flight while a key is worked on.
//
// Two entry points share the kernel.  `attention_decode` takes q as it is (already normed and
// rotated; the row's key and value already in their pages).  `attention_decode_fused` takes a step
// of decoded tokens as the raw fused projection qkv[N, (nh + 2 nkv) hd]: the kernel norms and
// rotates q on the fly (every slice's workgroup does, it is a few hundred operations), norms and
// rotates the row's own new key, writes it and the new value to their page (the workgroup of head
// chunk 0 whose key slice holds the row's position does) and uses them from LDS instead of
// reading them back.
//
// The slices are merged by a separate kernel: letting the last workgroup to arrive merge them in
// place needs device-scope fences, and on this chip (one L2 per XCD) each such fence writes back
// and invalidates an L2, which cost 130 us a call when it was tried.
//
// Visibility is by position only: row n sees keys lo .. pos[n] of its request
// (lo = max(0, pos - window + 1), window 0 = all).
#include "common.h"
#include "lane8.h"

namespace {
constexpr int SEG_PAGES = 512;  // page ids of a key slice kept in LDS at a time

struct DecodeArgs {
  const int* pos;
  const int* row_req;
  const int* table;
  int max_pages, page_size, num_pages;
  int page_shift;  // log2(page_size) if it is a power of two, else -1
  int nh, nkv, hd;
  long ldq, ldo;   // row strides of q (or of the raw qkv rows) and of the output
  float scale;
  int window;
  int n_splits;
  int head_chunks;  // workgroups per kv head along the group's query heads
  // raw rows only: what to do to q and to the new key before they are used
  const float* q_gain;    // [hd] or null
  const float* k_gain;    // [hd] or null
  float eps;
  const float* inv_freq;  // [rot/2] or null
  int rot, variant;       // 0 half split, 1 interleaved
  const float2* cs_table; // [table_len, rot/2] (cos, sin) of the first positions, or null
  int table_len;
};

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

template <int LPK, int GT, bool RAW, int NW>
__global__ __launch_bounds__(NW * WAVE, GT <= 4 ? (NW == 8 ? 4 : 3) : 2) void attention_decode_kernel(const bf16* __restrict__ qkv, bf16* __restrict__ kpages,
                                                               bf16* __restrict__ vpages, float* __restrict__ partial,
                                                               bf16* __restrict__ out, DecodeArgs a) {
  constexpr int KPW = WAVE / LPK;
  constexpr int MAX_HD = LPK * EPL;
  __shared__ float s_ml[NW][GT][2];
  __shared__ float s_acc[NW][GT][MAX_HD];
  __shared__ float s_knew[MAX_HD], s_vnew[MAX_HD];
  __shared__ float s_q[GT][MAX_HD];
  __shared__ int s_pages[SEG_PAGES];

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
  per = (per + NW * KPW - 1) / (NW * KPW) * (NW * KPW);
  const int k0 = lo + split * per;
  const int k1 = min(k0 + per, p + 1);
  const int* table = a.table + (size_t)a.row_req[row] * a.max_pages;
  const bf16* qrow = qkv + (size_t)row * a.ldq;

  // Everything that does not hang on earlier arithmetic is asked for first: the query heads, the
  // row's own key and value, the page ids of the slice's first segment (kept in registers until
  // the prologue below is through, then put into LDS).
  // (query head g is prepared by wave g % NW alone and handed to the others through LDS)
  uint4 qraw[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g)
    qraw[g] = (g < gcount && g % NW == wave && active) ? *(const uint4*)(qrow + (size_t)(kvh * G + g0 + g) * hd + e0)
                                                       : make_uint4(0, 0, 0, 0);
  const bool has_new = RAW && p >= k0 && p < k1;  // raw rows: this slice holds the row's own position
  const bool new_lane = has_new && wave == NW - 1 && grp == 0;  // the last wave has the fewest query heads to prepare
  uint4 knew_raw = make_uint4(0, 0, 0, 0), vnew_raw = make_uint4(0, 0, 0, 0);
  if (new_lane && active) {
    knew_raw = *(const uint4*)(qrow + (size_t)(a.nh + kvh) * hd + e0);
    vnew_raw = *(const uint4*)(qrow + (size_t)(a.nh + a.nkv + kvh) * hd + e0);
  }
  constexpr int PRE = (SEG_PAGES + NW * WAVE - 1) / (NW * WAVE);
  const int first_page0 = a.page_shift >= 0 ? k0 >> a.page_shift : k0 / a.page_size;
  const int seg1_0 = min(k1, (first_page0 + SEG_PAGES) * a.page_size);
  int pre_page[PRE];
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    const int j = threadIdx.x + i * NW * WAVE;
    pre_page[i] = (j < SEG_PAGES && (first_page0 + j) * a.page_size < seg1_0) ? table[first_page0 + j] : 0;
  }

  Rot8 rt;
  if (RAW) rt = rotation8(e0, a.inv_freq, a.rot, a.variant, p, a.cs_table, a.table_len);
  const bool rotate = a.inv_freq != nullptr;
  // raw rows: the row's own key and value; the last wave's first LPK lanes prepare them for everyone
  if (new_lane) {
    float kf[EPL], vf[EPL];
    unpack8(knew_raw, kf);
    unpack8(vnew_raw, vf);
    norm_rope8<LPK>(kf, e0, hd, a.k_gain, a.eps, rotate, rt, a.rot, a.variant, lane);
    if (active) {
      // what later steps read from the page is the bfloat16 value: use the same value now
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        const bf16 kb = (bf16)kf[i];
        kf[i] = (float)kb;
        s_knew[e0 + i] = kf[i];
        s_vnew[e0 + i] = vf[i];
      }
    }
  }

  float qf[GT][EPL];
  float m[GT], l[GT], acc[GT][EPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) { acc[g][i] = 0.f; qf[g][i] = 0.f; }
    if (g < gcount && g % NW == wave) {
      float qv[EPL];
      unpack8(qraw[g], qv);
      if (RAW) {
        norm_rope8<LPK>(qv, e0, hd, a.q_gain, a.eps, rotate, rt, a.rot, a.variant, lane);
#pragma unroll
        for (int i = 0; i < EPL; ++i) qv[i] = (float)(bf16)qv[i];   // q is bfloat16 where it is stored
      }
      if (grp == 0 && active) {
#pragma unroll
        for (int i = 0; i < EPL; ++i) s_q[g][e0 + i] = qv[i] * a.scale;
      }
    }
  }

  // The slice's page ids go to LDS first (one round trip for all of them, instead of a dependent
  // table load in front of every key's loads); the loads of the next two keys are issued before the
  // current key is worked on, so that memory latency overlaps the arithmetic.
  for (int seg0 = k0; seg0 < k1; seg0 += SEG_PAGES * a.page_size) {
    const int first_page = a.page_shift >= 0 ? seg0 >> a.page_shift : seg0 / a.page_size;
    const int seg1 = min(k1, (first_page + SEG_PAGES) * a.page_size);
    if (seg0 != k0) __syncthreads();  // the previous segment's ids are no longer read
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      const int j = threadIdx.x + i * NW * WAVE;
      if (j < SEG_PAGES && (first_page + j) * a.page_size < seg1) {
        const int page = seg0 == k0 ? pre_page[i] : table[first_page + j];
        s_pages[j] = page;
      }
    }
    __syncthreads();  // the ids, and at the first segment the queries and the row's own key and value, are in LDS
    if (seg0 == k0) {
#pragma unroll
      for (int g = 0; g < GT; ++g)
#pragma unroll
        for (int i = 0; i < EPL; ++i) qf[g][i] = (g < gcount && active) ? s_q[g][e0 + i] : 0.f;
    }
    if (new_lane && hc == 0 && active && p >= seg0 && p < seg1) {
      // the row's own key and value go to their page (its id has just been staged)
      const int lp = a.page_shift >= 0 ? p >> a.page_shift : p / a.page_size;
      const int page = s_pages[lp - first_page];
      if (page >= 0 && page < a.num_pages) {   // the host never asks for another; never write outside
        // (both are bfloat16 values held as float: the upper 16 bits are the element)
        uint32_t kw[4], vw[4];
#pragma unroll
        for (int i = 0; i < EPL; i += 2) {
          kw[i / 2] = (__float_as_uint(s_knew[e0 + i]) >> 16) | (__float_as_uint(s_knew[e0 + i + 1]) & 0xffff0000u);
          vw[i / 2] = (__float_as_uint(s_vnew[e0 + i]) >> 16) | (__float_as_uint(s_vnew[e0 + i + 1]) & 0xffff0000u);
        }
        const size_t off = (((size_t)page * a.nkv + kvh) * a.page_size + (p - lp * a.page_size)) * hd + e0;
        *(uint4*)(kpages + off) = make_uint4(kw[0], kw[1], kw[2], kw[3]);
        *(uint4*)(vpages + off) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
      }
    }
    auto fetch = [&](int key, uint4& kr, uint4& vr) {
      kr = vr = make_uint4(0, 0, 0, 0);
      if (key < seg1 && !(RAW && key == p) && active) {
        const int lp = a.page_shift >= 0 ? key >> a.page_shift : key / a.page_size;
        const int page = min(max(s_pages[lp - first_page], 0), a.num_pages - 1);  // never read outside the pool
        const size_t off = (((size_t)page * a.nkv + kvh) * a.page_size + (key - lp * a.page_size)) * hd + e0;
        kr = *(const uint4*)(kpages + off);
        vr = *(const uint4*)(vpages + off);
      }
    };
    uint4 kraw[3], vraw[3];
    // the wave's first key of this segment keeps the global stride pattern k0 + (NW it + wave) KPW + grp
    int key = k0 + wave * KPW + grp;
    if (key < seg0) key += (seg0 - key + NW * KPW - 1) / (NW * KPW) * (NW * KPW);
    fetch(key, kraw[0], vraw[0]);
    fetch(key + NW * KPW, kraw[1], vraw[1]);
    for (; key < seg1; key += NW * KPW) {
      fetch(key + 2 * NW * KPW, kraw[2], vraw[2]);
      __builtin_amdgcn_sched_barrier(0);  // the loads above stay ahead of the arithmetic below
      float kf[EPL], vf[EPL];
      if (RAW && key == p) {
#pragma unroll
        for (int i = 0; i < EPL; ++i) { kf[i] = active ? s_knew[e0 + i] : 0.f; vf[i] = active ? s_vnew[e0 + i] : 0.f; }
      } else {
        unpack8(kraw[0], kf);
        unpack8(vraw[0], vf);
      }
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        if (g >= gcount) break;
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < EPL; ++i) d = fmaf(qf[g][i], kf[i], d);
        d = group_sum<LPK>(d);
        const float m_new = fmaxf(m[g], d);
        const float keep = __expf(m[g] - m_new);
        const float w = __expf(d - m_new);
        l[g] = l[g] * keep + w;
#pragma unroll
        for (int i = 0; i < EPL; ++i) acc[g][i] = fmaf(w, vf[i], acc[g][i] * keep);
        m[g] = m_new;
      }
      kraw[0] = kraw[1]; vraw[0] = vraw[1];
      kraw[1] = kraw[2]; vraw[1] = vraw[2];
    }
  }

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
  // the waves' streams of head g meet in wave g % NW
  if (grp != 0) return;
  for (int g = wave; g < gcount; g += NW) {
    float mm = s_ml[0][g][0], ll = s_ml[0][g][1], aa[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) aa[i] = s_acc[0][g][e0 + i];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
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

template <int LPK, bool RAW, int NW>
void launch_decode(int gt, dim3 grid, hipStream_t stream, const bf16* q, bf16* k, bf16* v, float* partial, bf16* out,
                   const DecodeArgs& a) {
  switch (gt) {
    case 1: attention_decode_kernel<LPK, 1, RAW, NW><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a); break;
    case 2: attention_decode_kernel<LPK, 2, RAW, NW><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a); break;
    case 4: attention_decode_kernel<LPK, 4, RAW, NW><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a); break;
    default: attention_decode_kernel<LPK, 8, RAW, NW><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a); break;
  }
}

template <int LPK, bool RAW>
void launch_waves(int waves, int gt, dim3 grid, hipStream_t stream, const bf16* q, bf16* k, bf16* v, float* partial,
                  bf16* out, const DecodeArgs& a) {
  // 8 waves keep their streams of up to 8 heads of up to LPK * 8 elements in LDS: only where that fits
  if (waves >= 8 && LPK * gt <= 128) launch_decode<LPK, RAW, 8>(gt, grid, stream, q, k, v, partial, out, a);
  else launch_decode<LPK, RAW, 4>(gt, grid, stream, q, k, v, partial, out, a);
}

template <bool RAW>
int run_decode(const bf16* q, bf16* kpages, bf16* vpages, bf16* out, float* partial, DecodeArgs a, int n_rows, int waves,
               hipStream_t stream) {
  const int G = a.nh / a.nkv;
  const int gt = G >= 8 ? 8 : (G > 2 ? 4 : G);  // 1, 2, 4 or 8 query heads per workgroup
  a.head_chunks = ceil_div(G, gt);
  a.page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;
  GIBBS_REQUIRE((long)a.nkv * a.head_chunks <= 65535, "attention_decode: too many heads");
  dim3 grid(n_rows, a.nkv * a.head_chunks, a.n_splits);
  const int lanes = a.hd / EPL;  // lanes that hold data; LPK is the next power of two
  if (lanes <= 2) launch_waves<2, RAW>(waves, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 4) launch_waves<4, RAW>(waves, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 8) launch_waves<8, RAW>(waves, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 16) launch_waves<16, RAW>(waves, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else launch_waves<32, RAW>(waves, gt, grid, stream, q, kpages, vpages, partial, out, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return gibbs_fail("attention_decode: %s", hipGetErrorString(e));
  if (a.n_splits > 1) {
    dim3 mgrid(n_rows, ceil_div(a.nh, 4));
    attention_merge_kernel<<<mgrid, 256, 0, stream>>>(partial, out, a.nh, a.hd, a.n_splits, a.ldo);
  }
  GIBBS_LAUNCH_STATUS("attention_decode");
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
                                        long ldo, float scale, int window, int n_splits, int waves, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_decode: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_decode: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 8 == 0 && hd <= 256, "attention_decode: head size %d must be a multiple of 8 up to 256", hd);
  GIBBS_REQUIRE(ldq % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_decode: q rows must be 16-byte aligned");
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention_decode: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode: bad cache geometry");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_decode: %d key slices need a workspace", n_splits);
  if (n_rows == 0) return 0;
  DecodeArgs a{};
  a.pos = pos; a.row_req = row_req; a.table = table; a.max_pages = max_pages; a.page_size = page_size;
  a.num_pages = num_pages; a.nh = nh; a.nkv = nkv; a.hd = hd; a.ldq = ldq; a.ldo = ldo; a.scale = scale;
  a.window = window; a.n_splits = n_splits;
  // the kernel only reads the pages here
  return run_decode<false>((const bf16*)q, (bf16*)kpages, (bf16*)vpages, (bf16*)out, partial, a, n_rows, waves, stream);
}

// qkv: [N, ld] bfloat16, raw projection (q heads, k heads, v heads) of N decoded tokens, one per request.
GIBBS_EXPORT int gibbs_attention_decode_fused(const void* qkv, void* kpages, void* vpages, void* out, float* partial,
                                              const float* q_gain, const float* k_gain, float eps,
                                              const float* inv_freq, int rot, int variant, const float* cs_table,
                                              int table_len, const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                                              int num_pages, int n_rows, int nh, int nkv, int hd, long ld, long ldo,
                                              float scale, int window, int n_splits, int waves, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_decode_fused: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_decode_fused: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 16 == 0 && hd <= 256, "attention_decode_fused: head size %d must be a multiple of 16 up to 256", hd);
  GIBBS_REQUIRE(ld % 8 == 0 && ((uintptr_t)qkv % 16) == 0 && ld >= (long)(nh + 2 * nkv) * hd, "attention_decode_fused: qkv rows must be 16-byte aligned and hold q, k and v");
  GIBBS_REQUIRE(ldo >= (long)nh * hd, "attention_decode_fused: output rows shorter than heads * hd");
  GIBBS_REQUIRE(!inv_freq || (rot > 0 && rot % 16 == 0 && rot <= hd), "attention_decode_fused: rotary_dim %d must be a multiple of 16 within the head size %d", rot, hd);
  GIBBS_REQUIRE(variant == 0 || variant == 1, "attention_decode_fused: unknown rotation variant %d", variant);
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode_fused: bad cache geometry");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_decode_fused: %d key slices need a workspace", n_splits);
  if (n_rows == 0) return 0;
  DecodeArgs a{};
  a.pos = pos; a.row_req = row_req; a.table = table; a.max_pages = max_pages; a.page_size = page_size;
  a.num_pages = num_pages; a.nh = nh; a.nkv = nkv; a.hd = hd; a.ldq = ld; a.ldo = ldo; a.scale = scale;
  a.window = window; a.n_splits = n_splits;
  a.q_gain = q_gain; a.k_gain = k_gain; a.eps = eps; a.inv_freq = inv_freq; a.rot = rot; a.variant = variant;
  a.cs_table = (const float2*)cs_table; a.table_len = cs_table ? table_len : 0;
  return run_decode<true>((const bf16*)qkv, (bf16*)kpages, (bf16*)vpages, (bf16*)out, partial, a, n_rows, waves, stream);
}
