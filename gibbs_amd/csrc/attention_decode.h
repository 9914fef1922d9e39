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
// partial (max, sum, values) and the slices are merged (see below).  The slice's page ids are
// staged in LDS, and the loads of the next two keys are in flight while a key is worked on.
//
// Two ways to walk the keys of a slice.  On the vector units: every LPK neighbouring lanes own one key
// at a time (as described above).  On the matrix cores (head sizes in steps of 16 up to 128, the
// default there): every wave takes tiles of 32 keys through a patch of LDS of its own; scores
// transposed, S^T = K Q^T with the kv head's query heads as the 16 columns, so that a lane holds 8
// scores of ONE head and the softmax needs two lane swaps per tile; exp(S - m) is, as it lies in the
// registers, the B operand of O^T += V^T P^T, and V^T comes from the tile as it was stored through
// the transposing LDS read of gfx950.  The vector walk costs about 20 instructions per key and wave,
// the matrix walk 4.
//
// Two entry points share the kernel.  `attention_decode` takes q as it is (already normed and
// rotated; the row's key and value already in their pages).  `attention_decode_fused` takes a step
// of decoded tokens as the raw fused projection qkv[N, (nh + 2 nkv) hd]: the kernel norms and
// rotates q on the fly (every slice's workgroup does, it is a few hundred operations), norms and
// rotates the row's own new key, writes it and the new value to their page (the workgroup of head
// chunk 0 whose key slice holds the row's position does) and uses them from LDS instead of
// reading them back.
//
// The slices of a (row, group of heads) are merged by the workgroup that finishes last: every workgroup writes its
// partial result through to memory (agent-scope stores), waits until the stores have arrived, and counts itself
// in with one relaxed agent-scope atomic; the one that counts last reads all the partial results with agent-scope
// loads, which pass its own L2, and leaves the counter at zero.  No fence: on this chip (one L2 per XCD) an
// agent-scope release or acquire fence writes back or invalidates a whole L2, which cost 130 us a call when every
// workgroup did it; the accesses above are coherent by themselves.  The chain (stores arrive, the count, the loads)
// takes about as long as the boundary to a second kernel: 0.8 us a call less than the merge kernel at 8 slices,
// 2.3 us at 64.  The merge kernel remains for calls with more (rows x groups of heads) than there are counters,
// and for callers that ask for it (kind + 4).
//
// Visibility is by position only: row n sees keys lo .. pos[n] of its request
// (lo = max(0, pos - window + 1), window 0 = all).
//
// This header holds the kernel and its launcher; attention_decode.hip and attention_decode_fused.hip
// instantiate it for prepared queries and for the raw fused projection (two translation units:
// the instantiations are most of the library's compile time).
#pragma once
#include "common.h"
#include "lane8.h"
#include "attention_merge.h"
#include <stdlib.h>

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef short short4v __attribute__((ext_vector_type(4)));
constexpr int SEG_PAGES = 512;  // page ids of a key slice kept in LDS at a time
constexpr int TILE = 32;        // keys per tile of the matrix-core walk

// Maximum / sum over the 4 lanes l, l ^ 16, l ^ 32, l ^ 48 (the lanes that hold one query head's scores in
// the matrix-core walk), every lane getting the result: two lane-swap instructions each.
__device__ __forceinline__ float row4_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float row4_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// 4 x 4 elements of a row-major 16-bit matrix in LDS, transposed: of the 16 lanes of a row of lanes, lane j
// passes the address of 4 consecutive elements and receives element j % 4 of the lanes j / 4, j / 4 + 4,
// j / 4 + 8, j / 4 + 12 (ds_read_b64_tr_b16).  With lane j pointing at V[key j / 4][d0 + 4 (j % 4)] it
// receives V[key 0..3][d0 + j]: the keys run along the register, as the matrix instruction wants them.
__device__ __forceinline__ short4v lds_read_transposed(const bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)p);
}

// Counters of the slices of a (row, group of heads) that have finished, for calls whose last slice merges.  Zero
// when the module is loaded, and the merging workgroup leaves zero behind.  One array per device and translation
// unit: calls that overlap on one device (two streams) would share it, as they would share a workspace.
constexpr int MERGE_COUNTERS = 1 << 15;
static __device__ int g_merge_counters[MERGE_COUNTERS];

// Two floats (8-byte aligned) written through to where every compute unit of the device sees them.
__device__ __forceinline__ void store_through2(float* p, float a, float b) {
  const unsigned long long v = ((unsigned long long)__float_as_uint(b) << 32) | __float_as_uint(a);
  __hip_atomic_store((unsigned long long*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_through(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One wave merges the slices of a (row, head) that other workgroups of the same kernel wrote with store_through2:
// out = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s, eight slices' loads in flight at a time.
// C: elements of a head per lane.
template <int C>
__device__ __forceinline__ void merge_slices_through(const float* ps, int n_splits, int hd, bf16* o, int lane) {
  const int stride = hd + 2;
  float M = -INFINITY, L = 0.f, v[C];
#pragma unroll
  for (int c = 0; c < C; ++c) v[c] = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += 8) {
    float ms[8], ls[8], av[8][C];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = min(s0 + j, n_splits - 1);      // (beyond the last slice: the last one again, weighted 0 below)
      ms[j] = load_through(ps + (size_t)s * stride);
      ls[j] = load_through(ps + (size_t)s * stride + 1);
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const int e = lane + c * WAVE;
        av[j][c] = load_through(ps + (size_t)s * stride + 2 + (e < hd ? e : 0));
      }
    }
    float Mn = M;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < n_splits) Mn = fmaxf(Mn, ms[j]);
    const float keep = M == -INFINITY ? 0.f : __expf(M - Mn);
    L *= keep;
#pragma unroll
    for (int c = 0; c < C; ++c) v[c] *= keep;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float w = (s0 + j < n_splits && ms[j] != -INFINITY) ? __expf(ms[j] - Mn) : 0.f;
      L = fmaf(w, ls[j], L);
#pragma unroll
      for (int c = 0; c < C; ++c) v[c] = fmaf(w, av[j][c], v[c]);
    }
    M = Mn;
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int e = lane + c * WAVE;
    if (e < hd) o[e] = (bf16)(v[c] * inv);
  }
}

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
  // A row's whole block table fits the staging area in LDS (no window, the caller's bound on the keys): its first
  // n_ids page ids are asked for at once, before the row's position is known (one dependent load less in front
  // of the first keys).  A row that is beyond the bound after all takes the ids of its slice as it would without.
  int ids_whole, n_ids;
  int merge_here;   // the last slice of a (row, group of heads) to finish merges them (else a second kernel does)
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

// MM: the keys of a slice are walked in tiles of 32 on the matrix cores (see the head of the file);
// otherwise key by key on the vector units.
template <int LPK, int GT, bool RAW, int NW, bool MM>
__global__ __launch_bounds__(NW * WAVE, GT <= 4 ? (NW == 8 ? 4 : 3) : 2) void attention_decode_kernel(const bf16* __restrict__ qkv, bf16* __restrict__ kpages,
                                                               bf16* __restrict__ vpages, float* __restrict__ partial,
                                                               bf16* __restrict__ out, const int* __restrict__ pos_,
                                                               const int* __restrict__ table_, DecodeArgs rest) {
  // (the pointers that the first loads hang on are scalar arguments: those arrive in registers with the wave,
  // the struct's fields by loads)
  DecodeArgs a = rest;
  a.pos = pos_;
  a.table = table_;
  constexpr int KPW = WAVE / LPK;
  constexpr int MAX_HD = LPK * EPL;
  __shared__ float s_ml[NW][GT][2];
  __shared__ float s_acc[NW][GT][MAX_HD];
  __shared__ float s_knew[MAX_HD], s_vnew[MAX_HD];
  __shared__ float s_q[GT][MAX_HD];
  __shared__ int s_pages[SEG_PAGES];
  constexpr int LDT = MAX_HD + 8;                       // row of a tile in LDS (padded against bank conflicts)
  __shared__ __attribute__((aligned(16))) bf16 s_tiles[MM ? NW * 2 * TILE * LDT : 8];   // a K and a V tile per wave

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

  // (row_req null: row n is request n, as in a step of decoded tokens alone)
  const int* table = a.table + (size_t)(a.row_req ? a.row_req[row] : row) * a.max_pages;
  constexpr int PRE = (SEG_PAGES + NW * WAVE - 1) / (NW * WAVE);
  int pre_page[PRE];
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    const int j = threadIdx.x + i * NW * WAVE;
    pre_page[i] = (a.ids_whole && j < a.n_ids) ? table[j] : 0;
  }
  const int p = a.pos[row];
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int len = p + 1 - lo;
  int per = (len + a.n_splits - 1) / a.n_splits;
  constexpr int UNIT = NW * (MM ? TILE : KPW);   // every wave gets whole tiles (or whole steps of keys)
  per = (per + UNIT - 1) / UNIT * UNIT;
  const int k0 = lo + split * per;
  const int k1 = min(k0 + per, p + 1);
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
  const bool whole = a.ids_whole && p < a.n_ids * a.page_size;
  const int first_page0 = whole ? 0 : (a.page_shift >= 0 ? k0 >> a.page_shift : k0 / a.page_size);
  const int seg1_0 = whole ? k1 : min(k1, (first_page0 + SEG_PAGES) * a.page_size);
  if (!whole) {
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      const int j = threadIdx.x + i * NW * WAVE;
      pre_page[i] = (j < SEG_PAGES && (first_page0 + j) * a.page_size < seg1_0) ? table[first_page0 + j] : 0;
    }
  }

  // The first segment's page ids go to LDS, and the loads of the wave's first tile of keys are asked for, before
  // the queries and the row's own key are prepared: the preparation (rotation factors that hang on the position,
  // norms, rotation) runs while those loads are on their way.
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    const int j = threadIdx.x + i * NW * WAVE;
    if (j < SEG_PAGES && (whole ? j < a.n_ids : (first_page0 + j) * a.page_size < seg1_0)) s_pages[j] = pre_page[i];
  }
  __syncthreads();  // the first segment's ids are in LDS
  // a key's and a value's 16 bytes of this lane; first_page: the page whose id is s_pages[0]
  auto fetch = [&](int key, int seg1, int first_page, uint4& kr, uint4& vr) {
    kr = vr = make_uint4(0, 0, 0, 0);
    if (key < seg1 && !(RAW && key == p) && active) {
      const int lp = a.page_shift >= 0 ? key >> a.page_shift : key / a.page_size;
      const int page = min(max(s_pages[lp - first_page], 0), a.num_pages - 1);  // never read outside the pool
      const size_t off = (((size_t)page * a.nkv + kvh) * a.page_size + (key - lp * a.page_size)) * hd + e0;
      kr = *(const uint4*)(kpages + off);
      vr = *(const uint4*)(vpages + off);
    }
  };
  constexpr int LPT = MM ? TILE / KPW : 1;   // loads of K (and of V) per tile of the matrix-core walk
  uint4 kreg[LPT], vreg[LPT];
  if constexpr (MM) {
    // (the matrix-core walk has one segment: the launcher sees to it that a slice's ids fit the staging area)
    if (wave * TILE < seg1_0 - k0) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) fetch(k0 + wave * TILE + i * KPW + grp, seg1_0, first_page0, kreg[i], vreg[i]);
    }
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
        for (int i = 0; i < EPL; ++i) s_q[g][e0 + i] = MM ? qv[i] : qv[i] * a.scale;   // (MM scales the scores instead)
      }
    }
  }

  // state of the matrix-core walk: this lane holds, of query head lane % 16, the scores of 8 keys per
  // tile, and of the output elements d = t*16 + (lane / 16)*4 + i
  constexpr int DTM = MAX_HD / 16, DSM = (DTM + 1) / 2;
  const int lr = lane % 16, g4 = lane / 16;
  bf16x8 qb[DSM];
  float mm_m = -1e30f, mm_l = 0.f;   // (a finite stand-in for 'no key yet': exp2 of anything minus it is 0)
  floatx4 mm_o[DTM];
#pragma unroll
  for (int t = 0; t < DTM; ++t) mm_o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The slice's page ids go to LDS first (one round trip for all of them, instead of a dependent
  // table load in front of every key's loads); the loads of the next two keys are issued before the
  // current key is worked on, so that memory latency overlaps the arithmetic.
  __syncthreads();  // the queries and the row's own key and value are in LDS
  for (int seg0 = k0; seg0 < k1; seg0 += SEG_PAGES * a.page_size) {
    const int first_page = seg0 == k0 ? first_page0 : (a.page_shift >= 0 ? seg0 >> a.page_shift : seg0 / a.page_size);
    const int seg1 = seg0 == k0 ? seg1_0 : min(k1, (first_page + SEG_PAGES) * a.page_size);
    if (seg0 != k0) {
      __syncthreads();  // the previous segment's ids are no longer read
#pragma unroll
      for (int i = 0; i < PRE; ++i) {
        const int j = threadIdx.x + i * NW * WAVE;
        if (j < SEG_PAGES && (first_page + j) * a.page_size < seg1) s_pages[j] = table[first_page + j];
      }
      __syncthreads();
    }
    if (seg0 == k0) {
      if constexpr (MM) {
        // B operands of S^T = K Q^T: column lr is query head g0 + lr, d = s*32 + g4*8 .. +8
#pragma unroll
        for (int s = 0; s < DSM; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int d = s * 32 + g4 * 8 + e;
            qb[s][e] = (lr < gcount && d < hd) ? (bf16)s_q[lr < GT ? lr : 0][d < MAX_HD ? d : 0] : (bf16)0.f;
          }
      } else {
#pragma unroll
        for (int g = 0; g < GT; ++g)
#pragma unroll
          for (int i = 0; i < EPL; ++i) qf[g][i] = (g < gcount && active) ? s_q[g][e0 + i] : 0.f;
      }
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
    if constexpr (MM) {
      // The wave's tiles of the slice: keys k0 + j*32 .. +32 for j = wave, wave + NW, ...  A tile travels
      // memory -> registers (one tile ahead) -> the wave's own patch of LDS (no barrier: only this wave
      // reads it) -> matrix instructions: S^T = K Q^T (this lane gets, of head lr, the keys c*16 + g4*4 + i),
      // softmax with one head per lane, O^T += V^T P^T with P^T straight from the registers and V^T by
      // transposing reads of the tile as it was stored.
      bf16 (*tK)[LDT] = reinterpret_cast<bf16 (*)[LDT]>(s_tiles + (size_t)wave * 2 * TILE * LDT);
      bf16 (*tV)[LDT] = tK + TILE;
      auto fetch_tile = [&](int t0) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) fetch(t0 + i * KPW + grp, seg1, first_page, kreg[i], vreg[i]);
      };
      const float scale2 = a.scale * 1.44269504088896340736f;
      const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
      const int n_tiles = (seg1 - k0 + TILE - 1) / TILE;
      for (int j = wave; j < n_tiles; j += NW) {   // (the wave's first tile was asked for before the preparation)
        const int t0 = k0 + j * TILE;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads of the previous tile are through
        if (active) {
#pragma unroll
          for (int i = 0; i < LPT; ++i) {
            *(uint4*)&tK[i * KPW + grp][e0] = kreg[i];
            *(uint4*)&tV[i * KPW + grp][e0] = vreg[i];
          }
        }
        if (j + NW < n_tiles) fetch_tile(k0 + (j + NW) * TILE);
        __builtin_amdgcn_sched_barrier(0);  // the loads above stay ahead of the arithmetic below
        if (RAW && p >= t0 && p < t0 + TILE && grp == 0 && active) {
          // the row's own key and value are not in their page yet (or not visibly): from LDS
#pragma unroll
          for (int i = 0; i < EPL; ++i) {
            tK[p - t0][e0 + i] = (bf16)s_knew[e0 + i];
            tV[p - t0][e0 + i] = (bf16)s_vnew[e0 + i];
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the tile is in LDS
        floatx4 s4[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          s4[c] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s2 = 0; s2 < DSM; ++s2) {
            const int d = s2 * 32 + g4 * 8;
            const bf16x8 kf = d < hd ? *(const bf16x8*)&tK[c * 16 + lr][d] : zero8;
            s4[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qb[s2], s4[c], 0, 0, 0);
          }
        }
        // keys beyond the slice (the last tile); maximum of the raw scores (the scale is positive)
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float v = t0 + c * 16 + g4 * 4 + i < seg1 ? s4[c][i] : -INFINITY;
            s4[c][i] = v;
            mx = fmaxf(mx, v);
          }
        mx = row4_max(mx);
        const float m_new = fmaxf(mm_m, mx);
        const float keep = __builtin_amdgcn_exp2f((mm_m - m_new) * scale2);
        const float shift = -m_new * scale2;
        mm_m = m_new;
        mm_l *= keep;
        bf16x8 pf;   // P^T as the B operand: element e is key (e / 4) * 16 + g4 * 4 + e % 4 of the tile
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float pr = __builtin_amdgcn_exp2f(fmaf(s4[c][i], scale2, shift));
            mm_l += pr;
            pf[c * 4 + i] = (bf16)pr;
          }
#pragma unroll
        for (int t = 0; t < DTM; ++t) {
          if (t * 16 >= hd) break;
#pragma unroll
          for (int i = 0; i < 4; ++i) mm_o[t][i] *= keep;
          // V^T of d = t*16 + lr, the same 8 keys: two transposing reads of 4 keys each
          const short4v v0 = lds_read_transposed(&tV[g4 * 4 + lr / 4][t * 16 + 4 * (lr % 4)]);
          const short4v v1 = lds_read_transposed(&tV[16 + g4 * 4 + lr / 4][t * 16 + 4 * (lr % 4)]);
          typedef short short8v __attribute__((ext_vector_type(8)));
          const short8v both = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
          mm_o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), pf, mm_o[t], 0, 0, 0);
        }
      }
    } else {
      uint4 kraw[3], vraw[3];
      // the wave's first key of this segment keeps the global stride pattern k0 + (NW it + wave) KPW + grp
      int key = k0 + wave * KPW + grp;
      if (key < seg0) key += (seg0 - key + NW * KPW - 1) / (NW * KPW) * (NW * KPW);
      fetch(key, seg1, first_page, kraw[0], vraw[0]);
      fetch(key + NW * KPW, seg1, first_page, kraw[1], vraw[1]);
      for (; key < seg1; key += NW * KPW) {
        fetch(key + 2 * NW * KPW, seg1, first_page, kraw[2], vraw[2]);
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
  }

  if constexpr (MM) {
    // this wave's stream of head lr, in the units of the fold below (natural logarithm, scaled scores)
    const float total = row4_sum(mm_l);
    if (lr < gcount) {
      if (g4 == 0) { s_ml[wave][lr][0] = mm_m * a.scale; s_ml[wave][lr][1] = total; }
#pragma unroll
      for (int t = 0; t < DTM; ++t) {
        if (t * 16 >= hd) break;
#pragma unroll
        for (int i = 0; i < 4; ++i) s_acc[wave][lr][t * 16 + g4 * 4 + i] = mm_o[t][i];
      }
    }
  } else {
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
  }
  __syncthreads();
  // the waves' streams of head g meet in wave g % NW
  const bool merge_here = a.n_splits > 1 && a.merge_here;
  if (grp == 0) {
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
      } else if (merge_here) {
        // stores that another workgroup, on another L2, reads in this same kernel: written through
        float* ps = partial + (((size_t)row * a.nh + head) * a.n_splits + split) * (hd + 2);
        if (sub == 0) store_through2(ps, mm, ll);
        if (active) {
#pragma unroll
          for (int i = 0; i < EPL; i += 2) store_through2(ps + 2 + e0 + i, aa[i], aa[i + 1]);
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
  if (!merge_here) return;
  // The slice of a (row, group of heads) that finishes last merges them all.  Every wave waits until its own
  // stores have arrived; then one thread counts the workgroup in.  The count, the stores above and the loads
  // below are agent-scope accesses (they pass the L2 of their XCD); no fence is needed besides: a fence would
  // write back and invalidate a whole L2 per workgroup.
  __builtin_amdgcn_s_waitcnt(0);   // (every counter: the stores are vmcnt)
  __syncthreads();
  __shared__ int s_last;
  int* counter = g_merge_counters + (size_t)row * gridDim.y + blockIdx.y;
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = before == a.n_splits - 1;
    if (s_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next call
  }
  __syncthreads();
  if (!s_last) return;
  constexpr int C = (MAX_HD + WAVE - 1) / WAVE;
  for (int g = wave; g < gcount; g += NW) {
    const int head = kvh * G + g0 + g;
    merge_slices_through<C>(partial + ((size_t)row * a.nh + head) * a.n_splits * (hd + 2), a.n_splits, hd,
                            out + (size_t)row * a.ldo + (size_t)head * hd, lane);
  }
}

template <int LPK, bool RAW, int NW, bool MM>
void launch_decode(int gt, dim3 grid, hipStream_t stream, const bf16* q, bf16* k, bf16* v, float* partial, bf16* out,
                   const DecodeArgs& a) {
  switch (gt) {
    case 1: attention_decode_kernel<LPK, 1, RAW, NW, MM><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a.pos, a.table, a); break;
    case 2: attention_decode_kernel<LPK, 2, RAW, NW, MM><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a.pos, a.table, a); break;
    case 4: attention_decode_kernel<LPK, 4, RAW, NW, MM><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a.pos, a.table, a); break;
    default: attention_decode_kernel<LPK, 8, RAW, NW, MM><<<grid, NW * WAVE, 0, stream>>>(q, k, v, partial, out, a.pos, a.table, a); break;
  }
}

template <int LPK, bool RAW>
void launch_waves(int waves, bool mm, int gt, dim3 grid, hipStream_t stream, const bf16* q, bf16* k, bf16* v,
                  float* partial, bf16* out, const DecodeArgs& a) {
  // 8 waves keep their streams of up to 8 heads of up to LPK * 8 elements in LDS: only where that fits
  const bool eight = waves >= 8 && LPK * gt <= 128;
  if constexpr (LPK <= 16) {   // (head sizes up to 128 on the matrix cores)
    if (mm) {
      if constexpr (LPK <= 8) {   // (8 waves' tiles of wider heads do not fit in LDS)
        if (eight) {
          launch_decode<LPK, RAW, 8, true>(gt, grid, stream, q, k, v, partial, out, a);
          return;
        }
      }
      launch_decode<LPK, RAW, 4, true>(gt, grid, stream, q, k, v, partial, out, a);
      return;
    }
  }
  if (eight) launch_decode<LPK, RAW, 8, false>(gt, grid, stream, q, k, v, partial, out, a);
  else launch_decode<LPK, RAW, 4, false>(gt, grid, stream, q, k, v, partial, out, a);
}

// kind: 0 = choose, 1 = vector units, 2 = matrix cores (refused where they cannot take the shape); + 4: the slices
// are merged by a second kernel even where the last slice to finish could do it
template <bool RAW>
int run_decode(const bf16* q, bf16* kpages, bf16* vpages, bf16* out, float* partial, DecodeArgs a, int n_rows, int waves,
               int kind, int max_keys, hipStream_t stream) {
  const int G = a.nh / a.nkv;
  const int gt = G >= 8 ? 8 : (G > 2 ? 4 : G);  // 1, 2, 4 or 8 query heads per workgroup
  a.head_chunks = ceil_div(G, gt);
  a.page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;
  GIBBS_REQUIRE((long)a.nkv * a.head_chunks <= 65535, "attention_decode: too many heads");
  dim3 grid(n_rows, a.nkv * a.head_chunks, a.n_splits);
  // The last slice to finish merges, where the counters reach; kind + 4 asks for the second kernel instead.
  a.merge_here = a.n_splits > 1 && !(kind & 4) && (long)n_rows * grid.y <= MERGE_COUNTERS;
  kind &= 3;
  const int lanes = a.hd / EPL;  // lanes that hold data; LPK is the next power of two
  // The matrix-core walk keeps the page ids of a whole key slice in LDS and takes head sizes in steps of
  // 16 up to 128.  The longest slice that the block table (or the caller's bound on the keys) allows:
  const long bound = max_keys > 0 ? min((long)max_keys, (long)a.max_pages * a.page_size) : (long)a.max_pages * a.page_size;
  const long longest = (bound + a.n_splits - 1) / a.n_splits + 8 * TILE;
  const bool mm_can = a.hd % 16 == 0 && a.hd <= 128 && longest / a.page_size + 2 <= SEG_PAGES;
  GIBBS_REQUIRE(kind != 2 || mm_can, "attention_decode: the matrix-core kernel takes head sizes in steps of 16 up to 128 and key slices of at most %d pages (head size %d, %ld keys a slice)", SEG_PAGES - 2, a.hd, longest);
  const bool mm = kind == 2 || (kind == 0 && mm_can);
  const long ids = (bound + a.page_size - 1) / a.page_size;
  a.ids_whole = a.window == 0 && ids <= SEG_PAGES;
  a.n_ids = (int)min(ids, (long)a.max_pages);
  if (lanes <= 2) launch_waves<2, RAW>(waves, mm, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 4) launch_waves<4, RAW>(waves, mm, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 8) launch_waves<8, RAW>(waves, mm, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else if (lanes <= 16) launch_waves<16, RAW>(waves, mm, gt, grid, stream, q, kpages, vpages, partial, out, a);
  else launch_waves<32, RAW>(waves, false, gt, grid, stream, q, kpages, vpages, partial, out, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return gibbs_fail("attention_decode: %s", hipGetErrorString(e));
  if (a.n_splits > 1 && !a.merge_here) {
    dim3 mgrid(n_rows, ceil_div(a.nh, 4));
    launch_attention_merge(mgrid, stream, partial, out, a.nh, a.hd, a.n_splits, a.ldo);
  }
  GIBBS_LAUNCH_STATUS("attention_decode");
}
}  // namespace
