// Paged causal attention for prompt portions on the gfx950 matrix cores (bfloat16 in, float32
// scores, maxima, sums and accumulators).
//
// A workgroup takes 64 consecutive query rows of one request and HPW query heads that share a kv head
// (1, 2 or 4 of the group's); 4 waves per head, each owning 16 of the rows.  One K and one V tile in LDS
// serve all of the workgroup's heads: with one head a workgroup re-reads every key and value of its rows'
// past for 64 x 64 scores, and at 8,192 rows and more that traffic through L2 and the compute units' L1s,
// not the arithmetic, bounds the kernel (32,768 rows: 69 GB a call, 8.4 TB/s).  Keys are walked in tiles of
// 64 aligned to absolute key index (so a row's sequence of operations does not depend on how the prompt
// was cut).  Per tile:
//   K and V tiles -> LDS as stored ([key][d]);
//   scores transposed, S^T (64 keys x 16 rows per wave) = K Q^T by v_mfma_f32_16x16x32_bf16 over d:
//   a lane then holds 16 scores of ONE query row (lane % 16), so that the online softmax needs no
//   exchange between lanes except two steps over the 4 lanes that share the row, and exp(S - m)
//   is, as it lies in the registers, the B operand of O^T += V^T P^T (the contraction runs over
//   the keys in any order, as long as V^T is read in the same one): P never goes through LDS.
//   V^T comes from the V tile as it was stored, through the transposing LDS read of gfx950.
// Keys come from the request's pages through its block table; row n sees keys lo .. pos[n]
// (lo = max(0, pos - window + 1), window 0 = all).  The step's own keys were written to the pages
// before this kernel runs.  Head sizes: multiples of 16 up to 128.
//
// Few rows over a long cache (a prompt portion late in a long prompt) give too few workgroups to fill
// the chip: the key tiles of a workgroup's rows are then cut into n_splits slices that run as
// workgroups of their own (grid z) and leave (max, sum, weighted values) for the merge kernel.
#include "common.h"
#include "attention_merge.h"

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

constexpr int BM = 64;   // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int SEG_PAGES = 1024;  // page ids kept in LDS at a time (a segment of the request's block table)

// Maximum / sum over the 4 lanes that hold one query row's scores (lanes l, l ^ 16, l ^ 32, l ^ 48),
// every lane getting the result: two lane-swap instructions each (rows of 16 lanes, halves of 32).
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

struct PrefillArgs {
  const int* cu;
  const int* ctx;
  const int* table;
  int n_req, max_pages, page_size, num_pages;
  int page_shift;  // log2(page_size) if it is a power of two, else -1
  int nh, nkv, hd;
  long ldq, ldo;
  float scale;
  int window;
  int n_splits;    // slices of the key tiles (1: the workgroup writes the finished rows)
};

// DT: head size = 16 * DT.  POW2: the page size is a power of two (shifts instead of divisions: an
// integer division costs dozens of instructions, several times per thread and tile).
// Five waves a SIMD are asked for: the walk over the keys is a chain of short waits (two barriers a tile, LDS, the
// next tile's loads) that other waves have to fill; head sizes up to 64 fit the 96 registers that leaves without
// spilling (at 8,192 rows 10 % faster than with four waves; six waves spill and are no faster).  Larger heads are
// left to the compiler: asked for five waves, head sizes 80 and 96 spill.
// HPW: query heads per workgroup (256 threads each).
template <int DT, bool POW2, int HPW>
__global__ __launch_bounds__(256 * HPW) __attribute__((amdgpu_waves_per_eu(DT <= 4 ? (HPW == 1 ? 5 : 4) : 1))) void attention_prefill_kernel(const bf16* __restrict__ q,
                                                                const bf16* __restrict__ kpages,
                                                                const bf16* __restrict__ vpages, bf16* __restrict__ out,
                                                                float* __restrict__ partial, PrefillArgs a) {
  constexpr int HD = 16 * DT;
  constexpr int DS = (DT + 1) / 2;  // steps of 32 over d
  // Rows of the tiles in LDS are padded against bank conflicts, K and V differently: a read of K operands has 16
  // lanes on 16 rows with 16 bytes each (row stride of 4 banks modulo 8), a transposing read of V has 32 lanes on
  // 8 rows with 32 bytes each (row stride of 8 banks modulo 16: with the stride of K the eighth row wraps onto
  // the first one's banks, and the read takes two turns).
  constexpr int LDK = HD + 8;
  constexpr int LDV = HD % 32 == 16 ? HD + 32 : HD + 16;
  constexpr int NT = 256 * HPW;     // threads of the workgroup
  // Tiles in LDS: three that take turns (one barrier a tile) where several heads share them; with one head a
  // workgroup, one tile and two barriers, so that five workgroups still fit a compute unit's LDS.
  constexpr int NB = HPW > 1 ? 3 : 1;
  __shared__ bf16 sK[NB][BN][LDK];
  __shared__ __attribute__((aligned(16))) bf16 sV[NB][BN][LDV];
  __shared__ int s_pages[SEG_PAGES];

  // which request and which 64 rows of it
  int tile = blockIdx.x, r = 0, qlen = 0;
  for (; r < a.n_req; ++r) {
    qlen = a.cu[r + 1] - a.cu[r];
    const int t = (qlen + BM - 1) / BM;
    if (tile < t) {
      tile = t - 1 - tile;  // a request's last rows see the most keys: those workgroups start first
      break;
    }
    tile -= t;
  }
  if (r >= a.n_req) return;
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = (tid / WAVE) % 4;                 // which 16 of the 64 rows
  const int head = blockIdx.y * HPW + tid / 256;     // (HPW divides the heads per kv head: all share kvh)
  const int kvh = head / (a.nh / a.nkv);
  const int lr = lane % 16, g = lane / 16;
  const int row_in_req0 = tile * BM;                 // first row of the tile inside the request's rows
  const int n0 = a.cu[r] + row_in_req0;              // its index among the step's rows
  const int p0 = a.ctx[r] + row_in_req0;             // its absolute position
  const int rows_here = min(BM, qlen - row_in_req0);
  const int* table = a.table + (size_t)r * a.max_pages;
  // (page, slot) of a key; page ids come from a segment of the block table held in LDS, so that a
  // tile's loads do not wait for a table load first
  int seg_first_page = 0;
  auto logical_page = [&](int ak) -> int { return POW2 ? ak >> a.page_shift : ak / a.page_size; };
  auto page_row = [&](const bf16* pages, int ak) -> const bf16* {
    const int lp = logical_page(ak);
    return pages + (((size_t)s_pages[lp - seg_first_page] * a.nkv + kvh) * a.page_size + (ak - lp * a.page_size)) * HD;
  };

  // Q fragments: A operand, lane holds row lr of the wave's 16 rows, d = s*32 + g*8 .. +8
  const int my_row = wave * 16 + lr;                 // row inside the tile this lane loads
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    const int d = s * 32 + g * 8;
    qf[s] = (my_row < rows_here && d < HD)
                ? *(const bf16x8*)(q + (size_t)(n0 + my_row) * a.ldq + (size_t)head * HD + d)
                : zero8;
  }
  // the query row this lane owns in S^T and O^T: wave*16 + lr; it sees keys above lo_row up to pos_row
  const int pos_row = p0 + min(wave * 16 + lr, rows_here - 1);
  const int lo_row = a.window > 0 ? pos_row - a.window : -1;

  // a finite stand-in for 'no key seen yet': exp2 of anything minus it is 0, with no special cases
  float m = -1e30f, l = 0.f;   // maximum of the raw scores; sum of this lane's share of the row
  floatx4 o[DT];               // O^T: d = t*16 + g*4 + i of row lr
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const float scale2 = a.scale * 1.44269504088896340736f;
  const int last_pos = p0 + rows_here - 1;
  const int first_key = a.window > 0 ? max(0, p0 - a.window + 1) : 0;
  const int wave_last = p0 + min(wave * 16 + 15, rows_here - 1);
  const int wave_first_key = a.window > 0 ? max(0, p0 + wave * 16 - a.window + 1) : 0;

  // One tile ahead: the next tile's keys and values travel from memory to registers while the
  // matrix cores work on the current tile, and go to LDS once everyone is done with it.
  constexpr int KCH = (BN * (HD / 8) + NT - 1) / NT;      // 16-byte chunks of K (and of V) per thread and tile
  uint4 kreg[KCH], vreg[KCH];
  // (a key's and its value's chunk lie at the same offset of their pools; with a page size that is a power of two
  // the offset is a page's stride times the page id plus a few shifts: an address costs a handful of instructions,
  // and the walk over the keys is bound by the vector instructions it issues)
  const size_t page_stride = (size_t)a.nkv * a.page_size * HD;
  const unsigned head_off = (unsigned)kvh * a.page_size * HD;
  auto load_tile = [&](int key0) {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT;
      const int key = c / (HD / 8), d = (c % (HD / 8)) * 8;
      kreg[i] = vreg[i] = make_uint4(0, 0, 0, 0);
      if (c < BN * (HD / 8) && key0 + key <= last_pos) {
        if constexpr (POW2) {
          const int ak = key0 + key;
          const unsigned page = (unsigned)s_pages[(ak >> a.page_shift) - seg_first_page];
          const size_t off = page * page_stride + (head_off + (unsigned)(ak & (a.page_size - 1)) * HD + d);
          kreg[i] = *(const uint4*)(kpages + off);
          vreg[i] = *(const uint4*)(vpages + off);
        } else {
          kreg[i] = *(const uint4*)(page_row(kpages, key0 + key) + d);
          vreg[i] = *(const uint4*)(page_row(vpages, key0 + key) + d);
        }
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT;
      if (c < BN * (HD / 8)) {
        *(uint4*)&sK[buf][c / (HD / 8)][(c % (HD / 8)) * 8] = kreg[i];
        *(uint4*)&sV[buf][c / (HD / 8)][(c % (HD / 8)) * 8] = vreg[i];
      }
    }
  };
  // the block-table segment that holds the pages of tile `key0` (tiles and segments are aligned)
  const int seg_keys = SEG_PAGES * a.page_size / BN * BN;   // keys per segment, whole tiles
  auto load_segment = [&](int key0) {
    seg_first_page = logical_page(key0 / seg_keys * seg_keys);
    const int last_page = logical_page(last_pos);
    for (int j = tid; j < SEG_PAGES && seg_first_page + j <= last_page; j += NT) {
      const int page = table[seg_first_page + j];
      s_pages[j] = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);  // never read outside the pool
    }
    __syncthreads();
  };

  // this workgroup's slice of the key tiles first_key / BN .. last_pos / BN
  int kt_first = first_key / BN, kt_stop = last_pos / BN + 1;
  if (a.n_splits > 1) {
    const int per = (kt_stop - kt_first + a.n_splits - 1) / a.n_splits;
    kt_first += blockIdx.z * per;
    kt_stop = min(kt_stop, kt_first + per);
  }
  auto ask_for = [&](int kt) {   // (uniform: everyone takes a new segment of page ids together)
    if ((kt * BN) % seg_keys == 0 || kt == kt_first) load_segment(kt * BN);
    load_tile(kt * BN);
  };
  // a wave whose rows see none of a tile's keys (or that has no rows) has nothing to do for it but take part
  auto busy = [&](int kt) { return !(kt * BN > wave_last || kt * BN + BN <= wave_first_key || wave * 16 >= rows_here); };
  // S^T = K Q^T: 4 sub-tiles of 16 keys; this lane gets S[row lr][key c*16 + g*4 + i]
  auto scores = [&](int buf, floatx4 (&s4)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s4[c] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int d = s * 32 + g * 8;
        const bf16x8 kf = d < HD ? *(const bf16x8*)&sK[buf][c * 16 + lr][d] : zero8;
        s4[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], s4[c], 0, 0, 0);
      }
    }
  };
  // mask, online softmax; P^T = exp(S^T - m) as B operands of the second product
  auto weights = [&](floatx4 (&s4)[4], int key0, bf16x8 (&pf)[2]) {
    // mask by position (only the tiles on the rows' diagonal, or with a window: the same for the whole wave,
    // and said so, or the selects are done for every tile), row maximum (of the raw scores: the scale is positive)
    const bool need_mask = __builtin_amdgcn_readfirstlane((int)(key0 + BN - 1 > p0 + wave * 16 || a.window > 0)) != 0;
    if (need_mask) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = key0 + c * 16 + g * 4 + i;
          const bool vis = (key <= pos_row) & (key > lo_row);
          s4[c][i] = vis ? s4[c][i] : -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s4[c][i]);
    mx = row4_max(mx);
    const float m_new = fmaxf(m, mx);
    const float keep = __builtin_amdgcn_exp2f((m - m_new) * scale2);
    const float shift = -m_new * scale2;
    m = m_new;
    l *= keep;
    // in units of log2 (exp(s) = exp2(s * log2 e)); element e of step kk is key (2 kk + e / 4) * 16 + g * 4 + e % 4
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s4[c][i], scale2, shift));
        l += p;
        pf[c / 2][(c % 2) * 4 + i] = (bf16)p;
      }
    // (most tiles leave every row's maximum as it was: a factor of exactly 1, and nothing to do)
    if (__builtin_amdgcn_ballot_w64(keep != 1.f) != 0) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[t][i] *= keep;
    }
  };
  // O^T += V^T P^T: k runs over the 64 keys in 2 steps of 32
  auto values = [&](int buf, const bf16x8 (&pf)[2]) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        // V^T of d = t*16 + lr, the 8 keys of pf[kk]: two transposing reads of 4 keys each
        const short4v v0 = lds_read_transposed(&sV[buf][(2 * kk) * 16 + g * 4 + lr / 4][t * 16 + 4 * (lr % 4)]);
        const short4v v1 = lds_read_transposed(&sV[buf][(2 * kk + 1) * 16 + g * 4 + lr / 4][t * 16 + 4 * (lr % 4)]);
        const short8v both = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), pf[kk], o[t], 0, 0, 0);
      }
    }
  };

  if constexpr (NB == 1) {
    // One tile in LDS: the tile that waits in registers (asked for one tile earlier) goes to LDS between two
    // barriers at the head of the iteration, and the next one is asked for.
    if (kt_first < kt_stop) ask_for(kt_first);
    for (int kt = kt_first; kt < kt_stop; ++kt) {
      __syncthreads();  // everyone is done with the previous tile
      store_tile(0);
      __syncthreads();
      if (kt + 1 < kt_stop) ask_for(kt + 1);
      // the loads above are to be in flight during the arithmetic below, not sunk to their use
      __builtin_amdgcn_sched_barrier(0);
      if (busy(kt)) {
        floatx4 s4[4];
        bf16x8 pf[2];
        scores(0, s4);
        weights(s4, kt * BN, pf);
        values(0, pf);
      }
    }
  } else {
    // Three tiles in LDS, taking turns; one barrier a tile.  Tile kt + 2 goes from registers to LDS at the end of
    // iteration kt (into the place of tile kt - 1, which everyone left one barrier ago), and tile kt + 3 is
    // asked for behind the barrier.  A wave asks the matrix cores for the scores of tile kt + 1 BEFORE it turns
    // the scores of tile kt into weights: the workgroup's waves go through a tile in step (the barrier sees to
    // that), so without this all of them would keep the matrix cores busy and the vector units idle, then the
    // other way round; this way a wave's own exponentials run while its next scores are computed.
    static_assert(NB == 3, "three tiles");
    if (kt_first < kt_stop) {
      ask_for(kt_first);
      store_tile(0);
      if (kt_first + 1 < kt_stop) {
        ask_for(kt_first + 1);
        store_tile(1);
      }
      __syncthreads();
      if (kt_first + 2 < kt_stop) ask_for(kt_first + 2);
    }
    floatx4 s_a[4], s_b[4];
    auto step = [&](int kt, int buf, floatx4 (&s_cur)[4], floatx4 (&s_next)[4]) {
      const int next_buf = buf == 2 ? 0 : buf + 1, free_buf = buf == 0 ? 2 : buf - 1;
      __builtin_amdgcn_sched_barrier(0);   // (the loads asked for stay in flight during the arithmetic)
      if (kt + 1 < kt_stop && busy(kt + 1)) scores(next_buf, s_next);
      if (busy(kt)) {
        bf16x8 pf[2];
        weights(s_cur, kt * BN, pf);
        values(buf, pf);
      }
      if (kt + 2 < kt_stop) store_tile(free_buf);
      __syncthreads();
      if (kt + 3 < kt_stop) ask_for(kt + 3);
    };
    if (kt_first < kt_stop && busy(kt_first)) scores(0, s_a);
    int buf = 0;
    for (int kt = kt_first; kt < kt_stop; kt += 2) {
      step(kt, buf, s_a, s_b);
      buf = buf == 2 ? 0 : buf + 1;
      if (kt + 1 < kt_stop) {
        step(kt + 1, buf, s_b, s_a);
        buf = buf == 2 ? 0 : buf + 1;
      }
    }
  }

  // row sum over the 4 lanes that share the row; store d = t*16 + g*4 .. +4 of row lr
  l = row4_sum(l);
  const int row = wave * 16 + lr;
  if (a.n_splits > 1) {
    // (max of the scaled scores, sum, weighted values) of this slice; a slice without keys leaves a
    // maximum far below any score and zeros, which the merge weighs with exp(-huge) = 0
    if (row < rows_here) {
      float* ps = partial + (((size_t)(n0 + row) * a.nh + head) * a.n_splits + blockIdx.z) * (HD + 2);
      if (g == 0) {
        ps[0] = m * a.scale;
        ps[1] = l;
      }
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) ps[2 + t * 16 + g * 4 + i] = o[t][i];
    }
    return;
  }
  if (row < rows_here) {
    const float inv = 1.0f / l;
    bf16* dst = out + (size_t)(n0 + row) * a.ldo + (size_t)head * HD + g * 4;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
      const bf16x4 v = {(bf16)(o[t][0] * inv), (bf16)(o[t][1] * inv), (bf16)(o[t][2] * inv), (bf16)(o[t][3] * inv)};
      if (a.ldo % 4 == 0) {
        *(bf16x4*)(dst + t * 16) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[t * 16 + i] = v[i];
      }
    }
  }
}
template <int DT, int HPW>
void launch_prefill_heads(dim3 grid, hipStream_t stream, const bf16* q, const bf16* k, const bf16* v, bf16* out, float* partial,
                          const PrefillArgs& a) {
  grid.y = a.nh / HPW;
  if (a.page_shift >= 0) attention_prefill_kernel<DT, true, HPW><<<grid, 256 * HPW, 0, stream>>>(q, k, v, out, partial, a);
  else attention_prefill_kernel<DT, false, HPW><<<grid, 256 * HPW, 0, stream>>>(q, k, v, out, partial, a);
}
template <int DT>
void launch_prefill(dim3 grid, int heads_per_wg, hipStream_t stream, const bf16* q, const bf16* k, const bf16* v, bf16* out,
                    float* partial, const PrefillArgs& a) {
  if constexpr (DT <= 4) {   // (larger heads keep one head a workgroup: their registers leave no room for more waves)
    if (heads_per_wg == 4) return launch_prefill_heads<DT, 4>(grid, stream, q, k, v, out, partial, a);
    if (heads_per_wg == 2) return launch_prefill_heads<DT, 2>(grid, stream, q, k, v, out, partial, a);
  }
  launch_prefill_heads<DT, 1>(grid, stream, q, k, v, out, partial, a);
}

}  // namespace

// q: [N, >= nh*hd] bfloat16 (row stride ldq), rows of request r are cu[r] .. cu[r+1] at positions
// ctx[r] ..; pages: [num_pages, nkv, page_size, hd]; out: [N, nh*hd] (row stride ldo).
// n_splits > 1: the key tiles of every workgroup's rows are cut into that many slices; partial is a
// workspace of (first_row + n_rows) * nh * n_splits * (hd + 2) floats.  cu may start above 0 (the requests
// of a step from some request on): first_row = cu[0] then, and n_rows counts the rows from there.
// heads_per_wg: query heads of a kv head's group that a workgroup takes (1, 2 or 4; 0 counts as 1; the step's
// rule for it is gibbs_rule_prefill_heads).
GIBBS_EXPORT int gibbs_attention_prefill(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                                         const int* cu, const int* ctx, const int* table, int n_req, int max_pages,
                                         int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ldq,
                                         long ldo, float scale, int window, int n_splits, int first_row, int heads_per_wg,
                                         hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && n_req >= 0 && nh > 0 && nkv > 0, "attention_prefill: bad sizes rows=%d requests=%d heads=%d kv=%d", n_rows, n_req, nh, nkv);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_prefill: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 16 == 0 && hd >= 16 && hd <= 128, "attention_prefill: head size %d must be a multiple of 16 up to 128", hd);
  GIBBS_REQUIRE(ldq % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_prefill: q rows must be 16-byte aligned");
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention_prefill: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_prefill: bad cache geometry");
  GIBBS_REQUIRE(nh <= 65535, "attention_prefill: too many heads (%d)", nh);
  GIBBS_REQUIRE(first_row >= 0, "attention_prefill: negative first row");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_prefill: %d key slices need a workspace", n_splits);
  GIBBS_REQUIRE(heads_per_wg == 0 || ((heads_per_wg == 1 || heads_per_wg == 2 || heads_per_wg == 4) && (nh / nkv) % heads_per_wg == 0 && (heads_per_wg == 1 || hd <= 64)),
                "attention_prefill: %d heads a workgroup (1, 2 or 4 of a kv head's %d; more than one for head sizes up to 64)", heads_per_wg, nh / nkv);
  if (n_rows == 0 || n_req == 0) return 0;
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  PrefillArgs a{cu, ctx, table, n_req, max_pages, page_size, num_pages, page_shift, nh, nkv, hd, ldq, ldo, scale, window, n_splits};
  dim3 grid(ceil_div(n_rows, BM) + n_req, nh, n_splits);
  const bf16 *qq = (const bf16*)q, *kk = (const bf16*)kpages, *vv = (const bf16*)vpages;
  bf16* oo = (bf16*)out;
  switch (hd / 16) {
    case 1: launch_prefill<1>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 2: launch_prefill<2>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 3: launch_prefill<3>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 4: launch_prefill<4>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 5: launch_prefill<5>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 6: launch_prefill<6>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    case 7: launch_prefill<7>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
    default: launch_prefill<8>(grid, heads_per_wg, stream, qq, kk, vv, oo, partial, a); break;
  }
  if (n_splits > 1) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return gibbs_fail("attention_prefill: %s", hipGetErrorString(e));
    dim3 mgrid(n_rows, ceil_div(nh, 4));
    launch_attention_merge(mgrid, stream, partial + (size_t)first_row * nh * n_splits * (hd + 2), oo + (size_t)first_row * ldo,
                           nh, hd, n_splits, ldo);
  }
  GIBBS_LAUNCH_STATUS("attention_prefill");
}
