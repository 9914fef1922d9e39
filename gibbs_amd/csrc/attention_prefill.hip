// Paged causal attention for prompt portions on the gfx950 matrix cores (bfloat16 in, float32
// scores, maxima, sums and accumulators).
//
// A workgroup takes 64 consecutive query rows of one request and one query head; each of its 4
// waves owns 16 of the rows.  Keys are walked in tiles of 64 aligned to absolute key index (so a
// row's sequence of operations does not depend on how the prompt was cut).  Per tile:
//   K tile -> LDS as stored ([key][d]): it is the B operand of S = Q K^T as it lies
//   V tile -> LDS transposed ([d][key]): the B operand of O += P V must be contiguous along keys
//   S (16 x 64 per wave) = v_mfma_f32_16x16x32_bf16 over d;  scale, mask by position;
//   online softmax per row (row maxima by shuffles over the 16 lanes that share a row);
//   P -> bfloat16 -> the wave's LDS patch -> back as the A operand;  O += P V.
// Keys come from the request's pages through its block table; row n sees keys lo .. pos[n]
// (lo = max(0, pos - window + 1), window 0 = all).  The step's own keys were written to the pages
// before this kernel runs.  Head sizes: multiples of 16 up to 128.
#include "common.h"

namespace {
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int BM = 64;   // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int LDP = BN + 8;

struct PrefillArgs {
  const int* cu;
  const int* ctx;
  const int* table;
  int n_req, max_pages, page_size, num_pages;
  int nh, nkv, hd;
  long ldq, ldo;
  float scale;
  int window;
};

template <int DT>  // head size = 16 * DT
__global__ __launch_bounds__(256) void attention_prefill_kernel(const bf16* __restrict__ q,
                                                                const bf16* __restrict__ kpages,
                                                                const bf16* __restrict__ vpages, bf16* __restrict__ out,
                                                                PrefillArgs a) {
  constexpr int HD = 16 * DT;
  constexpr int DS = (DT + 1) / 2;  // steps of 32 over d
  constexpr int LDK = HD + 8;
  __shared__ bf16 sK[BN][LDK];
  __shared__ bf16 sVT[HD][LDP];
  __shared__ bf16 sP[4][16][LDP];

  // which request and which 64 rows of it
  int tile = blockIdx.x, r = 0, qlen = 0;
  for (; r < a.n_req; ++r) {
    qlen = a.cu[r + 1] - a.cu[r];
    const int t = (qlen + BM - 1) / BM;
    if (tile < t) break;
    tile -= t;
  }
  if (r >= a.n_req) return;
  const int head = blockIdx.y;
  const int kvh = head / (a.nh / a.nkv);
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int lr = lane % 16, g = lane / 16;
  const int row_in_req0 = tile * BM;                 // first row of the tile inside the request's rows
  const int n0 = a.cu[r] + row_in_req0;              // its index among the step's rows
  const int p0 = a.ctx[r] + row_in_req0;             // its absolute position
  const int rows_here = min(BM, qlen - row_in_req0);
  const int* table = a.table + (size_t)r * a.max_pages;

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
  // rows this lane owns in S and O: wave*16 + g*4 + i
  int pos_i[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) pos_i[i] = p0 + min(wave * 16 + g * 4 + i, rows_here - 1);

  float m[4], l[4];
  floatx4 o[DT];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m[i] = -INFINITY; l[i] = 0.f; }
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int last_pos = p0 + rows_here - 1;
  const int first_key = a.window > 0 ? max(0, p0 - a.window + 1) : 0;
  const int wave_last = p0 + min(wave * 16 + 15, rows_here - 1);
  const int wave_first_key = a.window > 0 ? max(0, p0 + wave * 16 - a.window + 1) : 0;

  for (int kt = first_key / BN; kt * BN <= last_pos; ++kt) {
    const int key0 = kt * BN;
    __syncthreads();  // everyone is done with the previous tile
    // K tile: 64 keys x HD, 16-byte chunks
    for (int c = tid; c < BN * (HD / 8); c += 256) {
      const int key = c / (HD / 8), d = (c % (HD / 8)) * 8;
      const int ak = key0 + key;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (ak <= last_pos) {
        int page = table[ak / a.page_size];
        page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);
        v = *(const uint4*)(kpages + (((size_t)page * a.nkv + kvh) * a.page_size + ak % a.page_size) * HD + d);
      }
      *(uint4*)&sK[key][d] = v;
    }
    // V tile transposed: a thread takes two neighbouring keys x 8 d and writes 8 packed pairs
    for (int c = tid; c < (BN / 2) * (HD / 8); c += 256) {
      const int kp = c % (BN / 2), d = (c / (BN / 2)) * 8;
      uint4 v0 = make_uint4(0, 0, 0, 0), v1 = v0;
      const int ak = key0 + 2 * kp;
      if (ak <= last_pos) {
        int page = table[ak / a.page_size];
        page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);
        v0 = *(const uint4*)(vpages + (((size_t)page * a.nkv + kvh) * a.page_size + ak % a.page_size) * HD + d);
      }
      if (ak + 1 <= last_pos) {
        int page = table[(ak + 1) / a.page_size];
        page = page < 0 ? 0 : (page >= a.num_pages ? a.num_pages - 1 : page);
        v1 = *(const uint4*)(vpages + (((size_t)page * a.nkv + kvh) * a.page_size + (ak + 1) % a.page_size) * HD + d);
      }
      const uint32_t w0[4] = {v0.x, v0.y, v0.z, v0.w}, w1[4] = {v1.x, v1.y, v1.z, v1.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // elements d+2j and d+2j+1 of both keys
        const uint32_t lo = (w0[j] & 0xffffu) | (w1[j] << 16);
        const uint32_t hi = (w0[j] >> 16) | (w1[j] & 0xffff0000u);
        *(uint32_t*)&sVT[d + 2 * j][2 * kp] = lo;
        *(uint32_t*)&sVT[d + 2 * j + 1][2 * kp] = hi;
      }
    }
    __syncthreads();
    // a wave whose rows see none of this tile's keys has nothing to do (it still takes part in the barriers)
    if (key0 > wave_last || key0 + BN <= wave_first_key) continue;

    // S = Q K^T: 4 sub-tiles of 16 keys
    floatx4 s4[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s4[c] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int d = s * 32 + g * 8;
        const bf16x8 kf = d < HD ? *(const bf16x8*)&sK[c * 16 + lr][d] : zero8;
        s4[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[s], kf, s4[c], 0, 0, 0);
      }
    }
    // scale, mask, row maxima: this lane holds S[row g*4+i][key c*16+lr]
    const bool need_mask = key0 + BN - 1 > p0 + wave * 16 || a.window > 0;
    float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int key = key0 + c * 16 + lr;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = s4[c][i] * a.scale;
        if (need_mask) {
          const bool vis = key <= pos_i[i] && (a.window == 0 || key > pos_i[i] - a.window);
          v = vis ? v : -INFINITY;
        }
        s4[c][i] = v;
        mx[i] = fmaxf(mx[i], v);
      }
    }
    float keep[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) mx[i] = fmaxf(mx[i], __shfl_xor(mx[i], off, WAVE));
      const float m_new = fmaxf(m[i], mx[i]);
      // a row that has seen no key yet keeps m = -inf: exp(-inf - -inf) must not be taken
      keep[i] = (m_new == -INFINITY) ? 1.f : __expf(m[i] - m_new);
      m[i] = m_new;
      l[i] *= keep[i];
    }
    // P = exp(S - m) -> bfloat16 -> the wave's patch of LDS
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = (m[i] == -INFINITY) ? 0.f : __expf(s4[c][i] - m[i]);
        l[i] += p;
        sP[wave][g * 4 + i][c * 16 + lr] = (bf16)p;
      }
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= keep[i];
    // the wave reads back what its own lanes wrote: LDS operations of a wave complete in order
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // O += P V: k runs over the 64 keys in 2 steps of 32
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const bf16x8 pf = *(const bf16x8*)&sP[wave][lr][kk * 32 + g * 8];
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const bf16x8 vf = *(const bf16x8*)&sVT[t * 16 + lr][kk * 32 + g * 8];
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[t], 0, 0, 0);
      }
    }
  }

  // row sums over the 16 lanes that share the rows; store
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) l[i] += __shfl_xor(l[i], off, WAVE);
    const int row = wave * 16 + g * 4 + i;
    if (row >= rows_here) continue;
    const float inv = 1.0f / l[i];
    bf16* dst = out + (size_t)(n0 + row) * a.ldo + (size_t)head * HD;
#pragma unroll
    for (int t = 0; t < DT; ++t) dst[t * 16 + lr] = (bf16)(o[t][i] * inv);
  }
}
}  // namespace

// q: [N, >= nh*hd] bfloat16 (row stride ldq), rows of request r are cu[r] .. cu[r+1] at positions
// ctx[r] ..; pages: [num_pages, nkv, page_size, hd]; out: [N, nh*hd] (row stride ldo).
GIBBS_EXPORT int gibbs_attention_prefill(const void* q, const void* kpages, const void* vpages, void* out,
                                         const int* cu, const int* ctx, const int* table, int n_req, int max_pages,
                                         int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ldq,
                                         long ldo, float scale, int window, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && n_req >= 0 && nh > 0 && nkv > 0, "attention_prefill: bad sizes rows=%d requests=%d heads=%d kv=%d", n_rows, n_req, nh, nkv);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_prefill: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 16 == 0 && hd >= 16 && hd <= 128, "attention_prefill: head size %d must be a multiple of 16 up to 128", hd);
  GIBBS_REQUIRE(ldq % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_prefill: q rows must be 16-byte aligned");
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention_prefill: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_prefill: bad cache geometry");
  GIBBS_REQUIRE(nh <= 65535, "attention_prefill: too many heads (%d)", nh);
  if (n_rows == 0 || n_req == 0) return 0;
  PrefillArgs a{cu, ctx, table, n_req, max_pages, page_size, num_pages, nh, nkv, hd, ldq, ldo, scale, window};
  dim3 grid(ceil_div(n_rows, BM) + n_req, nh);
  const bf16 *qq = (const bf16*)q, *kk = (const bf16*)kpages, *vv = (const bf16*)vpages;
  bf16* oo = (bf16*)out;
  switch (hd / 16) {
    case 1: attention_prefill_kernel<1><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 2: attention_prefill_kernel<2><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 3: attention_prefill_kernel<3><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 4: attention_prefill_kernel<4><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 5: attention_prefill_kernel<5><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 6: attention_prefill_kernel<6><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    case 7: attention_prefill_kernel<7><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
    default: attention_prefill_kernel<8><<<grid, 256, 0, stream>>>(qq, kk, vv, oo, a); break;
  }
  GIBBS_LAUNCH_STATUS("attention_prefill");
}
