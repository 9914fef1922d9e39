// Helpers for kernels in which a lane holds 8 consecutive bfloat16 elements (16 bytes) of a head
// and LPK neighbouring lanes hold the head: sums over the lane group, per-head RMSNorm and rotary
// position encoding in that layout.
#pragma once
#include "common.h"

constexpr int EPL = 8;  // head-dim elements per lane (16 bytes of bfloat16)

// Cosine and sine of a rotation angle: the one place that computes them, so that the table and
// every kernel that rotates beyond the table agree to the bit.
__device__ __forceinline__ void rope_cos_sin(float angle, float* c, float* s) {
  *c = cosf(angle);
  *s = sinf(angle);
}

__device__ __forceinline__ void unpack8(const uint4& raw, float* f) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

__device__ __forceinline__ uint4 pack8(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16 lo = (bf16)f[2 * i], hi = (bf16)f[2 * i + 1];
    w[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Sum over the LPK neighbouring lanes that share a key, every one of them getting the total.
// Data-parallel-primitive moves (a few cycles each) instead of LDS permutes (tens of cycles each,
// and this sum sits on the critical path of every key): swap within pairs, within quads, then
// mirror the half row (lane i <-> 7 - i: the other quad) and the row (i <-> 15 - i: the other half).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
  if (LPK >= 2) v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  if (LPK >= 4) v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  if (LPK >= 8) v += dpp_move<0x141>(v);  // row_half_mirror
  if (LPK >= 16) v += dpp_move<0x140>(v); // row_mirror
  if (LPK >= 32) v += __shfl_xor(v, 16, WAVE);
  return v;
}

// Rotation factors of this lane's 8 elements at position `pos` (the same for every head).
struct Rot8 {
  float c[EPL], s[EPL];
};

// `table`: (cos, sin) of positions 0 .. table_len-1, [table_len, rot/2], made by rope_table from the
// same float32 angles with the same functions; later positions are computed here.
__device__ __forceinline__ Rot8 rotation8(int e0, const float* inv_freq, int rot, int variant, int pos,
                                          const float2* table, int table_len) {
  Rot8 r;
  const int half = rot / 2;
  const bool tabled = table && pos < table_len;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = e0 + i;
    r.c[i] = 1.f;
    r.s[i] = 0.f;
    if (inv_freq && e < rot) {
      const int j = variant == 1 ? e / 2 : (e < half ? e : e - half);
      if (tabled) {
        const float2 cs = table[(size_t)pos * half + j];
        r.c[i] = cs.x;
        r.s[i] = cs.y;
      } else {
        rope_cos_sin((float)pos * inv_freq[j], &r.c[i], &r.s[i]);
      }
    }
  }
  return r;
}

// Norm (optional) and rotation of one head held 8 elements per lane by LPK neighbouring lanes.
// `v` are this lane's elements e0 .. e0+7 of the head; returns them normed and rotated.
// `gain8`: the norm's gain for this lane's elements, already in registers (a caller that norms several heads
// reads it once); `normed` false: no norm.
template <int LPK>
__device__ __forceinline__ void norm_rope8_with(float* v, int e0, int hd, bool normed, const float* gain8, float eps,
                                                bool rotate, const Rot8& rt, int rot, int variant, int lane) {
  const bool active = e0 < hd;
  if (normed) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) ss += v[i] * v[i];
    ss = group_sum<LPK>(ss);
    const float sc = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
    for (int i = 0; i < EPL; ++i) v[i] = active ? v[i] * sc * gain8[i] : 0.f;
  }
  if (!rotate) return;
  const int half = rot / 2;
  if (variant == 1) {  // pairs (2j, 2j+1) lie in one lane
#pragma unroll
    for (int i = 0; i < EPL; i += 2) {
      if (e0 + i + 1 < rot) {
        const float x0 = v[i], x1 = v[i + 1];
        v[i] = x0 * rt.c[i] - x1 * rt.s[i];
        v[i + 1] = x0 * rt.s[i] + x1 * rt.c[i];
      }
    }
    return;
  }
  // half split: element e pairs with e + half (e < half) or e - half; the partner lies half/8 lanes away
  const int shift = half / EPL;  // half is a multiple of 8 (rotary sizes in steps of 16)
  const int base = lane - lane % LPK;
  const int sub = lane % LPK;
  const bool low = e0 < half;
  const int partner = base + (low ? sub + shift : sub - shift);
  const int src = (partner >= base && partner < base + LPK) ? partner : lane;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const float other = __shfl(v[i], src, WAVE);
    if (e0 + i < rot) v[i] = low ? v[i] * rt.c[i] - other * rt.s[i] : other * rt.s[i] + v[i] * rt.c[i];
  }
}

// The same with the gain read here (null: no norm).
template <int LPK>
__device__ __forceinline__ void norm_rope8(float* v, int e0, int hd, const float* gain, float eps, bool rotate,
                                           const Rot8& rt, int rot, int variant, int lane) {
  float gain8[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) gain8[i] = (gain && e0 < hd) ? gain[e0 + i] : 1.f;
  norm_rope8_with<LPK>(v, e0, hd, gain != nullptr, gain8, eps, rotate, rt, rot, variant, lane);
}
