// Per-token-group quantisation body shared by the stand-alone quant kernels and the fused-MoE
// prologue kernel (which quantises the hidden states in the same launch that sorts the tokens).
#pragma once
#include "common.h"

namespace sglamd {

// ceil(log2(x)) for a positive normal float, from its bit pattern.
__device__ __forceinline__ int log2_ceil_bits(float x) {
  uint32_t b = __float_as_uint(x);
  int e = (int)((b >> 23) & 0xff);
  return e - 127 + ((b & 0x7fffffu) != 0);
}
__device__ __forceinline__ float pow2_int(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }

template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

struct GroupQuantArgs {
  const void* in;
  void* q;
  void* s;
  int64_t num_groups;      // rows * groups_per_row
  int groups_per_row;
  int layout;
  int64_t scale_stride;
  float eps, min8, max8;
  int form;
  int q_is_fp8;
  int fuse_silu_mul;       // input rows are [gate | up] of 2*hidden; x = T(silu(gate)) * up
  int64_t hidden;          // output elements per row (used by the fused variant)
  // masked (DeepEP) layout: rows are [expert][token]; only tokens < masked_m[expert] are quantised, and the
  // UE8M0 scale words of expert e start scale_expert_stride int32 words after those of expert e-1
  const int32_t* masked_m;
  int tokens_per_expert;
  int64_t scale_expert_stride;
};

// T: input storage tag; GROUP: elements per group.  ELEMS elements per lane (32 bytes),
// LPG = GROUP / ELEMS lanes share a group.
template <typename T, int GROUP>
__device__ __forceinline__ void group_quant_body(const GroupQuantArgs& a, const int64_t lane_global) {
  typedef typename T::storage S;
  constexpr int ELEMS = 32 / (int)sizeof(S);
  constexpr int LPG = GROUP / ELEMS;
  static_assert(LPG >= 1 && LPG <= 64 && (LPG & (LPG - 1)) == 0, "group must span 1..64 lanes");

  const int64_t g = lane_global / LPG;
  const int sub = (int)(lane_global % LPG);
  bool active = g < a.num_groups;
  if (a.masked_m && active) {
    const int64_t r = g / a.groups_per_row;
    active = (int)(r % a.tokens_per_expert) < a.masked_m[r / a.tokens_per_expert];
  }
  // Lanes past the end keep running (they take part in the cross-lane max) on group 0's
  // address range but store nothing.
  const int64_t gg = active ? g : 0;

  float x[ELEMS];
  float amax = a.eps;
  if (!a.fuse_silu_mul) {
    const S* src = (const S*)a.in + gg * GROUP + sub * ELEMS;
    v4i raw0 = *(const v4i*)src;
    v4i raw1 = *((const v4i*)src + 1);
    S buf[ELEMS];
    __builtin_memcpy(&buf[0], &raw0, 16);
    __builtin_memcpy(&buf[ELEMS / 2], &raw1, 16);
#pragma unroll
    for (int i = 0; i < ELEMS; i++) x[i] = T::to_f32(buf[i]);
  } else {
    // gate and up halves of one [2*hidden] row; silu is rounded to T, the product is rounded to T
    const int64_t row = gg / a.groups_per_row;
    const int64_t col = (gg % a.groups_per_row) * GROUP + sub * ELEMS;
    const S* gsrc = (const S*)a.in + row * 2 * a.hidden + col;
    const S* usrc = gsrc + a.hidden;
    v4i g0 = *(const v4i*)gsrc, g1 = *((const v4i*)gsrc + 1);
    v4i u0 = *(const v4i*)usrc, u1 = *((const v4i*)usrc + 1);
    S gb[ELEMS], ub[ELEMS];
    __builtin_memcpy(&gb[0], &g0, 16);
    __builtin_memcpy(&gb[ELEMS / 2], &g1, 16);
    __builtin_memcpy(&ub[0], &u0, 16);
    __builtin_memcpy(&ub[ELEMS / 2], &u1, 16);
#pragma unroll
    for (int i = 0; i < ELEMS; i++) {
      const float gv = T::to_f32(gb[i]);
      const float sv = T::to_f32(T::from_f32(gv / (1.0f + expf(-gv))));
      x[i] = T::to_f32(T::from_f32(sv * T::to_f32(ub[i])));
    }
  }
#pragma unroll
  for (int i = 0; i < ELEMS; i++) amax = fmaxf(amax, fabsf(x[i]));
  amax = group_max<LPG>(amax);

  const bool ue8m0 = a.layout == SGLAMD_SCALE_COL_MAJOR_UE8M0;
  float s_store;   // value written as the scale (or whose exponent byte is written)
  float mul = 0.f; // reciprocal form: multiplier applied to x
  if (a.form == SGLAMD_QUANT_FORM_DIVIDE) {
    s_store = amax / a.max8;
    if (ue8m0) s_store = pow2_int(log2_ceil_bits(fmaxf(s_store, 1e-10f)));
  } else {
    if (ue8m0) {
      int e = log2_ceil_bits(amax * (1.0f / a.max8));
      mul = pow2_int(-e);
      s_store = pow2_int(e);
    } else {
      s_store = amax * (1.0f / a.max8);
      mul = a.max8 / amax;
    }
  }

  float y[ELEMS];
  if (a.form == SGLAMD_QUANT_FORM_DIVIDE) {
#pragma unroll
    for (int i = 0; i < ELEMS; i++) y[i] = clampf(x[i] / s_store, a.min8, a.max8);
  } else {
#pragma unroll
    for (int i = 0; i < ELEMS; i++) y[i] = clampf(x[i] * mul, a.min8, a.max8);
  }

  if (!active) return;

  uint8_t* dst = (uint8_t*)a.q + gg * GROUP + sub * ELEMS;
  uint32_t w[ELEMS / 4];
  if (a.q_is_fp8) {
#pragma unroll
    for (int i = 0; i < ELEMS / 4; i++) w[i] = pack4_e4m3(y[4 * i], y[4 * i + 1], y[4 * i + 2], y[4 * i + 3]);
  } else {
#pragma unroll
    for (int i = 0; i < ELEMS / 4; i++) {
      uint32_t b0 = (uint32_t)(int)y[4 * i] & 0xff, b1 = (uint32_t)(int)y[4 * i + 1] & 0xff;
      uint32_t b2 = (uint32_t)(int)y[4 * i + 2] & 0xff, b3 = (uint32_t)(int)y[4 * i + 3] & 0xff;
      w[i] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    }
  }
  if constexpr (ELEMS == 16) {
    v4i o = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    *(v4i*)dst = o;
  } else {
    v2i o = {(int)w[0], (int)w[1]};
    *(v2i*)dst = o;
  }

  if (sub == 0) {
    const int64_t row = gg / a.groups_per_row;
    const int col = (int)(gg % a.groups_per_row);
    if (a.layout == SGLAMD_SCALE_ROW_MAJOR) {
      ((float*)a.s)[gg] = s_store;
    } else if (a.layout == SGLAMD_SCALE_COL_MAJOR) {
      ((float*)a.s)[(int64_t)col * a.scale_stride + row] = s_store;
    } else {
      int64_t word = (int64_t)(col >> 2) * a.scale_stride + row;
      if (a.masked_m)
        word = (row / a.tokens_per_expert) * a.scale_expert_stride + (int64_t)(col >> 2) * a.scale_stride +
               row % a.tokens_per_expert;
      uint8_t* sp = (uint8_t*)a.s + (word << 2);
      sp[col & 3] = (uint8_t)(__float_as_uint(s_store) >> 23);
      if (col == a.groups_per_row - 1) {
        for (int k = (col & 3) + 1; k < 4; k++) sp[k] = 0;
      }
    }
  }
}

}  // namespace sglamd
