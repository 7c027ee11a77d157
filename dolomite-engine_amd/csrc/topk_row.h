// Top-k of one row of router logits by one wavefront, and the fp32 softmax over the k winners
// (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:250-255, 338-344), shared by the stand-alone top-k kernel
// and the general fused router.  Tie rule: value descending, then expert index ascending; NaN is the largest
// value and -0.0 ties with +0.0.
#pragma once

#include "common.h"

// Order-preserving map float -> uint32 (larger float <=> larger key); NaN is the largest key and
// -0.0 is folded onto +0.0 so that it ties with it, as a floating-point comparison would.
__device__ __forceinline__ uint32_t ordered_key(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    uint32_t lo = __shfl_xor((uint32_t)v, off, MI_WAVE);
    uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off, MI_WAVE);
    uint64_t o = ((uint64_t)hi << 32) | lo;
    v = o > v ? o : v;
  }
  return v;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

// All 64 lanes call this for one row.  Lane l passes the values of experts l, l + 64, ... (VPL of them; entries
// at or beyond E are ignored).  A candidate is the 64-bit key (ordered(value) << 32) | ~expert, so a plain
// unsigned max implements the tie rule.  Round j finds the j-th winner with a butterfly max; the lane that owns
// it retires it.  Lane j keeps winner j, then lanes [0, k) do the softmax and write gates_row[j] / idx_row[j].
template <typename T, int VPL>
__device__ __forceinline__ void topk_softmax_row(const float (&vals)[VPL], int E, int k, T* __restrict__ gates_row,
                                                 int32_t* __restrict__ idx_row) {
  const int lane = threadIdx.x & 63;
  uint64_t keys[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = lane + i * 64;
    // 0 is below every real candidate (real keys have a non-zero low word)
    keys[i] = e < E ? (((uint64_t)ordered_key(vals[i]) << 32) | (uint32_t)(~(uint32_t)e)) : 0ull;
  }
  float my_val = 0.f;
  int my_idx = 0;
  for (int j = 0; j < k; ++j) {
    uint64_t best = 0ull;
#pragma unroll
    for (int i = 0; i < VPL; ++i) best = keys[i] > best ? keys[i] : best;
    best = wave_max_u64(best);
    const int e = (int)(~(uint32_t)best);
    // the owner retires the winner and publishes its value
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      if (keys[i] == best) {
        v = vals[i];
        keys[i] = 0ull;
      }
    }
    v = __shfl(v, e & 63, MI_WAVE);
    if (lane == j) {
      my_val = v;
      my_idx = e;
    }
  }
  // softmax over the k winners in fp32; winner 0 is the maximum
  const float vmax = __shfl(my_val, 0, MI_WAVE);
  const float p = (lane < k) ? expf(my_val - vmax) : 0.f;
  const float denom = wave_sum_f32(p);
  if (lane < k) {
    Elt<T>::store(gates_row + lane, p / denom);
    idx_row[lane] = my_idx;
  }
}

// ---- four rows per wavefront ------------------------------------------------------------------------------
// Up to 256 experts and k <= 16: a row belongs to 16 lanes, so a wavefront selects for four rows at once and every
// exchange between lanes is a DPP move inside a row of 16 (no LDS traffic; the one-row-per-wavefront form above
// spends its time in the 13 cross-lane permutes of every round).

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_row_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, false);
}

// maximum over the 16 lanes of a row: lanes i ^ 1 and i ^ 2 (quad permutes), then 7 - i inside the half row and
// 15 - i inside the row -- after every step all lanes of the span hold the span's maximum
__device__ __forceinline__ uint64_t row16_max_u64(uint64_t v) {
#define MI_ROW16_MAX_STEP(CTRL)                                                   \
  {                                                                               \
    const uint32_t lo = dpp_row_u32<CTRL>((uint32_t)v);                           \
    const uint32_t hi = dpp_row_u32<CTRL>((uint32_t)(v >> 32));                   \
    const uint64_t o = ((uint64_t)hi << 32) | lo;                                 \
    v = o > v ? o : v;                                                            \
  }
  MI_ROW16_MAX_STEP(0xB1)   // quad_perm [1, 0, 3, 2]
  MI_ROW16_MAX_STEP(0x4E)   // quad_perm [2, 3, 0, 1]
  MI_ROW16_MAX_STEP(0x141)  // row_half_mirror
  MI_ROW16_MAX_STEP(0x140)  // row_mirror
#undef MI_ROW16_MAX_STEP
  return v;
}

// sum over the 16 lanes of a row, added in the order of wave_sum_f32 (partners at distance 8, 4, 2, 1: after the
// step at distance d the values repeat with period d, so a rotation by d delivers the partner's value): with the
// terms of lanes >= 16 zero the two give the same bits
__device__ __forceinline__ float row16_sum_f32(float v) {
  v += __uint_as_float(dpp_row_u32<0x128>(__float_as_uint(v)));  // row_ror:8
  v += __uint_as_float(dpp_row_u32<0x124>(__float_as_uint(v)));  // row_ror:4
  v += __uint_as_float(dpp_row_u32<0x122>(__float_as_uint(v)));  // row_ror:2
  v += __uint_as_float(dpp_row_u32<0x121>(__float_as_uint(v)));  // row_ror:1
  return v;
}

// inverse of ordered_key (NaN comes back as the default NaN, -0.0 as +0.0: neither changes the softmax)
__device__ __forceinline__ float ordered_value(uint32_t key) {
  if (key == 0xffffffffu) return __uint_as_float(0x7fc00000u);
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// All 64 lanes call this; lane l works for the row of its 16-lane group, `row_ok` says whether that row exists.
// Lane j of a group (j = l % 16) passes the values of experts j, j + 16, ... (VPL of them; entries at or beyond E
// are ignored).  Same candidates, same tie rule and the same arithmetic as topk_softmax_row: the two write the
// same bits.  k <= 16.
template <typename T, int VPL>
__device__ __forceinline__ void topk_softmax_row16(const float (&vals)[VPL], int E, int k, bool row_ok,
                                                   T* __restrict__ gates_row, int32_t* __restrict__ idx_row) {
  const int j16 = threadIdx.x & 15;
  uint64_t keys[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = j16 + i * 16;
    keys[i] = e < E ? (((uint64_t)ordered_key(vals[i]) << 32) | (uint32_t)(~(uint32_t)e)) : 0ull;
  }
  float my_val = 0.f, vmax = 0.f;
  int my_idx = 0;
  for (int j = 0; j < k; ++j) {
    uint64_t best = 0ull;
#pragma unroll
    for (int i = 0; i < VPL; ++i) best = keys[i] > best ? keys[i] : best;
    best = row16_max_u64(best);
#pragma unroll
    for (int i = 0; i < VPL; ++i) keys[i] = keys[i] == best ? 0ull : keys[i];  // the owner retires the winner
    const float v = ordered_value((uint32_t)(best >> 32));
    if (j == 0) vmax = v;
    if (j16 == j) {
      my_val = v;
      my_idx = (int)(~(uint32_t)best);
    }
  }
  const float p = (j16 < k) ? expf(my_val - vmax) : 0.f;
  const float denom = row16_sum_f32(p);
  if (row_ok && j16 < k) {
    Elt<T>::store(gates_row + j16, p / denom);
    idx_row[j16] = my_idx;
  }
}

