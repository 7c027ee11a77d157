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
