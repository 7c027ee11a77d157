// General form of the fused router and the element-wise part of its backward.
//
// mi_moe_router_fused's streaming kernels (router_fused.hip) are built around 16-bit logits and at most 64
// experts.  This file covers what they do not: fp32 -- the dtype of the reference's own correctness
// configuration -- and 65 .. 256 experts or k up to 64, so that MoE._compute_routing_weights
// (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:246-257) never needs a library GEMM for its logits.
//
//   router_general_kernel    one workgroup per 16 tokens: the four waves split the contraction, partial logits
//                            meet in LDS in a fixed order, then one wave per token row runs the shared top-k
//                            (topk_row.h: value descending, expert index ascending) and the fp32 softmax
//   router_dlogits_kernel    gradient of the router's outputs w.r.t. the (T, E) logits: the softmax over the k
//                            picked logits backwards, scattered to the picked experts, plus the gradient that
//                            arrives at the logits themselves (the auxiliary loss).  The two products that follow
//                            (d x = d logits @ W_gate, d W_gate = d logits^T @ x) are the grouped GEMM and the
//                            grouped weight-gradient kernel run with one expert that owns every row.
#include "common.h"
#include "topk_row.h"

template <typename T> struct GMfma;
template <> struct GMfma<bf16_t> {
  static constexpr int KSTEP = 64;  // contraction elements per step and wave: 16 per lane group
  static __device__ __forceinline__ void run(const u32x4 (&w)[2], const u32x4 (&x)[2], f32x4& acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[0]), __builtin_bit_cast(bf16x8, x[0]), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[1]), __builtin_bit_cast(bf16x8, x[1]), acc, 0, 0, 0);
  }
};
template <> struct GMfma<f16_t> {
  static constexpr int KSTEP = 64;
  static __device__ __forceinline__ void run(const u32x4 (&w)[2], const u32x4 (&x)[2], f32x4& acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w[0]), __builtin_bit_cast(f16x8, x[0]), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w[1]), __builtin_bit_cast(f16x8, x[1]), acc, 0, 0, 0);
  }
};
// fp32: a lane holds 8 consecutive k; instruction i (16x16x4) takes element i of both operands, so its four k
// slots (the lane groups) are four different k -- any assignment works as long as both operands use the same one
template <> struct GMfma<float> {
  static constexpr int KSTEP = 32;
  static __device__ __forceinline__ void run(const u32x4 (&w)[2], const u32x4 (&x)[2], f32x4& acc) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(w[h][i]), __uint_as_float(x[h][i]), acc, 0, 0, 0);
  }
};

#define ROUTER_GENERAL_MAX_E 256
#define ROUTER_GENERAL_MAX_K 64

// The tail both forms of the general kernel share.  Lane (r, q) of the wave that owns expert block eb holds the
// fp32 sums of token r, experts 16 * eb + 4 * q + i: round to the model dtype, add the bias and round again, keep
// the logit as fp32 in lg[token][expert] for the selection and write it out if the caller wants the logits.
template <typename T, int EP>
__device__ __forceinline__ void general_store_logits(const f32x4& sum, int eb, int r, int q, int tok0, int Trows, int E,
                                                     const float* __restrict__ bias, float* __restrict__ lg,
                                                     T* __restrict__ logits_out) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = eb * 16 + 4 * q + i;
    float v = Elt<T>::round(sum[i]);
    if (e < E) {
      if (bias != nullptr) v = Elt<T>::round(v + bias[e]);
      lg[r * EP + e] = v;
      if (logits_out != nullptr && tok0 + r < Trows) Elt<T>::store(logits_out + (size_t)(tok0 + r) * E + e, v);
    }
  }
}

// top-k and softmax: wave w takes tokens 4 w .. 4 w + 3 -- all four at once, 16 lanes per token, where k allows
// it, else one after the other with lane l on the experts l, l + 64, ...
template <typename T, int NEB>
__device__ __forceinline__ void general_topk(const float* __restrict__ lg, int wave, int r, int q, int tok0, int Trows,
                                             int E, int k, T* __restrict__ gates, int32_t* __restrict__ idx) {
  constexpr int EP = 16 * NEB;
  constexpr int VPL = (NEB + 3) / 4;  // candidates per lane with one row per wave
  if (k <= 16) {
    const int row = wave * 4 + q;
    const bool row_ok = tok0 + row < Trows;
    float vals[NEB];
#pragma unroll
    for (int c = 0; c < NEB; ++c) {
      const int e = r + c * 16;
      vals[c] = e < E ? lg[row * EP + e] : 0.f;
    }
    const size_t trow = row_ok ? (size_t)(tok0 + row) : (size_t)(Trows - 1);
    topk_softmax_row16<T, NEB>(vals, E, k, row_ok, gates + trow * k, idx + trow * k);
    return;
  }
  const int lane = q * 16 + r;
  for (int i = 0; i < 4; ++i) {
    const int row = wave * 4 + i;
    if (tok0 + row >= Trows) break;  // (wave-uniform)
    float vals[VPL];
#pragma unroll
    for (int c = 0; c < VPL; ++c) {
      const int e = lane + c * 64;
      vals[c] = e < E ? lg[row * EP + e] : 0.f;
    }
    topk_softmax_row<T, VPL>(vals, E, k, gates + (size_t)(tok0 + row) * k, idx + (size_t)(tok0 + row) * k);
  }
}

// NEB: expert blocks of 16 (E <= 16 * NEB).  LDS: [4 waves][NEB][64 lanes] partial accumulators, then
// [16 tokens][16 * NEB] logits as fp32.
// SPLIT (few tokens, with the caller's workspace): blockIdx.y cuts the contraction into ranges of `steps_per_split`
// steps; a workgroup adds up its range as below and writes the 16 x EP sums raw, [group][split][block][lane], and
// router_general_finish_kernel adds a group's ranges in order and does the rest.  One workgroup per 16 tokens
// alone leaves a decode batch on a handful of CUs, each pulling all gate weights through its four waves.
template <typename T, int NEB, bool SPLIT>
__global__ __launch_bounds__(256) void router_general_kernel(const T* __restrict__ x, const T* __restrict__ gw,
                                                             const float* __restrict__ bias, int Trows, int H, int E,
                                                             int k, T* __restrict__ logits_out, T* __restrict__ gates,
                                                             int32_t* __restrict__ idx, f32x4* __restrict__ partial,
                                                             int steps_per_split) {
  constexpr int KSTEP = GMfma<T>::KSTEP;
  constexpr int LPL = KSTEP / 4;                   // elements per lane and step (two 16-byte loads)
  constexpr int HALF = LPL / 2;
  constexpr int EP = 16 * NEB;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  f32x4* red = reinterpret_cast<f32x4*>(smem_raw);                    // [4][NEB][64]
  float* lg = reinterpret_cast<float*>(smem_raw + 4 * NEB * 64 * 16);  // [16][EP]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tok0 = blockIdx.x * 16;
  int t = tok0 + r;
  if (t > Trows - 1) t = Trows - 1;
  const T* xrow = x + (size_t)t * H;

  f32x4 acc[NEB];
#pragma unroll
  for (int eb = 0; eb < NEB; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int neb = (E + 15) >> 4;
  // wave w takes the steps first + w, first + w + 4, ... of the workgroup's range (all of them without SPLIT)
  const int nsteps = (H + KSTEP - 1) / KSTEP;
  const int first = SPLIT ? (int)blockIdx.y * steps_per_split : 0;
  const int last = SPLIT ? (first + steps_per_split < nsteps ? first + steps_per_split : nsteps) : nsteps;
  for (int st = first + wave; st < last; st += 4) {
    const int k0 = st * KSTEP;
    const int kpos = k0 + q * LPL;
    const bool valid = kpos < H;  // the matrix instruction runs on all lanes: out-of-range k contributes zeros
    u32x4 xa[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    if (valid) {
      xa[0] = *reinterpret_cast<const u32x4*>(xrow + kpos);
      xa[1] = *reinterpret_cast<const u32x4*>(xrow + kpos + HALF);
    }
#pragma unroll
    for (int eb = 0; eb < NEB; ++eb) {
      if (eb < neb) {
        int e = eb * 16 + r;
        if (e > E - 1) e = E - 1;  // surplus rows of the last block re-read the last expert; never used
        u32x4 wa[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if (valid) {
          const T* wrow = gw + (size_t)e * H + kpos;
          wa[0] = *reinterpret_cast<const u32x4*>(wrow);
          wa[1] = *reinterpret_cast<const u32x4*>(wrow + HALF);
        }
        GMfma<T>::run(wa, xa, acc[eb]);
      }
    }
  }
#pragma unroll
  for (int eb = 0; eb < NEB; ++eb) red[(wave * NEB + eb) * 64 + lane] = acc[eb];
  __syncthreads();
  // wave w adds up the blocks w, w + 4, ... in wave order (the logits do not depend on scheduling); lane (r, q)
  // holds token r, experts 16 * eb + 4 * q + i
#pragma unroll
  for (int eb0 = 0; eb0 < NEB; eb0 += 4) {
    const int eb = eb0 + wave;
    if (eb < NEB && eb < neb) {
      f32x4 sum = red[eb * 64 + lane];
#pragma unroll
      for (int w = 1; w < 4; ++w) sum += red[(w * NEB + eb) * 64 + lane];
      if constexpr (SPLIT) {
        partial[(((size_t)blockIdx.x * gridDim.y + blockIdx.y) * NEB + eb) * 64 + lane] = sum;
      } else {
        general_store_logits<T, EP>(sum, eb, r, q, tok0, Trows, E, bias, lg, logits_out);
      }
    }
  }
  if constexpr (SPLIT) return;
  __syncthreads();
  general_topk<T, NEB>(lg, wave, r, q, tok0, Trows, E, k, gates, idx);
}

// Second launch of the SPLIT form: one workgroup per 16 tokens adds the ranges' sums in range order, then rounds,
// adds the bias, writes the logits and selects exactly as the single launch does.
template <typename T, int NEB>
__global__ __launch_bounds__(256) void router_general_finish_kernel(const f32x4* __restrict__ partial, int splits,
                                                                    const float* __restrict__ bias, int Trows, int E,
                                                                    int k, T* __restrict__ logits_out,
                                                                    T* __restrict__ gates, int32_t* __restrict__ idx) {
  constexpr int EP = 16 * NEB;
  __shared__ float lg[16 * EP];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tok0 = blockIdx.x * 16;
  const int neb = (E + 15) >> 4;
#pragma unroll
  for (int eb0 = 0; eb0 < NEB; eb0 += 4) {
    const int eb = eb0 + wave;
    if (eb < NEB && eb < neb) {
      const f32x4* src = partial + ((size_t)blockIdx.x * splits * NEB + eb) * 64 + lane;
      // eight ranges' loads in flight at a time (the additions stay in range order)
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
      for (int sp0 = 0; sp0 < splits; sp0 += 8) {
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[j] = sp0 + j < splits ? src[(size_t)(sp0 + j) * NEB * 64] : (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (sp0 + j < splits) sum += v[j];
      }
      general_store_logits<T, EP>(sum, eb, r, q, tok0, Trows, E, bias, lg, logits_out);
    }
  }
  __syncthreads();
  general_topk<T, NEB>(lg, wave, r, q, tok0, Trows, E, k, gates, idx);
}

// Ranges of the contraction for few tokens: enough workgroups for about two per CU, a step per wave at least.
static int router_general_splits(int T_, int H, int dtype) {
  const int kstep = dtype == MI_MOE_F32 ? 32 : 64;
  const int nsteps = mi_ceil_div(H, kstep);
  if (T_ < 1) return 1;
  const int groups = mi_ceil_div(T_, 16);
  int splits = mi_ceil_div(512, groups);
  if (splits > nsteps / 4) splits = nsteps / 4;
  return splits < 2 ? 1 : splits;
}
// partial sums of the SPLIT form: [group][split][block of 16 experts][lane] f32x4, for the most ranges any dtype takes
size_t mi_router_general_ws_bytes(int T_, int H, int E) {
  if (E <= 64) return 0;  // (up to 64 experts the general kernel serves fp32 and large k only: one launch)
  const int splits = router_general_splits(T_, H, MI_MOE_F32);
  if (splits < 2) return 0;
  const int neb = E <= 128 ? 8 : 16;
  return (size_t)mi_ceil_div(T_, 16) * splits * neb * 64 * sizeof(f32x4);
}

template <typename T, int NEB>
static int launch_router_general(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                 void* logits_out, void* gates, int32_t* idx, void* ws, int splits, hipStream_t s) {
  constexpr size_t lds = (size_t)4 * NEB * 64 * 16 + (size_t)16 * 16 * NEB * 4;
  const int groups = mi_ceil_div(T_, 16);
  if (splits >= 2) {
    auto kern = router_general_kernel<T, NEB, true>;
    if (lds > 64 * 1024) {
      static std::atomic<uint64_t> lds_ok{0};
      const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok);
      if (rc != MI_MOE_OK) return rc;
    }
    const int nsteps = mi_ceil_div(H, GMfma<T>::KSTEP);
    const int sps = mi_ceil_div(nsteps, splits);
    const int used = mi_ceil_div(nsteps, sps);  // every range has a step
    hipLaunchKernelGGL(kern, dim3(groups, used), dim3(256), lds, s, static_cast<const T*>(x), static_cast<const T*>(gw),
                       bias, T_, H, E, k, static_cast<T*>(logits_out), static_cast<T*>(gates), idx,
                       static_cast<f32x4*>(ws), sps);
    hipLaunchKernelGGL((router_general_finish_kernel<T, NEB>), dim3(groups), dim3(256), 0, s,
                       static_cast<const f32x4*>(ws), used, bias, T_, E, k, static_cast<T*>(logits_out),
                       static_cast<T*>(gates), idx);
    return mi_launch_status();
  }
  auto kern = router_general_kernel<T, NEB, false>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_ok{0};
    const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok);
    if (rc != MI_MOE_OK) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(groups), dim3(256), lds, s, static_cast<const T*>(x),
                     static_cast<const T*>(gw), bias, T_, H, E, k, static_cast<T*>(logits_out),
                     static_cast<T*>(gates), idx, static_cast<f32x4*>(nullptr), 0);
  return mi_launch_status();
}

template <typename T>
static int router_general_by_blocks(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                    void* logits_out, void* gates, int32_t* idx, void* ws, int splits, hipStream_t s) {
  if (E <= 64) return launch_router_general<T, 4>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
  if (E <= 128) return launch_router_general<T, 8>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
  return launch_router_general<T, 16>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
}

// Shapes the general kernel takes: whole 16-byte pieces per lane and step.
int mi_router_general_ok(int H, int E, int k, int dtype) {
  if (E < 1 || E > ROUTER_GENERAL_MAX_E || k < 1 || k > ROUTER_GENERAL_MAX_K || k > E) return 0;
  if (dtype == MI_MOE_F32) return H % 8 == 0;
  return (dtype == MI_MOE_BF16 || dtype == MI_MOE_F16) && H % 16 == 0;
}

// Called by mi_moe_router_fused (router_fused.hip) for what its streaming kernels do not take; arguments are
// validated there.  `ws` (or null) holds mi_router_general_ws_bytes(T, H, E) bytes: with more than 64 experts and
// few tokens the contraction is then cut into ranges over many workgroups.
int mi_router_general(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k, int dtype,
                      void* logits_out, void* gates, int32_t* idx, void* ws, hipStream_t s) {
  const int splits = (ws != nullptr && E > 64) ? router_general_splits(T_, H, dtype) : 1;
  switch (dtype) {
    case MI_MOE_F32:
      return router_general_by_blocks<float>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
    case MI_MOE_F16:
      return router_general_by_blocks<f16_t>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
    case MI_MOE_BF16:
      return router_general_by_blocks<bf16_t>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, ws, splits, s);
    default: return MI_MOE_EDTYPE;
  }
}

// ------------------------------------------------------------------------------------------------
// backward: d logits
// ------------------------------------------------------------------------------------------------
//
// gates[t, j] = softmax_j(logits[t, idx[t, j]]) in fp32, rounded to the model dtype (moe.py:250-255).  With
// g = d loss / d gates and p the fp32 softmax of the picked logits,
//     d picked_j = p_j * (g_j - sum_i p_i g_i),
// rounded to the model dtype like autograd's cast back, scattered to expert idx[t, j] of a zero (T, E) row and
// added to the gradient `extra` that reaches the logits directly (the auxiliary loss), with one more rounding --
// the sequence of roundings autograd goes through on the eager branch.  One wave per token row.
template <typename T>
__global__ __launch_bounds__(256) void router_dlogits_kernel(const T* __restrict__ logits, const int32_t* __restrict__ idx,
                                                             const T* __restrict__ d_gates, const T* __restrict__ extra,
                                                             int Trows, int E, int k, T* __restrict__ d_logits) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= Trows) return;
  const T* lrow = logits + (size_t)row * E;
  T* drow = d_logits + (size_t)row * E;
  // picked logit, its expert and the incoming gradient of slot j = lane (k <= 64)
  int e_j = 0;
  float z = -INFINITY, g = 0.f;
  if (lane < k) {
    e_j = idx[(size_t)row * k + lane];
    z = Elt<T>::load(lrow + e_j);
    g = d_gates != nullptr ? Elt<T>::load(d_gates + (size_t)row * k + lane) : 0.f;
  }
  float zmax = z;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) zmax = fmaxf(zmax, __shfl_xor(zmax, off, MI_WAVE));
  float p = lane < k ? expf(z - zmax) : 0.f;
  p /= wave_sum_f32(p);
  const float dot = wave_sum_f32(p * g);
  const float dz = Elt<T>::round(p * (g - dot));
  // every entry of the row has one writer: lane l owns experts l, l + 64, ... and looks its experts up among the
  // k picked ones (a token's k experts are distinct)
  for (int e = lane; e - lane < E; e += 64) {
    const bool in_row = e < E;
    const float base = (in_row && extra != nullptr) ? Elt<T>::load(extra + (size_t)row * E + e) : 0.f;
    float val = base;
    if (d_gates != nullptr) {
      for (int j = 0; j < k; ++j) {
        const int ej = __shfl(e_j, j, MI_WAVE);
        const float dzj = __shfl(dz, j, MI_WAVE);
        if (ej == e) val = extra != nullptr ? Elt<T>::round(dzj + base) : dzj;
      }
    }
    if (in_row) Elt<T>::store(drow + e, val);
  }
}

extern "C" int mi_moe_router_dlogits(const void* logits, const int32_t* idx, const void* d_gates, const void* d_logits_extra,
                                     int T, int E, int k, int dtype, void* d_logits_out, mi_moe_stream_t stream) {
  if (T < 0 || E < 1 || k < 1 || k > E || k > ROUTER_GENERAL_MAX_K) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_F32 && dtype != MI_MOE_F16 && dtype != MI_MOE_BF16) return MI_MOE_EDTYPE;
  if (T == 0) return MI_MOE_OK;
  if (!logits || !idx || !d_logits_out) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(mi_ceil_div(T, 4)), block(256);
  switch (dtype) {
    case MI_MOE_F32:
      hipLaunchKernelGGL((router_dlogits_kernel<float>), grid, block, 0, s, static_cast<const float*>(logits), idx,
                         static_cast<const float*>(d_gates), static_cast<const float*>(d_logits_extra), T, E, k,
                         static_cast<float*>(d_logits_out));
      break;
    case MI_MOE_F16:
      hipLaunchKernelGGL((router_dlogits_kernel<f16_t>), grid, block, 0, s, static_cast<const f16_t*>(logits), idx,
                         static_cast<const f16_t*>(d_gates), static_cast<const f16_t*>(d_logits_extra), T, E, k,
                         static_cast<f16_t*>(d_logits_out));
      break;
    default:
      hipLaunchKernelGGL((router_dlogits_kernel<bf16_t>), grid, block, 0, s, static_cast<const bf16_t*>(logits), idx,
                         static_cast<const bf16_t*>(d_gates), static_cast<const bf16_t*>(d_logits_extra), T, E, k,
                         static_cast<bf16_t*>(d_logits_out));
  }
  return mi_launch_status();
}
