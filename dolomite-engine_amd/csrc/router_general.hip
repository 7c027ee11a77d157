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

// NEB: expert blocks of 16 (E <= 16 * NEB).  LDS: [4 waves][NEB][64 lanes] partial accumulators, then
// [16 tokens][16 * NEB] logits as fp32.
template <typename T, int NEB>
__global__ __launch_bounds__(256) void router_general_kernel(const T* __restrict__ x, const T* __restrict__ gw,
                                                             const float* __restrict__ bias, int Trows, int H, int E,
                                                             int k, T* __restrict__ logits_out, T* __restrict__ gates,
                                                             int32_t* __restrict__ idx) {
  constexpr int KSTEP = GMfma<T>::KSTEP;
  constexpr int LPL = KSTEP / 4;                   // elements per lane and step (two 16-byte loads)
  constexpr int HALF = LPL / 2;
  constexpr int EP = 16 * NEB;
  constexpr int VPL = (NEB + 3) / 4;               // candidates per lane in the top-k
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
  for (int k0 = wave * KSTEP; k0 < H; k0 += 4 * KSTEP) {
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
  }
  __syncthreads();
  // top-k and softmax: wave w takes tokens 4 w .. 4 w + 3 -- all four at once, 16 lanes per token, where k allows
  // it, else one after the other with lane l on the experts l, l + 64, ...
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

template <typename T, int NEB>
static int launch_router_general(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                 void* logits_out, void* gates, int32_t* idx, hipStream_t s) {
  constexpr size_t lds = (size_t)4 * NEB * 64 * 16 + (size_t)16 * 16 * NEB * 4;
  auto kern = router_general_kernel<T, NEB>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_ok{0};
    const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok);
    if (rc != MI_MOE_OK) return rc;
  }
  hipLaunchKernelGGL(kern, dim3(mi_ceil_div(T_, 16)), dim3(256), lds, s, static_cast<const T*>(x),
                     static_cast<const T*>(gw), bias, T_, H, E, k, static_cast<T*>(logits_out),
                     static_cast<T*>(gates), idx);
  return mi_launch_status();
}

template <typename T>
static int router_general_by_blocks(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                    void* logits_out, void* gates, int32_t* idx, hipStream_t s) {
  if (E <= 64) return launch_router_general<T, 4>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
  if (E <= 128) return launch_router_general<T, 8>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
  return launch_router_general<T, 16>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
}

// Shapes the general kernel takes: whole 16-byte pieces per lane and step.
int mi_router_general_ok(int H, int E, int k, int dtype) {
  if (E < 1 || E > ROUTER_GENERAL_MAX_E || k < 1 || k > ROUTER_GENERAL_MAX_K || k > E) return 0;
  if (dtype == MI_MOE_F32) return H % 8 == 0;
  return (dtype == MI_MOE_BF16 || dtype == MI_MOE_F16) && H % 16 == 0;
}

// Called by mi_moe_router_fused (router_fused.hip) for what its streaming kernels do not take; arguments are
// validated there.
int mi_router_general(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k, int dtype,
                      void* logits_out, void* gates, int32_t* idx, hipStream_t s) {
  switch (dtype) {
    case MI_MOE_F32: return router_general_by_blocks<float>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
    case MI_MOE_F16: return router_general_by_blocks<f16_t>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
    case MI_MOE_BF16: return router_general_by_blocks<bf16_t>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, s);
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
