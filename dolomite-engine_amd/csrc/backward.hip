// Element-wise pieces of the backward pass of the expert computation (HBM-bound, one pass each).
//
//   swiglu_backward:     a = up * silu(gate)  =>  d_up = d_a * silu(gate),
//                        d_gate = d_a * up * sigmoid(gate) * (1 + gate * (1 - sigmoid(gate)))
//                        (the forward is GLUActivation with SiLU,
//                        lm_engine/hf_models/modeling_utils/activations/glu.py:42-43).  With the router weight g
//                        of the row's slot, d_a is taken as g * d_act, and the same pass can emit g * a (the
//                        operand of the down-projection's weight gradient) and <d_act, a>, which is the gradient
//                        of the slot's router weight: <dy[t], W a> = <W^T dy[t], a>.
//   combine_grad_gates:  y[t] = sum_j g[t, j] * o[t*k + j]  =>  d_g[t, j] = <dy[t], o[t*k + j]>
//                        (the gates contraction of moe.py:282-290).
// fp32 arithmetic, one rounding to the model dtype.  All three element types: a 16-byte chunk is 8 values of a
// 16-bit type or 4 of fp32.
#include "common.h"

template <typename T> struct Chunk {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const u32x4& v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = unpack_lo<T>(v[i]);
      f[2 * i + 1] = unpack_hi<T>(v[i]);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&f)[8]) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack2<T>(f[2 * i], f[2 * i + 1]);
    return o;
  }
};
template <> struct Chunk<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const u32x4& v, float (&f)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&f)[4]) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = __float_as_uint(f[i]);
    return o;
  }
};

// one wave per sorted row: the lanes stride over the row in 16-byte chunks
template <typename T>
__global__ __launch_bounds__(256) void swiglu_backward_kernel(const T* __restrict__ h, const T* __restrict__ d_act,
                                                              const T* __restrict__ gates,
                                                              const int32_t* __restrict__ sorted_scattered,
                                                              T* __restrict__ d_h, T* __restrict__ act_g,
                                                              T* __restrict__ d_gates, int L, int I) {
  constexpr int CE = Chunk<T>::N;
  const int lane = threadIdx.x & 63;
  const int cpr = I / CE;
  for (int row = blockIdx.x * 4 + (threadIdx.x >> 6); row < L; row += gridDim.x * 4) {
    const int slot = sorted_scattered != nullptr ? sorted_scattered[row] : row;
    const float g = gates != nullptr ? Elt<T>::load(gates + slot) : 1.0f;
    const T* hr = h + (size_t)row * 2 * I;
    T* dr = d_h + (size_t)row * 2 * I;
    float dot = 0.f;
    for (int c = lane; c < cpr; c += 64) {
      float up[CE], gt[CE], da[CE], du[CE], dg[CE], ag[CE];
      Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(hr + c * CE), up);
      Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(hr + I + c * CE), gt);
      Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(d_act + (size_t)row * I + c * CE), da);
#pragma unroll
      for (int i = 0; i < CE; ++i) {
        const float sig = 1.0f / (1.0f + __expf(-gt[i]));
        const float act = up[i] * gt[i] * sig;
        dot = fmaf(da[i], act, dot);
        const float das = da[i] * g;
        du[i] = das * gt[i] * sig;
        dg[i] = das * up[i] * sig * (1.0f + gt[i] * (1.0f - sig));
        ag[i] = act * g;
      }
      *reinterpret_cast<u32x4*>(dr + c * CE) = Chunk<T>::pack(du);
      *reinterpret_cast<u32x4*>(dr + I + c * CE) = Chunk<T>::pack(dg);
      if (act_g != nullptr) *reinterpret_cast<u32x4*>(act_g + (size_t)row * I + c * CE) = Chunk<T>::pack(ag);
    }
    if (d_gates != nullptr) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, MI_WAVE);
      if (lane == 0) Elt<T>::store(d_gates + slot, dot);
    }
  }
}

// one wave per token: the lanes stride over the row in 16-byte chunks, k dot products, butterfly sums
template <typename T>
__global__ __launch_bounds__(256) void combine_grad_gates_kernel(const T* __restrict__ o, const T* __restrict__ dy,
                                                                 T* __restrict__ d_gates, int Trows, int k, int H) {
  constexpr int CE = Chunk<T>::N;
  const int lane = threadIdx.x & 63;
  const int cpr = H / CE;
  for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < Trows; t += gridDim.x * 4) {
    for (int j = 0; j < k; ++j) {
      const T* orow = o + ((size_t)t * k + j) * H;
      float acc = 0.f;
      for (int c = lane; c < cpr; c += 64) {
        float a[CE], b[CE];
        Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(orow + c * CE), a);
        Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(dy + (size_t)t * H + c * CE), b);
#pragma unroll
        for (int i = 0; i < CE; ++i) acc = fmaf(a[i], b[i], acc);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, MI_WAVE);
      if (lane == 0) Elt<T>::store(d_gates + (size_t)t * k + j, acc);
    }
  }
}

// a = up * silu(gate) from a stored pre-activation h = [up | gate]: the activation of the unfused forward that a
// training step takes when it keeps h for the backward instead of recomputing it.  fp32 arithmetic on the rounded
// h, one rounding of the result (what GLUActivation does to the output of the grouped GEMM, activations/glu.py:42-43).
template <typename T>
__global__ __launch_bounds__(256) void swiglu_forward_kernel(const T* __restrict__ h, T* __restrict__ act, long chunks,
                                                             int cpr) {
  // chunk c: row c / cpr, columns CE * (c % cpr) .. + CE
  constexpr int CE = Chunk<T>::N;
  for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (long)gridDim.x * 256) {
    const long row = c / cpr;
    const int col = (int)(c - row * cpr) * CE;
    const T* hp = h + row * (long)(2 * cpr * CE) + col;
    float up[CE], gt[CE], out[CE];
    Chunk<T>::unpack(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(hp)), up);
    Chunk<T>::unpack(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(hp + cpr * CE)), gt);
#pragma unroll
    for (int i = 0; i < CE; ++i) out[i] = up[i] * silu_f32(gt[i]);
    __builtin_nontemporal_store(Chunk<T>::pack(out), reinterpret_cast<u32x4*>(act + row * (long)(cpr * CE) + col));
  }
}

extern "C" int mi_moe_swiglu_forward(const void* h, void* act_out, int L, int I, int dtype, mi_moe_stream_t stream) {
  if (L < 0 || I < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16 && dtype != MI_MOE_F32) return MI_MOE_EDTYPE;
  const int ce = dtype == MI_MOE_F32 ? 4 : 8;  // values per 16-byte chunk
  if (I % ce != 0) return MI_MOE_EUNSUPPORTED;
  if (L == 0) return MI_MOE_OK;
  if (!h || !act_out) return MI_MOE_ENULL;
  if (!mi_aligned(h, 16) || !mi_aligned(act_out, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long chunks = (long)L * (I / ce);
  long blocks = (chunks + 255) / 256;
  if (blocks > 256L * 32) blocks = 256L * 32;
  if (dtype == MI_MOE_BF16)
    hipLaunchKernelGGL((swiglu_forward_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const bf16_t*>(h), static_cast<bf16_t*>(act_out), chunks, I / ce);
  else if (dtype == MI_MOE_F16)
    hipLaunchKernelGGL((swiglu_forward_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const f16_t*>(h), static_cast<f16_t*>(act_out), chunks, I / ce);
  else
    hipLaunchKernelGGL((swiglu_forward_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const float*>(h), static_cast<float*>(act_out), chunks, I / ce);
  return mi_launch_status();
}

extern "C" int mi_moe_swiglu_backward(const void* h, const void* d_act, const void* gates,
                                      const int32_t* sorted_scattered, void* d_h, void* act_g, void* d_gates, int L,
                                      int I, int dtype, mi_moe_stream_t stream) {
  if (L < 0 || I < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16 && dtype != MI_MOE_F32) return MI_MOE_EDTYPE;
  if (I % (dtype == MI_MOE_F32 ? 4 : 8) != 0) return MI_MOE_EUNSUPPORTED;
  if (L == 0) return MI_MOE_OK;
  if (!h || !d_act || !d_h) return MI_MOE_ENULL;
  if (!mi_aligned(h, 16) || !mi_aligned(d_act, 16) || !mi_aligned(d_h, 16) || !mi_aligned(act_g, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  long blocks = ((long)L + 3) / 4;
  if (blocks > 256L * 64) blocks = 256L * 64;
  if (dtype == MI_MOE_BF16)
    hipLaunchKernelGGL((swiglu_backward_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const bf16_t*>(h), static_cast<const bf16_t*>(d_act),
                       static_cast<const bf16_t*>(gates), sorted_scattered, static_cast<bf16_t*>(d_h),
                       static_cast<bf16_t*>(act_g), static_cast<bf16_t*>(d_gates), L, I);
  else if (dtype == MI_MOE_F16)
    hipLaunchKernelGGL((swiglu_backward_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const f16_t*>(h), static_cast<const f16_t*>(d_act), static_cast<const f16_t*>(gates),
                       sorted_scattered, static_cast<f16_t*>(d_h), static_cast<f16_t*>(act_g),
                       static_cast<f16_t*>(d_gates), L, I);
  else
    hipLaunchKernelGGL((swiglu_backward_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const float*>(h), static_cast<const float*>(d_act), static_cast<const float*>(gates),
                       sorted_scattered, static_cast<float*>(d_h), static_cast<float*>(act_g),
                       static_cast<float*>(d_gates), L, I);
  return mi_launch_status();
}

extern "C" int mi_moe_combine_grad_gates(const void* o, const void* dy, void* d_gates, int T, int k, int H, int dtype,
                                         mi_moe_stream_t stream) {
  if (T < 0 || k < 1 || H < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16 && dtype != MI_MOE_F32) return MI_MOE_EDTYPE;
  if (H % (dtype == MI_MOE_F32 ? 4 : 8) != 0) return MI_MOE_EUNSUPPORTED;
  if (T == 0) return MI_MOE_OK;
  if (!o || !dy || !d_gates) return MI_MOE_ENULL;
  if (!mi_aligned(o, 16) || !mi_aligned(dy, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  long blocks = ((long)T + 3) / 4;
  if (blocks > 256L * 32) blocks = 256L * 32;
  if (dtype == MI_MOE_BF16)
    hipLaunchKernelGGL((combine_grad_gates_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const bf16_t*>(o), static_cast<const bf16_t*>(dy), static_cast<bf16_t*>(d_gates), T, k, H);
  else if (dtype == MI_MOE_F16)
    hipLaunchKernelGGL((combine_grad_gates_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const f16_t*>(o), static_cast<const f16_t*>(dy), static_cast<f16_t*>(d_gates), T, k, H);
  else
    hipLaunchKernelGGL((combine_grad_gates_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const float*>(o), static_cast<const float*>(dy), static_cast<float*>(d_gates), T, k, H);
  return mi_launch_status();
}
