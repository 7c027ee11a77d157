// Gate-weighted combine of the k expert outputs of every token:
//     y[t, :] = sum_j gates[t, j] * o[t*k + j, :]
// fp32 accumulation in slot order j = 0..k-1, one rounding to the model dtype.
// Stands in for the gates contraction inside the external scattered_experts(gates=...) call at
// lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:282-290 (eager twin: moe.py:305-307).
//
// HBM-bound: every thread owns one 16-byte column chunk of one token and streams its k source rows,
// so a wavefront reads k contiguous 1 KiB segments and writes one.
#include "common.h"

template <typename T> struct Chunk;  // 16-byte chunk <-> floats
template <> struct Chunk<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 v = {__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    return v;
  }
};
template <typename T> struct Chunk16 {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = unpack_lo<T>(v[i]);
      f[2 * i + 1] = unpack_hi<T>(v[i]);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 v = {pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])};
    return v;
  }
};
template <> struct Chunk<bf16_t> : Chunk16<bf16_t> {};
template <> struct Chunk<f16_t> : Chunk16<f16_t> {};

template <typename T>
__global__ __launch_bounds__(256) void combine_vec_kernel(const T* __restrict__ o, const T* __restrict__ gates,
                                                          T* __restrict__ y, int Trows, int k, int H) {
  constexpr int V = Chunk<T>::N;
  const int cpr = H / V;  // chunks per row
  const long total = (long)Trows * cpr;
  for (long id = (long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long)gridDim.x * 256) {
    const int t = (int)(id / cpr);
    const int c = (int)(id - (long)t * cpr);
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    const T* src = o + ((size_t)t * k) * H + (size_t)c * V;
    const T* g = gates + (size_t)t * k;
#pragma unroll 4
    for (int j = 0; j < k; ++j) {
      const float gj = Elt<T>::load(g + j);
      const u32x4 v = *reinterpret_cast<const u32x4*>(src + (size_t)j * H);
      float f[V];
      Chunk<T>::unpack(v, f);
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] = fmaf(gj, f[i], acc[i]);
    }
    *reinterpret_cast<u32x4*>(y + (size_t)t * H + (size_t)c * V) = Chunk<T>::pack(acc);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void combine_scalar_kernel(const T* __restrict__ o, const T* __restrict__ gates,
                                                             T* __restrict__ y, int Trows, int k, int H) {
  const long total = (long)Trows * H;
  for (long id = (long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long)gridDim.x * 256) {
    const int t = (int)(id / H);
    const int h = (int)(id - (long)t * H);
    float acc = 0.f;
    for (int j = 0; j < k; ++j)
      acc = fmaf(Elt<T>::load(gates + (size_t)t * k + j), Elt<T>::load(o + ((size_t)t * k + j) * H + h), acc);
    Elt<T>::store(y + id, acc);
  }
}

template <typename T>
static int launch_combine(const void* o, const void* gates, void* y, int T_, int k, int H, hipStream_t s) {
  constexpr int V = Chunk<T>::N;
  const bool vec = (H % V == 0) && mi_aligned(o, 16) && mi_aligned(y, 16);
  const long work = vec ? (long)T_ * (H / V) : (long)T_ * H;
  long blocks = (work + 255) / 256;
  if (blocks > 256L * 64) blocks = 256L * 64;
  if (vec)
    hipLaunchKernelGGL((combine_vec_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const T*>(o),
                       static_cast<const T*>(gates), static_cast<T*>(y), T_, k, H);
  else
    hipLaunchKernelGGL((combine_scalar_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const T*>(o), static_cast<const T*>(gates), static_cast<T*>(y), T_, k, H);
  return mi_launch_status();
}

extern "C" int mi_moe_combine(const void* o, const void* gates, void* y, int T, int k, int H, int dtype,
                              mi_moe_stream_t stream) {
  if (T < 0 || k < 1 || H < 1) return MI_MOE_ESHAPE;
  if ((double)T * k * H >= 9.0e18) return MI_MOE_ESHAPE;
  if (T == 0) return MI_MOE_OK;
  if (!o || !gates || !y) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI_MOE_F32: return launch_combine<float>(o, gates, y, T, k, H, s);
    case MI_MOE_F16: return launch_combine<f16_t>(o, gates, y, T, k, H, s);
    case MI_MOE_BF16: return launch_combine<bf16_t>(o, gates, y, T, k, H, s);
    default: return MI_MOE_EDTYPE;
  }
}
