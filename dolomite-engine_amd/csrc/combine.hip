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

// A workgroup walks whole token rows (grid-stride over tokens, threads over the row's 16-byte chunks): no
// division per element, the k gates of a row are wave-uniform, and with K known at compile time all k loads
// of a chunk are in flight together.  K == 0 is the run-time-k version.
// Tail of the transformer block, each step rounded to the model dtype exactly as the separate torch operations
// round it: + shared-expert output (moe.py:214), * m_residual, + residual (mixins/dense/layer.py:61-66).
struct CombineTail {
  const void* shared;    // (T, H) or null
  const void* residual;  // (T, H) or null
  float scale;
  int has_scale;
};

template <typename T, int V>
__device__ __forceinline__ void combine_tail(float (&acc)[V], const CombineTail& tail, size_t off) {
  if (tail.shared == nullptr && tail.residual == nullptr && !tail.has_scale) return;
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = Elt<T>::round(acc[i]);
  if (tail.shared != nullptr) {
    float f[V];
    Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(static_cast<const T*>(tail.shared) + off), f);
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = Elt<T>::round(acc[i] + f[i]);
  }
  if (tail.has_scale) {
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = Elt<T>::round(acc[i] * tail.scale);
  }
  if (tail.residual != nullptr) {
    float f[V];
    Chunk<T>::unpack(*reinterpret_cast<const u32x4*>(static_cast<const T*>(tail.residual) + off), f);
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = acc[i] + f[i];
  }
}

template <typename T, int K>
__global__ __launch_bounds__(256) void combine_vec_kernel(const T* __restrict__ o, const T* __restrict__ gates,
                                                          T* __restrict__ y, int Trows, int k_rt, int H,
                                                          CombineTail tail) {
  constexpr int V = Chunk<T>::N;
  const int k = K > 0 ? K : k_rt;
  const int cpr = H / V;  // chunks per row
  for (int t = blockIdx.x; t < Trows; t += gridDim.x) {
    const T* g = gates + (size_t)t * k;
    const T* row = o + ((size_t)t * k) * H;
    for (int c = threadIdx.x; c < cpr; c += blockDim.x) {
      float acc[V];
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] = 0.f;
      const T* src = row + (size_t)c * V;
      if (K > 0) {
        u32x4 v[K > 0 ? K : 1];
#pragma unroll
        for (int j = 0; j < K; ++j) v[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (size_t)j * H));
#pragma unroll
        for (int j = 0; j < K; ++j) {
          const float gj = Elt<T>::load(g + j);
          float f[V];
          Chunk<T>::unpack(v[j], f);
#pragma unroll
          for (int i = 0; i < V; ++i) acc[i] = fmaf(gj, f[i], acc[i]);
        }
      } else {
#pragma unroll 4
        for (int j = 0; j < k; ++j) {
          const float gj = Elt<T>::load(g + j);
          const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (size_t)j * H));
          float f[V];
          Chunk<T>::unpack(v, f);
#pragma unroll
          for (int i = 0; i < V; ++i) acc[i] = fmaf(gj, f[i], acc[i]);
        }
      }
      combine_tail<T, V>(acc, tail, (size_t)t * H + (size_t)c * V);
      __builtin_nontemporal_store(Chunk<T>::pack(acc), reinterpret_cast<u32x4*>(y + (size_t)t * H + (size_t)c * V));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void combine_scalar_kernel(const T* __restrict__ o, const T* __restrict__ gates,
                                                             T* __restrict__ y, int Trows, int k, int H,
                                                             CombineTail tail) {
  const long total = (long)Trows * H;
  for (long id = (long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long)gridDim.x * 256) {
    const int t = (int)(id / H);
    const int h = (int)(id - (long)t * H);
    float acc = 0.f;
    for (int j = 0; j < k; ++j)
      acc = fmaf(Elt<T>::load(gates + (size_t)t * k + j), Elt<T>::load(o + ((size_t)t * k + j) * H + h), acc);
    if (tail.shared != nullptr || tail.residual != nullptr || tail.has_scale) {
      acc = Elt<T>::round(acc);
      if (tail.shared != nullptr) acc = Elt<T>::round(acc + Elt<T>::load(static_cast<const T*>(tail.shared) + id));
      if (tail.has_scale) acc = Elt<T>::round(acc * tail.scale);
      if (tail.residual != nullptr) acc = acc + Elt<T>::load(static_cast<const T*>(tail.residual) + id);
    }
    Elt<T>::store(y + id, acc);
  }
}

template <typename T, int K>
static void launch_combine_vec(const void* o, const void* gates, void* y, int T_, int k, int H, CombineTail tail,
                               hipStream_t s) {
  constexpr int V = Chunk<T>::N;
  const int cpr = H / V;
  int threads = cpr >= 256 ? 256 : (cpr + 63) / 64 * 64;  // whole waves, at most one pass over short rows
  long blocks = T_;
  // one workgroup per token row as long as the grid allows: handed out one by one as workgroups retire, the rows
  // stream faster than with a fixed share of rows per workgroup (32768 tokens of 1536: 0.163 -> 0.156 ms)
  if (blocks > (1L << 20)) blocks = 1L << 20;
  hipLaunchKernelGGL((combine_vec_kernel<T, K>), dim3((unsigned)blocks), dim3(threads), 0, s,
                     static_cast<const T*>(o), static_cast<const T*>(gates), static_cast<T*>(y), T_, k, H, tail);
}

template <typename T>
static int launch_combine(const void* o, const void* gates, void* y, int T_, int k, int H, CombineTail tail,
                          hipStream_t s) {
  constexpr int V = Chunk<T>::N;
  const bool vec = (H % V == 0) && mi_aligned(o, 16) && mi_aligned(y, 16) &&
                   (tail.shared == nullptr || mi_aligned(tail.shared, 16)) &&
                   (tail.residual == nullptr || mi_aligned(tail.residual, 16));
  if (vec) {
    switch (k) {
      case 1: launch_combine_vec<T, 1>(o, gates, y, T_, k, H, tail, s); break;
      case 2: launch_combine_vec<T, 2>(o, gates, y, T_, k, H, tail, s); break;
      case 4: launch_combine_vec<T, 4>(o, gates, y, T_, k, H, tail, s); break;
      case 6: launch_combine_vec<T, 6>(o, gates, y, T_, k, H, tail, s); break;
      case 8: launch_combine_vec<T, 8>(o, gates, y, T_, k, H, tail, s); break;
      default: launch_combine_vec<T, 0>(o, gates, y, T_, k, H, tail, s); break;
    }
  } else {
    const long work = (long)T_ * H;
    long blocks = (work + 255) / 256;
    if (blocks > 256L * 64) blocks = 256L * 64;
    hipLaunchKernelGGL((combine_scalar_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const T*>(o), static_cast<const T*>(gates), static_cast<T*>(y), T_, k, H, tail);
  }
  return mi_launch_status();
}

static int combine_entry(const void* o, const void* gates, void* y, int T, int k, int H, int dtype, CombineTail tail,
                         mi_moe_stream_t stream) {
  if (T < 0 || k < 1 || H < 1) return MI_MOE_ESHAPE;
  if ((double)T * k * H >= 9.0e18) return MI_MOE_ESHAPE;
  if (T == 0) return MI_MOE_OK;
  if (!o || !gates || !y) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI_MOE_F32: return launch_combine<float>(o, gates, y, T, k, H, tail, s);
    case MI_MOE_F16: return launch_combine<f16_t>(o, gates, y, T, k, H, tail, s);
    case MI_MOE_BF16: return launch_combine<bf16_t>(o, gates, y, T, k, H, tail, s);
    default: return MI_MOE_EDTYPE;
  }
}

extern "C" int mi_moe_combine(const void* o, const void* gates, void* y, int T, int k, int H, int dtype,
                              mi_moe_stream_t stream) {
  const CombineTail none = {nullptr, nullptr, 1.0f, 0};
  return combine_entry(o, gates, y, T, k, H, dtype, none, stream);
}

extern "C" int mi_moe_combine_block_tail(const void* o, const void* gates, const void* shared, const void* residual,
                                         float residual_scale, int has_scale, void* y, int T, int k, int H,
                                         int dtype, mi_moe_stream_t stream) {
  const CombineTail tail = {shared, residual, residual_scale, has_scale != 0};
  return combine_entry(o, gates, y, T, k, H, dtype, tail, stream);
}
