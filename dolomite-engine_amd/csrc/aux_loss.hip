// Training-mode auxiliary loss of the router (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:346-369,
// single data-parallel rank) and its gradient with respect to the logits:
//
//   loss = E * sum_e  A_e / max(sum A, eps) * f_e / max(sum f, eps)  +  0.1 * mean_t( logsumexp(logits[t])^2 )
//   A_e = sum_t softmax(logits[t])_e,  f_e = number of (token, slot) pairs routed to expert e,  eps = 1e-12
//
// Forward: one pass over the (T, E) logits -- a wave per row computes the row's logsumexp and probabilities
// and keeps per-lane sums; a workgroup writes one partial per column [A (E) | f (E) | sum lse^2]; a second kernel
// adds each column's partials in a fixed order (deterministic) and a third, one workgroup, forms the loss and
// w_e = d loss / d A_e.
// Backward: d logits[t, j] = g * p_tj * ( w_j - sum_e p_te w_e  +  0.2 / T * lse_t ), one more pass.
// All arithmetic in fp32 from the logits as stored; the eager module rounds its intermediates to the model
// dtype instead, so the two agree to that dtype's rounding, not bit for bit.
#include "common.h"

#define AUX_MAX_E 256
#define AUX_ROWS_PER_BLOCK 32

// lane holds experts lane, lane + 64, ... (NE = ceil(E / 64) <= 4 of them); returns the row's logsumexp and
// leaves the probabilities in p[]
template <typename T>
__device__ __forceinline__ float aux_row_softmax(const T* __restrict__ row, int E, int lane, float (&p)[4]) {
  float x[4];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = lane + 64 * i;
    x[i] = e < E ? Elt<T>::load(row + e) : -INFINITY;
    mx = fmaxf(mx, x[i]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, MI_WAVE));
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    p[i] = lane + 64 * i < E ? __expf(x[i] - mx) : 0.f;
    sum += p[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, MI_WAVE);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < 4; ++i) p[i] *= inv;
  return mx + __logf(sum);
}

template <typename T>
__global__ __launch_bounds__(256) void aux_loss_partial_kernel(const T* __restrict__ logits, const int32_t* __restrict__ topk_idx,
                                                               float* __restrict__ partial, int Trows, int E, int k) {
  __shared__ float acc[4][AUX_MAX_E];
  __shared__ int cnt[AUX_MAX_E];
  __shared__ float zsum[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
  __syncthreads();
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  float z = 0.f;
  const int row0 = blockIdx.x * AUX_ROWS_PER_BLOCK;
  const int row1 = row0 + AUX_ROWS_PER_BLOCK < Trows ? row0 + AUX_ROWS_PER_BLOCK : Trows;
  for (int t = row0 + wave; t < row1; t += 4) {
    float p[4];
    const float lse = aux_row_softmax<T>(logits + (size_t)t * E, E, lane, p);
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] += p[i];
    z = fmaf(lse, lse, z);
    for (int j = lane; j < k; j += 64) {
      const int e = topk_idx[(size_t)t * k + j];
      if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);  // integer: the order does not matter
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (lane + 64 * i < E) acc[wave][lane + 64 * i] = a[i];
  if (lane == 0) zsum[wave] = z;
  __syncthreads();
  // partial[column][block], columns = [A (E) | f (E) | sum lse^2]
  float* out = partial + blockIdx.x;
  const size_t nb = gridDim.x;
  for (int e = threadIdx.x; e < E; e += 256) {
    out[e * nb] = ((acc[0][e] + acc[1][e]) + acc[2][e]) + acc[3][e];
    out[(E + e) * nb] = (float)cnt[e];
  }
  if (threadIdx.x == 0) out[2 * E * nb] = ((zsum[0] + zsum[1]) + zsum[2]) + zsum[3];
}

// column sums of the partials: a wave per column, lanes stride over the blocks, then a fixed butterfly -- the same
// order every run
__global__ __launch_bounds__(256) void aux_loss_colsum_kernel(const float* __restrict__ partial, float* __restrict__ colsum,
                                                              int nblocks, int ncols) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= ncols) return;
  float s = 0.f;
  for (int b = lane; b < nblocks; b += 64) s += partial[(size_t)c * nblocks + b];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, MI_WAVE);
  if (lane == 0) colsum[c] = s;
}

// loss_w[0] = loss, loss_w[1 + e] = d loss / d A_e
__global__ __launch_bounds__(256) void aux_loss_finish_kernel(const float* __restrict__ colsum, float* __restrict__ loss_w,
                                                              int Trows, int E) {
  __shared__ float A[AUX_MAX_E], F[AUX_MAX_E];
  __shared__ float scal[4];
  for (int e = threadIdx.x; e < E; e += 256) {
    A[e] = colsum[e];
    F[e] = colsum[E + e];
  }
  if (threadIdx.x == 0) scal[3] = colsum[2 * E];
  __syncthreads();
  if (threadIdx.x == 0) {
    float sa = 0.f, sf = 0.f, dot = 0.f;
    for (int e = 0; e < E; ++e) {
      sa += A[e];
      sf += F[e];
    }
    sa = fmaxf(sa, 1e-12f);
    sf = fmaxf(sf, 1e-12f);
    for (int e = 0; e < E; ++e) dot = fmaf(A[e] / sa, F[e] / sf, dot);
    const float sw = (float)E * dot;
    scal[0] = sa;
    scal[1] = sf;
    scal[2] = sw;
    loss_w[0] = sw + 0.1f * (scal[3] / (float)Trows);
  }
  __syncthreads();
  // d/dA_e [ sum_e' A_e' c_e' / S ] = (c_e - switch) / S  with c_e = E f_e / sum f  (S = sum A above its floor)
  for (int e = threadIdx.x; e < E; e += 256) loss_w[1 + e] = ((float)E * F[e] / scal[1] - scal[2]) / scal[0];
}

template <typename T>
__global__ __launch_bounds__(256) void aux_loss_backward_kernel(const T* __restrict__ logits, const float* __restrict__ loss_w,
                                                                const float* __restrict__ grad, T* __restrict__ d_logits,
                                                                int Trows, int E) {
  const int lane = threadIdx.x & 63;
  const float g = grad[0];
  const float zc = 0.2f / (float)Trows;
  float w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = lane + 64 * i < E ? loss_w[1 + lane + 64 * i] : 0.f;
  for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < Trows; t += gridDim.x * 4) {
    float p[4];
    const float lse = aux_row_softmax<T>(logits + (size_t)t * E, E, lane, p);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s = fmaf(p[i], w[i], s);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, MI_WAVE);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = lane + 64 * i;
      if (e < E) Elt<T>::store(d_logits + (size_t)t * E + e, g * p[i] * ((w[i] - s) + zc * lse));
    }
  }
}

static int aux_blocks(int T) { return mi_ceil_div(T, AUX_ROWS_PER_BLOCK); }

extern "C" size_t mi_moe_aux_loss_workspace_bytes(int T, int E) {
  if (T < 1 || E < 1) return 0;
  // [partials: (2E + 1) columns x blocks][column sums: 2E + 1]
  return ((size_t)aux_blocks(T) + 1) * (2 * (size_t)E + 1) * sizeof(float);
}

template <typename T>
static void aux_forward_launch(const void* logits, const int32_t* idx, float* ws, float* loss_w, int Trows, int E, int k,
                               hipStream_t s) {
  const int nb = aux_blocks(Trows);
  hipLaunchKernelGGL((aux_loss_partial_kernel<T>), dim3(nb), dim3(256), 0, s, static_cast<const T*>(logits), idx, ws,
                     Trows, E, k);
  const int ncols = 2 * E + 1;
  float* colsum = ws + (size_t)nb * ncols;
  hipLaunchKernelGGL(aux_loss_colsum_kernel, dim3(mi_ceil_div(ncols, 4)), dim3(256), 0, s, ws, colsum, nb, ncols);
  hipLaunchKernelGGL(aux_loss_finish_kernel, dim3(1), dim3(256), 0, s, colsum, loss_w, Trows, E);
}

extern "C" int mi_moe_aux_loss(const void* logits, const int32_t* topk_idx, float* loss_w, void* workspace,
                               size_t workspace_bytes, int T, int E, int k, int dtype, mi_moe_stream_t stream) {
  if (T < 1 || E < 1 || k < 1) return MI_MOE_ESHAPE;
  if (E > AUX_MAX_E) return MI_MOE_EUNSUPPORTED;
  if (!logits || !topk_idx || !loss_w) return MI_MOE_ENULL;
  if (!workspace || workspace_bytes < mi_moe_aux_loss_workspace_bytes(T, E)) return MI_MOE_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  switch (dtype) {
    case MI_MOE_F32: aux_forward_launch<float>(logits, topk_idx, ws, loss_w, T, E, k, s); break;
    case MI_MOE_F16: aux_forward_launch<f16_t>(logits, topk_idx, ws, loss_w, T, E, k, s); break;
    case MI_MOE_BF16: aux_forward_launch<bf16_t>(logits, topk_idx, ws, loss_w, T, E, k, s); break;
    default: return MI_MOE_EDTYPE;
  }
  return mi_launch_status();
}

extern "C" int mi_moe_aux_loss_backward(const void* logits, const float* loss_w, const float* grad, void* d_logits, int T,
                                        int E, int dtype, mi_moe_stream_t stream) {
  if (T < 1 || E < 1) return MI_MOE_ESHAPE;
  if (E > AUX_MAX_E) return MI_MOE_EUNSUPPORTED;
  if (!logits || !loss_w || !grad || !d_logits) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  long blocks = ((long)T + 3) / 4;
  if (blocks > 256L * 16) blocks = 256L * 16;
  switch (dtype) {
    case MI_MOE_F32:
      hipLaunchKernelGGL((aux_loss_backward_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, s,
                         static_cast<const float*>(logits), loss_w, grad, static_cast<float*>(d_logits), T, E);
      break;
    case MI_MOE_F16:
      hipLaunchKernelGGL((aux_loss_backward_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                         static_cast<const f16_t*>(logits), loss_w, grad, static_cast<f16_t*>(d_logits), T, E);
      break;
    case MI_MOE_BF16:
      hipLaunchKernelGGL((aux_loss_backward_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                         static_cast<const bf16_t*>(logits), loss_w, grad, static_cast<bf16_t*>(d_logits), T, E);
      break;
    default: return MI_MOE_EDTYPE;
  }
  return mi_launch_status();
}
