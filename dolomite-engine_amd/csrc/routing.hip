// Routing stage of the scattered-MoE forward on gfx950:
//   * top-k + softmax over the selected logits (wave64 shuffle reductions, one row per wavefront)
//   * expert histogram
//   * stable counting sort of the flat expert ids (LDS histograms -> prefix sums -> stable scatter)
//
// Stands in for lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:250-255, 263-271, 338-344 and
// the external continuous_count op used at moe.py:38-44.
#include "common.h"
#include "sort_block.h"
#include "topk_row.h"

// ------------------------------------------------------------------------------------------------
// top-k softmax
// ------------------------------------------------------------------------------------------------

// One wavefront per row; lane l owns experts l, l + 64, ... (topk_row.h): more than 256 experts or k > 16.
template <typename T, int VPL>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ logits, int Trows, int E, int k,
                                                           T* __restrict__ gates, int32_t* __restrict__ idx) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= Trows) return;
  const T* src = logits + (size_t)row * E;
  float vals[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = lane + i * 64;
    vals[i] = e < E ? Elt<T>::load(src + e) : 0.f;
  }
  topk_softmax_row<T, VPL>(vals, E, k, gates + (size_t)row * k, idx + (size_t)row * k);
}

// Four rows per wavefront, 16 lanes per row (topk_row.h): up to 256 experts, k <= 16.  Lane j of a row's group
// loads experts j, j + 16, ...: 16 consecutive values per load and row.
template <typename T, int VPL>
__global__ __launch_bounds__(256) void topk_softmax_rows16_kernel(const T* __restrict__ logits, int Trows, int E, int k,
                                                                  T* __restrict__ gates, int32_t* __restrict__ idx) {
  const int j16 = threadIdx.x & 15;
  const int row = blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool row_ok = row < Trows;
  const int rr = row_ok ? row : Trows - 1;  // surplus groups re-read the last row and write nothing
  const T* src = logits + (size_t)rr * E;
  float vals[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = j16 + i * 16;
    vals[i] = e < E ? Elt<T>::load(src + e) : 0.f;
  }
  topk_softmax_row16<T, VPL>(vals, E, k, row_ok, gates + (size_t)rr * k, idx + (size_t)rr * k);
}

template <typename T>
static int launch_topk(const void* logits, int T_, int E, int k, void* gates, int32_t* idx, hipStream_t s) {
  dim3 grid(mi_ceil_div(T_, 4)), block(256);
  const T* lg = static_cast<const T*>(logits);
  T* gt = static_cast<T*>(gates);
  if (E <= 256 && k <= 16) {
    dim3 grid16(mi_ceil_div(T_, 16));
    if (E <= 16)
      hipLaunchKernelGGL((topk_softmax_rows16_kernel<T, 1>), grid16, block, 0, s, lg, T_, E, k, gt, idx);
    else if (E <= 32)
      hipLaunchKernelGGL((topk_softmax_rows16_kernel<T, 2>), grid16, block, 0, s, lg, T_, E, k, gt, idx);
    else if (E <= 64)
      hipLaunchKernelGGL((topk_softmax_rows16_kernel<T, 4>), grid16, block, 0, s, lg, T_, E, k, gt, idx);
    else if (E <= 128)
      hipLaunchKernelGGL((topk_softmax_rows16_kernel<T, 8>), grid16, block, 0, s, lg, T_, E, k, gt, idx);
    else
      hipLaunchKernelGGL((topk_softmax_rows16_kernel<T, 16>), grid16, block, 0, s, lg, T_, E, k, gt, idx);
    return mi_launch_status();
  }
  if (E <= 64)
    hipLaunchKernelGGL((topk_softmax_kernel<T, 1>), grid, block, 0, s, lg, T_, E, k, gt, idx);
  else if (E <= 128)
    hipLaunchKernelGGL((topk_softmax_kernel<T, 2>), grid, block, 0, s, lg, T_, E, k, gt, idx);
  else if (E <= 256)
    hipLaunchKernelGGL((topk_softmax_kernel<T, 4>), grid, block, 0, s, lg, T_, E, k, gt, idx);
  else
    hipLaunchKernelGGL((topk_softmax_kernel<T, 16>), grid, block, 0, s, lg, T_, E, k, gt, idx);
  return mi_launch_status();
}

extern "C" int mi_moe_router_topk_softmax(const void* logits, int T, int E, int k, int dtype, void* gates_out,
                                          int32_t* idx_out, mi_moe_stream_t stream) {
  if (T < 0 || E < 1 || E > 1024 || k < 1 || k > E || k > 64) return MI_MOE_ESHAPE;
  if (T == 0) return MI_MOE_OK;
  if (!logits || !gates_out || !idx_out) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI_MOE_F32: return launch_topk<float>(logits, T, E, k, gates_out, idx_out, s);
    case MI_MOE_F16: return launch_topk<f16_t>(logits, T, E, k, gates_out, idx_out, s);
    case MI_MOE_BF16: return launch_topk<bf16_t>(logits, T, E, k, gates_out, idx_out, s);
    default: return MI_MOE_EDTYPE;
  }
}

// ------------------------------------------------------------------------------------------------
// histogram of expert ids
// ------------------------------------------------------------------------------------------------

__global__ void zero_u32_kernel(uint32_t* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

__global__ __launch_bounds__(256) void count_kernel(const int32_t* __restrict__ ids, int L, int E,
                                                    uint32_t* __restrict__ counts) {
  __shared__ uint32_t hist[1024];
  for (int e = threadIdx.x; e < E; e += blockDim.x) hist[e] = 0u;
  __syncthreads();
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < L; i += gridDim.x * blockDim.x) {
    int e = ids[i];
    if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1u);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    uint32_t c = hist[e];
    if (c) atomicAdd(&counts[e], c);
  }
}

extern "C" int mi_moe_count(const int32_t* ids, int L, int E, uint32_t* counts_out, mi_moe_stream_t stream) {
  if (L < 0 || E < 1 || E > 1024) return MI_MOE_ESHAPE;
  if (!counts_out || (L > 0 && !ids)) return MI_MOE_ENULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(zero_u32_kernel, dim3(mi_ceil_div(E, 256)), dim3(256), 0, s, counts_out, E);
  if (L > 0) {
    int blocks = mi_ceil_div(L, 256 * 8);
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(count_kernel, dim3(blocks), dim3(256), 0, s, ids, L, E, counts_out);
  }
  return mi_launch_status();
}

// ------------------------------------------------------------------------------------------------
// stable counting sort of expert ids
// ------------------------------------------------------------------------------------------------
//
// The L slots are cut into chunks of SORT_CHUNK consecutive slots, one block per chunk.
//   pass 1  per-chunk histogram in LDS                   -> ws[e * nblk + b]
//   pass 2  per expert: exclusive scan over the chunks (in place) and the expert's total (ws tail)
//   pass 3  every block scans the expert totals (expert bases; block 0 writes the inclusive expert_offsets);
//           each chunk is re-read in order; wave w of the block owns a contiguous quarter of the
//           chunk and walks it 64 slots at a time, so "earlier slot" == "earlier wave, earlier step,
//           lower lane" and ranks come from a match-any ballot: the scatter is stable.
// Small inputs (one chunk) run all three passes inside a single block and need no workspace.

__global__ __launch_bounds__(SORT_THREADS) void sort_hist_kernel(const int32_t* __restrict__ ids, int L, int E,
                                                                 int nblk, int32_t* __restrict__ ws) {
  __shared__ int hist[SORT_MAX_E];
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) hist[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * SORT_CHUNK;
#pragma unroll
  for (int j = 0; j < SORT_CHUNK / SORT_THREADS; ++j) {
    int i = base + j * SORT_THREADS + threadIdx.x;
    if (i < L) {
      int e = ids[i];
      if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) ws[(size_t)e * nblk + blockIdx.x] = hist[e];
}

// Pass 2: one wave per expert (16 per block, ceil(E / 16) blocks).  Lane l owns the chunks [l * C, (l + 1) * C),
// C = ceil(nblk / 64): its loads are all in flight at once (a walk along the row 64 chunks at a time pays one
// memory latency per step), the lane totals are scanned across the wave and the exclusive prefixes written back in
// place.  The expert's total goes to ws[E * nblk + e]; the scan over the experts is left to pass 3, so that no
// block here waits for another.
#define SORT_SCAN_BATCH 8
__global__ __launch_bounds__(1024) void sort_scan_kernel(int E, int nblk, int32_t* __restrict__ ws) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 16 + (threadIdx.x >> 6);
  if (e >= E) return;
  int32_t* row = ws + (size_t)e * nblk;
  const int C = (nblk + 63) >> 6;
  const int begin = lane * C;
  int end = begin + C;
  if (end > nblk) end = nblk;
  // lane total (batches of independent loads)
  int total = 0;
  for (int b0 = begin; b0 < end; b0 += SORT_SCAN_BATCH) {
    int v[SORT_SCAN_BATCH];
#pragma unroll
    for (int i = 0; i < SORT_SCAN_BATCH; ++i) v[i] = b0 + i < end ? row[b0 + i] : 0;
#pragma unroll
    for (int i = 0; i < SORT_SCAN_BATCH; ++i) total += v[i];
  }
  const int incl = wave_incl_scan_i32(total, lane);
  int run = incl - total;  // slots of this expert in the chunks before this lane's
  for (int b0 = begin; b0 < end; b0 += SORT_SCAN_BATCH) {
    int v[SORT_SCAN_BATCH];
#pragma unroll
    for (int i = 0; i < SORT_SCAN_BATCH; ++i) v[i] = b0 + i < end ? row[b0 + i] : 0;  // (cached: just read)
#pragma unroll
    for (int i = 0; i < SORT_SCAN_BATCH; ++i) {
      if (b0 + i < end) row[b0 + i] = run;
      run += v[i];
    }
  }
  if (lane == 63) ws[(size_t)E * nblk + e] = incl;
}

// `chunk`: slots per block (SORT_CHUNK, or what one workgroup of the fused router counted in one turn).  Every block
// scans the E expert totals itself (first wave) to get the experts' first output positions; block 0 also writes the
// inclusive expert_offsets.
__global__ __launch_bounds__(SORT_THREADS) void sort_scatter_kernel(const int32_t* __restrict__ ids, int L, int E,
                                                                    int nbits, int nblk, int chunk,
                                                                    const int32_t* __restrict__ ws,
                                                                    int32_t* __restrict__ sorted_expert,
                                                                    int32_t* __restrict__ sorted_scattered,
                                                                    int32_t* __restrict__ expert_offsets) {
  extern __shared__ int wcnt[];  // SORT_WAVES * E counters, then E expert bases
  int* ebase = wcnt + SORT_WAVES * E;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < SORT_WAVES * E; i += SORT_THREADS) wcnt[i] = 0;
  if (wave == SORT_WAVES - 1) {  // (the last wave: the others start on the histogram meanwhile)
    const int32_t* totals = ws + (size_t)E * nblk;
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int v = e < E ? totals[e] : 0;
      const int inc = wave_incl_scan_i32(v, lane);
      if (e < E) {
        ebase[e] = carry + inc - v;
        if (blockIdx.x == 0) expert_offsets[e] = carry + inc;
      }
      carry += __shfl(inc, 63, MI_WAVE);
    }
  }
  __syncthreads();
  const int chunk_begin = blockIdx.x * chunk;
  int chunk_end = chunk_begin + chunk;
  if (chunk_end > L) chunk_end = L;
  const int per_wave = (chunk + SORT_WAVES - 1) / SORT_WAVES;
  sort_wave_hist(ids, chunk_begin, chunk_end, per_wave, E, wcnt);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
    int run = ws[(size_t)e * nblk + blockIdx.x] + ebase[e];
#pragma unroll
    for (int w = 0; w < SORT_WAVES; ++w) {
      int c = wcnt[w * E + e];
      wcnt[w * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
  sort_scatter_chunk(ids, chunk_begin, chunk_end, per_wave, E, nbits, wcnt, sorted_expert, sorted_scattered);
}

// Whole problem in one block: histogram, expert scan and scatter without touching a workspace.
__global__ __launch_bounds__(SORT_THREADS) void sort_single_block_kernel(const int32_t* __restrict__ ids, int L,
                                                                         int E, int nbits,
                                                                         int32_t* __restrict__ sorted_expert,
                                                                         int32_t* __restrict__ sorted_scattered,
                                                                         int32_t* __restrict__ expert_offsets) {
  extern __shared__ int smem[];  // SORT_WAVES * E counters, then E totals
  sort_single_block(ids, L, E, nbits, sorted_expert, sorted_scattered, expert_offsets, smem);
}


extern "C" size_t mi_moe_sort_bin_workspace_bytes(int L, int E) {
  if (L <= SORT_SINGLE_BLOCK_MAX || E < 1) return 0;
  size_t nblk = (size_t)mi_ceil_div(L, SORT_CHUNK);
  return ((size_t)E * nblk + (size_t)E) * sizeof(int32_t);
}

extern "C" int mi_moe_sort_bin(const int32_t* topk_idx, int T, int k, int E, int32_t* sorted_expert,
                               int32_t* sorted_scattered, int32_t* expert_offsets, void* ws, size_t ws_bytes,
                               mi_moe_stream_t stream) {
  if (T < 0 || k < 1 || E < 1 || E > SORT_MAX_E) return MI_MOE_ESHAPE;
  if ((int64_t)T * k > (int64_t)0x7fffffff - SORT_CHUNK) return MI_MOE_ESHAPE;
  if (!expert_offsets) return MI_MOE_ENULL;
  const int L = T * k;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (L > 0 && (!topk_idx || !sorted_expert || !sorted_scattered)) return MI_MOE_ENULL;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  if (L <= SORT_SINGLE_BLOCK_MAX) {
    size_t lds = (size_t)(SORT_WAVES + 1) * E * sizeof(int);
    hipLaunchKernelGGL(sort_single_block_kernel, dim3(1), dim3(SORT_THREADS), lds, s, topk_idx, L, E, nbits,
                       sorted_expert, sorted_scattered, expert_offsets);
    return mi_launch_status();
  }
  const int nblk = mi_ceil_div(L, SORT_CHUNK);
  if (ws_bytes < mi_moe_sort_bin_workspace_bytes(L, E) || !ws) return MI_MOE_EWORKSPACE;
  if (!mi_aligned(ws, 16)) return MI_MOE_EALIGN;
  int32_t* w = static_cast<int32_t*>(ws);
  hipLaunchKernelGGL(sort_hist_kernel, dim3(nblk), dim3(SORT_THREADS), 0, s, topk_idx, L, E, nblk, w);
  hipLaunchKernelGGL(sort_scan_kernel, dim3(mi_ceil_div(E, 16)), dim3(1024), 0, s, E, nblk, w);
  size_t lds = (size_t)(SORT_WAVES + 1) * E * sizeof(int);
  hipLaunchKernelGGL(sort_scatter_kernel, dim3(nblk), dim3(SORT_THREADS), lds, s, topk_idx, L, E, nbits, nblk,
                     SORT_CHUNK, w, sorted_expert, sorted_scattered, expert_offsets);
  return mi_launch_status();
}

// Passes 2 and 3 alone, for a caller that has produced pass 1 itself: the fused router (router_fused.hip) writes
// ws[e * nblk + b] = number of slots of chunk b that go to expert e, chunks of `chunk` consecutive slots, nblk =
// ceil(L / chunk); ws has room for E more words behind the histograms.  Arguments are validated by the caller.
int mi_sort_after_hist(const int32_t* topk_idx, int L, int E, int chunk, int32_t* sorted_expert,
                       int32_t* sorted_scattered, int32_t* expert_offsets, int32_t* ws, hipStream_t s) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const int nblk = mi_ceil_div(L, chunk);
  hipLaunchKernelGGL(sort_scan_kernel, dim3(mi_ceil_div(E, 16)), dim3(1024), 0, s, E, nblk, ws);
  const size_t lds = (size_t)(SORT_WAVES + 1) * E * sizeof(int);
  hipLaunchKernelGGL(sort_scatter_kernel, dim3(nblk), dim3(SORT_THREADS), lds, s, topk_idx, L, E, nbits, nblk, chunk, ws,
                     sorted_expert, sorted_scattered, expert_offsets);
  return mi_launch_status();
}

// ------------------------------------------------------------------------------------------------
// mi_moe_sort_bin with its workspace inside the library: for callers that cannot allocate.
// ------------------------------------------------------------------------------------------------
//
// The chunk histograms and expert bases of the three-pass sort live in a fixed array in device memory instead of a
// caller workspace.  The array's name is only a handle on the host: the address the kernels get comes from
// hipGetSymbolAddress, asked once per device (each device holds its own copy at its own address) the first time the
// entry point runs with that device current.  Nothing in the array has to start at zero: every word pass 2 and
// pass 3 read was written by pass 1 / pass 2 of the same call.  Calls that overlap on one device share the array and
// race.

#include <mutex>

#define SORT_STATIC_BYTES MI_MOE_SORT_BIN_STATIC_BYTES
#define SORT_STATIC_MAX_DEVICES 64

static __device__ __align__(256) unsigned char scratch[SORT_STATIC_BYTES];

static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[SORT_STATIC_MAX_DEVICES];  // written once per device under the mutex, read-only afterwards

// Device address of `scratch` on the current device (0 with *rc set on failure).
static int32_t* sort_static_scratch(int* rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { *rc = (int)e; return nullptr; }
  if (dev < 0 || dev >= SORT_STATIC_MAX_DEVICES) { *rc = MI_MOE_EUNSUPPORTED; return nullptr; }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) { *rc = (int)e; return nullptr; }
    if (!p || !mi_aligned(p, 16)) { *rc = MI_MOE_EALIGN; return nullptr; }
    g_scratch_ptr[dev] = p;
  }
  *rc = MI_MOE_OK;
  return static_cast<int32_t*>(g_scratch_ptr[dev]);
}

extern "C" int mi_moe_sort_bin_static(const int32_t* topk_idx, int T, int k, int E, int32_t* sorted_expert,
                                      int32_t* sorted_scattered, int32_t* expert_offsets, mi_moe_stream_t stream) {
  if (T < 0 || k < 1 || E < 1 || E > SORT_MAX_E) return MI_MOE_ESHAPE;
  if ((int64_t)T * k > (int64_t)0x7fffffff - SORT_CHUNK) return MI_MOE_ESHAPE;
  if (!expert_offsets) return MI_MOE_ENULL;
  const int L = T * k;
  if (L > 0 && (!topk_idx || !sorted_expert || !sorted_scattered)) return MI_MOE_ENULL;
  const size_t need = mi_moe_sort_bin_workspace_bytes(L, E);
  if (need > SORT_STATIC_BYTES) return MI_MOE_ETOOLARGE;
  int32_t* ws = nullptr;
  if (need) {
    int rc = MI_MOE_OK;
    ws = sort_static_scratch(&rc);
    if (!ws) return rc;
  }
  // the one-block path (need == 0) touches no workspace; otherwise the same three launches on the library's array
  return mi_moe_sort_bin(topk_idx, T, k, E, sorted_expert, sorted_scattered, expert_offsets, ws, need, stream);
}
