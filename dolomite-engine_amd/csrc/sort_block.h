// Block-level pieces of the stable counting sort of expert ids (see routing.hip), shared with the small-batch router,
// whose last workgroup sorts the ids it has just written.
#pragma once

#include "common.h"

#define SORT_THREADS 256
#define SORT_WAVES (SORT_THREADS / 64)
#define SORT_CHUNK 2048
#define SORT_MAX_E 1024

__device__ __forceinline__ int wave_incl_scan_i32(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int o = __shfl_up(v, off, MI_WAVE);
    if (lane >= off) v += o;
  }
  return v;
}

// Stable scatter of one chunk [chunk_begin, chunk_end).  wbase[w * E + e] must hold, on entry, the
// output position of the first slot of expert e seen by wave w.
__device__ __forceinline__ void sort_scatter_chunk(const int32_t* __restrict__ ids, int chunk_begin, int chunk_end,
                                                   int per_wave, int E, int nbits, int* wbase,
                                                   int32_t* __restrict__ sorted_expert,
                                                   int32_t* __restrict__ sorted_scattered) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int* mybase = wbase + wave * E;
  const int begin = chunk_begin + wave * per_wave;
  int end = begin + per_wave;
  if (end > chunk_end) end = chunk_end;
  for (int s0 = begin; s0 < end; s0 += 64) {
    const int slot = s0 + lane;
    const bool valid = slot < end;
    int e = valid ? ids[slot] : 0;
    const bool ok = valid && (unsigned)e < (unsigned)E;
    if (!ok) e = 0;
    uint64_t peers = __ballot(ok);
    for (int b = 0; b < nbits; ++b) {
      uint64_t bal = __ballot((e >> b) & 1);
      peers &= ((e >> b) & 1) ? bal : ~bal;
    }
    if (ok) {
      const uint64_t below = peers & ((1ull << lane) - 1ull);
      const int rank = __popcll(below);
      const int pos = mybase[e] + rank;
      sorted_expert[pos] = e;
      sorted_scattered[pos] = slot;
      // every lane of the group has read mybase[e] (one LDS instruction, wave-wide) before the
      // group's first lane bumps it for the next step
      if (below == 0ull) mybase[e] += __popcll(peers);
    }
  }
}

// Per-wave histograms of a chunk into wcnt[w * E + e] (LDS, pre-zeroed).
__device__ __forceinline__ void sort_wave_hist(const int32_t* __restrict__ ids, int chunk_begin, int chunk_end,
                                               int per_wave, int E, int* wcnt) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int begin = chunk_begin + wave * per_wave;
  int end = begin + per_wave;
  if (end > chunk_end) end = chunk_end;
  for (int s = begin + lane; s < end; s += 64) {
    int e = ids[s];
    if ((unsigned)e < (unsigned)E) atomicAdd(&wcnt[wave * E + e], 1);
  }
}

// Whole problem in one block of SORT_THREADS threads: histogram, expert scan and scatter without touching a
// workspace.  `smem`: (SORT_WAVES + 1) * E ints of LDS.
__device__ __forceinline__ void sort_single_block(const int32_t* __restrict__ ids, int L, int E, int nbits,
                                                  int32_t* __restrict__ sorted_expert,
                                                  int32_t* __restrict__ sorted_scattered,
                                                  int32_t* __restrict__ expert_offsets, int* smem) {
  int* wcnt = smem;
  int* totals = smem + SORT_WAVES * E;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < SORT_WAVES * E; i += SORT_THREADS) wcnt[i] = 0;
  __syncthreads();
  const int per_wave = mi_ceil_div_dev(mi_ceil_div_dev(L, SORT_WAVES), 64) * 64;
  sort_wave_hist(ids, 0, L, per_wave, E, wcnt);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
    int t = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; ++w) t += wcnt[w * E + e];
    totals[e] = t;
  }
  __syncthreads();
  if (wave == 0) {
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      int e = e0 + lane;
      int v = e < E ? totals[e] : 0;
      int inc = wave_incl_scan_i32(v, lane);
      if (e < E) {
        expert_offsets[e] = carry + inc;
        totals[e] = carry + inc - v;  // exclusive base
      }
      carry += __shfl(inc, 63, MI_WAVE);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
    int run = totals[e];
#pragma unroll
    for (int w = 0; w < SORT_WAVES; ++w) {
      int c = wcnt[w * E + e];
      wcnt[w * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
  sort_scatter_chunk(ids, 0, L, per_wave, E, nbits, wcnt, sorted_expert, sorted_scattered);
}

#define SORT_SINGLE_BLOCK_MAX 8192
