// Fused router: logits = x @ gate_w^T (rounded to the model dtype, optional bias), top-k with the
// canonical tie rule, fp32 softmax over the k winners -- one pass over x, nothing but the (T,k)
// results (and optionally the logits) written.
// Stands in for MoE._compute_routing_weights, lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:246-257.
//
// HBM-bound on reading x.  A wavefront works on groups of 16 tokens and all (<= 64) experts:
//   * v_mfma_f32_16x16x32 with the gate weights as operand A (16 experts x 32 k) and the tokens as
//     operand B, so lane (r = l%16, q = l/16) ends with logits of token r for experts 16*eb + 4q + i;
//   * lane (r, q) streams 16 consecutive k of its token row per 64-wide K step (two dwordx4), so the four
//     q-lanes of a token cover one full 128-byte line; both operands use that same lane->k assignment;
//   * top-k: a token's 64 candidates live in 4 lanes x 16 registers; each of the k rounds takes a
//     per-lane maximum of 64-bit keys (ordered value << 32 | ~expert) and a 2-step butterfly.
#include "common.h"
#include "sort_block.h"

template <typename T> struct RMfma;
template <> struct RMfma<bf16_t> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct RMfma<f16_t> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

#define ROUTER_KMAX 8

// The logits are values of a 16-bit type, so (value, expert) orders as ONE 32-bit integer:
//   bits 31..16  the value's bit pattern made monotonic (NaN largest, -0 == +0),
//   bits 15..0   0xffff - expert (the lower expert wins a tie).
// The value is recovered from the winner's key, so no second array follows the keys around.
template <typename T> struct Bits16;
template <> struct Bits16<bf16_t> {
  static constexpr uint32_t INF = 0x7f80u;
  static __device__ __forceinline__ uint32_t of(float rounded) { return __float_as_uint(rounded) >> 16; }
  static __device__ __forceinline__ float value(uint32_t u) { return __uint_as_float(u << 16); }
};
template <> struct Bits16<f16_t> {
  static constexpr uint32_t INF = 0x7c00u;
  static __device__ __forceinline__ uint32_t of(float rounded) {
    const f16_t h = (f16_t)rounded;
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
  }
  static __device__ __forceinline__ float value(uint32_t u) {
    const uint16_t b = (uint16_t)u;
    return (float)__builtin_bit_cast(f16_t, b);
  }
};
template <typename T>
__device__ __forceinline__ uint32_t router_ordered16(uint32_t u) {
  if ((u & 0x7fffu) > Bits16<T>::INF) return 0xffffu;  // NaN
  if (u == 0x8000u) u = 0u;                             // -0 == +0
  return (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
}
template <typename T>
__device__ __forceinline__ float router_value_of_key(uint32_t key) {
  const uint32_t o = key >> 16;
  return Bits16<T>::value((o & 0x8000u) ? (o ^ 0x8000u) : (~o & 0xffffu));
}

// max over the four lanes (q = 0..3) that hold one token's candidates: lanes l, l^16, l^32, l^48.
// v_permlane16_swap with both operands x leaves {x of the even row, x of the odd row} of each row pair in the
// two results, v_permlane32_swap the same for the two halves; a max of the two results is the butterfly step.
__device__ __forceinline__ uint32_t router_max4(uint32_t x) {
  const auto a = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  const uint32_t m = a[0] > a[1] ? a[0] : a[1];
  const auto b = __builtin_amdgcn_permlane32_swap(m, m, false, false);
  return b[0] > b[1] ? b[0] : b[1];
}

// Epilogue for one group of 16 tokens: lane (r = token, q) holds acc[eb][i] = logit of expert
// 16*eb + 4*q + i.  Rounds to the model dtype, adds the optional bias, optionally stores the logits,
// selects the top-k (value descending, expert ascending) and writes the softmax of the k winners.
// `hist` (LDS, E counters shared by the workgroup, or null) receives one count per selected expert.
template <typename T>
__device__ __forceinline__ void router_epilogue(const f32x4 (&acc)[4], int t, bool tvalid, int q,
                                                const float* __restrict__ bias, int E, int k,
                                                T* __restrict__ logits_out, T* __restrict__ gates,
                                                int32_t* __restrict__ idx, int* hist = nullptr) {
  uint32_t keys[16];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = eb * 16 + 4 * q + i;
      float v = Elt<T>::round(acc[eb][i]);
      if (bias != nullptr && e < E) v = Elt<T>::round(v + bias[e]);
      keys[eb * 4 + i] = e < E ? ((router_ordered16<T>(Bits16<T>::of(v)) << 16) | (0xffffu - (uint32_t)e)) : 0u;
      if (logits_out != nullptr && tvalid && e < E) Elt<T>::store(logits_out + (size_t)t * E + e, v);
    }
  }
  float wv[ROUTER_KMAX];
  int wi[ROUTER_KMAX];
#pragma unroll
  for (int j = 0; j < ROUTER_KMAX; ++j) {
    wv[j] = 0.f;
    wi[j] = 0;
    if (j < k) {
      uint32_t best = keys[0];
#pragma unroll
      for (int c = 1; c < 16; ++c) best = keys[c] > best ? keys[c] : best;
      best = router_max4(best);
#pragma unroll
      for (int c = 0; c < 16; ++c)
        if (keys[c] == best) keys[c] = 0u;
      wv[j] = router_value_of_key<T>(best);
      wi[j] = (int)(0xffffu - (best & 0xffffu));
    }
  }
  if (q == 0 && tvalid) {
    float p[ROUTER_KMAX];
    float denom = 0.f;
#pragma unroll
    for (int j = 0; j < ROUTER_KMAX; ++j) {
      p[j] = j < k ? expf(wv[j] - wv[0]) : 0.f;
      denom += p[j];
    }
#pragma unroll
    for (int j = 0; j < ROUTER_KMAX; ++j) {
      if (j < k) {
        Elt<T>::store(gates + (size_t)t * k + j, p[j] / denom);
        idx[(size_t)t * k + j] = wi[j];
        if (hist != nullptr) atomicAdd(&hist[wi[j]], 1);
      }
    }
  }
}

// Many tokens, gate weights held in LDS (reading the gate weights (E x H) from L2 for every few groups would move
// more bytes than x itself).  A workgroup of eight waves copies the
// weights into LDS once (row pitch 2H + 16 bytes: the 16 rows of a fragment read then start in 16 different
// 16-byte bank groups) and then walks 16-token groups, one per wave and turn; x streams through a register ring
// DEPTH K steps deep (3 with eight waves: about 48 KB in flight per CU), and only the ceil(E / 16) expert blocks that exist are
// multiplied.
// With fewer than eight groups per CU fewer waves per workgroup walk groups (so that every CU takes part), with a
// deeper ring per wave (DEPTH 6) to keep as many bytes in flight; the workgroup still has eight waves for the copy
// of the weights (one wave alone took 20 us over it: 29 us for this kernel at 1024 - 4096 tokens).
#define ROUTER_LDS_WAVES 8
// NORM folds the RMSNorm in front of the layer (ln_2 of the transformer block, mixins/dense/layer.py:58-59;
// normalization.py:19-34 = torch.nn.RMSNorm) into the same kernel: a group's rows are streamed twice, first for
// the sum of squares, then (out of L2) normalised as torch does -- round(x * rstd * gamma), all in fp32, one
// rounding -- written to xnorm_out for the expert GEMMs and multiplied with the gate weights in that rounded
// form.  The separate RMSNorm pass (read and write of (T, H)) and the router's own read of its output are gone.
struct RouterNorm {
  const void* gamma;  // (H,) of the model dtype, or null: no scaling
  void* xnorm_out;    // (T, H)
  float eps;
};

// `chunk_hist` (or null): the first pass of the expert sort (routing.hip) done here.  The groups a workgroup takes
// in one turn are consecutive -- a chunk of nwaves * 16 tokens -- so the workgroup counts the experts its
// waves select in LDS and writes chunk_hist[e * nchunks + chunk], the layout the sort's scan pass reads; the sort
// then needs neither its histogram launch nor that launch's read of the expert ids.
// KS (at most four groups per workgroup: every group is walked in one turn): `ksplit` waves share a group and split its K
// steps (wave part p takes steps p, p + ksplit, ...), so that a group's row is walked in one or two round trips to
// memory instead of four; the partial logits meet in LDS (over the weights, which nobody needs any more, or behind
// them when they are smaller than the 32 KB this takes: `red_at`) and are added in part order.  Measured, hidden
// 1536, 40 experts: 13.0 us for this kernel from 1024 to 4096 tokens (20.5 - 20.9 us with one wave per group),
// 16.3 us at 8192, 21.8 us at 16384 tokens.  With the norm folded in, the sums of squares of a row's parts meet in
// LDS first (`ss_at`): 31.5 / 32.8 / 46.7 -> 15.2 / 17.2 / 35.5 us at 1024 / 4096 / 16384 tokens.
template <typename T, int DEPTH, bool NORM, bool KS = false>
__global__ __launch_bounds__(ROUTER_LDS_WAVES * 64) void router_fused_lds_kernel(
    const T* __restrict__ x, const T* __restrict__ gw, const float* __restrict__ bias, int Trows, int H, int E, int k,
    T* __restrict__ logits_out, T* __restrict__ gates, int32_t* __restrict__ idx, RouterNorm norm,
    int32_t* __restrict__ chunk_hist, int nchunks, int nwaves, int ksplit, int red_at, int ss_at) {
  typedef typename RMfma<T>::vec frag_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char wlds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int pitch = H * (int)sizeof(T) + 16;
  // the first `nwaves` waves walk token groups; the others only help to copy the weights (and keep the barriers)
  const int nsteps = (H + 63) >> 6;
  const int ngroups = (Trows + 15) >> 4;
  const int stride = gridDim.x * nwaves;
  // KS: wave = slot * ksplit + part
  const int part = KS ? wave % ksplit : 0;
  const int slot = KS ? wave / ksplit : wave;
  const int kstep = KS ? ksplit : 1;
  const int nmine = KS ? (nsteps - part + ksplit - 1) / ksplit : nsteps;  // K steps of this wave
  int grp = slot < nwaves ? blockIdx.x * nwaves + slot : ngroups;

  // x ring of the wave's current group; the first DEPTH steps of a group are requested before the previous
  // group's epilogue (for the first group: before the weights are copied), so their latency is hidden
  const T* xrow = x;
  u32x4 xr[DEPTH][2];
  auto load_x = [&](int step, u32x4 (&dst)[2]) {  // step: the wave's own count; K step step * kstep + part
    const int kpos = (step * kstep + part) * 64 + q * 16;
    dst[0] = dst[1] = (u32x4){0u, 0u, 0u, 0u};
    if (step < nmine && kpos < H) {  // the MFMA runs on all lanes: out-of-range k contributes zeros
      // Ordinary (cached) loads: with the norm the rows are read twice, and without it they are read again right
      // after, as the gathered operand of the up-projection -- which runs 1 - 1.5 % faster on rows this pass left in
      // the caches than on rows streamed through with the non-temporal policy (and this kernel is no slower).
      dst[0] = *reinterpret_cast<const u32x4*>(xrow + kpos);
      dst[1] = *reinterpret_cast<const u32x4*>(xrow + kpos + 8);
    }
  };
  auto open_group = [&](int g) {
    int t = g * 16 + r;
    if (t > Trows - 1) t = Trows - 1;
    xrow = x + (size_t)t * H;
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load_x(d, xr[d]);
  };
  if (grp < ngroups) open_group(grp);

  // ---- gate weights -> LDS (16-byte pieces; H % 16 == 0 is checked on the host) ----
  // eight loads in flight per thread: one load-wait-store per iteration would pay an L2 latency per piece
  const int pieces_per_row = H * (int)sizeof(T) / 16;
  const int pieces = E * pieces_per_row;
  for (int p0 = threadIdx.x; p0 < pieces; p0 += 8 * blockDim.x) {
    u32x4 v[8];
    int dst[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int p = p0 + i * blockDim.x;
      dst[i] = -1;
      if (p < pieces) {
        const int e = p / pieces_per_row, c = p - e * pieces_per_row;
        dst[i] = e * pitch + c * 16;
        v[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned char*>(gw) + (size_t)p * 16);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (dst[i] >= 0) *reinterpret_cast<u32x4*>(wlds + dst[i]) = v[i];
  }
  // NORM: gamma (or ones) as fp32 behind the weights; then the E counters of the chunk histogram
  float* glds = reinterpret_cast<float*>(wlds + (size_t)E * pitch);
  if (NORM) {
    const T* gamma = static_cast<const T*>(norm.gamma);
    for (int i = threadIdx.x; i < H; i += blockDim.x) glds[i] = gamma != nullptr ? Elt<T>::load(gamma + i) : 1.0f;
  }
  int* whist = reinterpret_cast<int*>(wlds + (size_t)E * pitch + (NORM ? (size_t)H * sizeof(float) : 0));
  if (chunk_hist != nullptr)
    for (int e = threadIdx.x; e < E; e += blockDim.x) whist[e] = 0;
  __syncthreads();

  const int neb = (E + 15) >> 4;
  int wbase[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    int e = eb * 16 + r;
    if (e > E - 1) e = E - 1;
    wbase[eb] = e * pitch;
  }
  // with a histogram every wave walks the same number of turns (a turn ends in workgroup barriers)
  const int nturns = KS ? 1 : (chunk_hist != nullptr ? (ngroups + stride - 1) / stride : 0);
  for (int turn = 0; (KS || chunk_hist != nullptr) ? turn < nturns : grp < ngroups; ++turn) {
    const bool active = grp < ngroups;
    f32x4 acc[4];
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float ss = 0.f, rstd = 1.0f;
    if (NORM && active) {
      // first pass over the group's rows (KS: over this wave's K steps of them): sum of squares of the 16 k this
      // lane holds per step, then over the four lanes of the token
      for (int s0 = 0; s0 < nmine; s0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
          const int step = s0 + d;
          if (step < nmine) {
            const u32x4 x0 = xr[d][0], x1 = xr[d][1];
            load_x(step + DEPTH, xr[d]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float a0 = unpack_lo<T>(x0[i]), a1 = unpack_hi<T>(x0[i]);
              const float b0 = unpack_lo<T>(x1[i]), b1 = unpack_hi<T>(x1[i]);
              ss = fmaf(a0, a0, ss); ss = fmaf(a1, a1, ss); ss = fmaf(b0, b0, ss); ss = fmaf(b1, b1, ss);
            }
          }
        }
      }
      ss += __shfl_xor(ss, 16, MI_WAVE);
      ss += __shfl_xor(ss, 32, MI_WAVE);
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) load_x(d, xr[d]);  // second pass, out of L2
    }
    if constexpr (NORM && KS) {
      // the parts of a row's sum of squares meet in LDS and every wave of the group adds them in part order
      float* ssred = reinterpret_cast<float*>(wlds + ss_at);
      if (q == 0) ssred[wave * 16 + r] = ss;
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the x loads of the second pass stay in flight
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      ss = 0.f;
      for (int p = 0; p < ksplit; ++p) ss += ssred[(wave - part + p) * 16 + r];
    }
    if (NORM) rstd = 1.0f / sqrtf(ss / (float)H + norm.eps);
    if (active) {
    T* xn_row = nullptr;
    if (NORM) {
      const int t = grp * 16 + r;
      if (t < Trows) xn_row = static_cast<T*>(norm.xnorm_out) + (size_t)t * H;
    }
    for (int s0 = 0; s0 < nmine; s0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int step = s0 + d;
        if (step < nmine) {
          const int kel = (step * kstep + part) * 64 + q * 16;
          const int kbyte = kel * (int)sizeof(T);
          const bool valid = kel < H;
          u32x4 x0 = xr[d][0], x1 = xr[d][1];
          load_x(step + DEPTH, xr[d]);
          if (NORM && valid) {
            const int kpos = kel;
            const f32x4* g4 = reinterpret_cast<const f32x4*>(glds + kpos);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const f32x4 ga = g4[i >> 1], gb = g4[2 + (i >> 1)];
              const int o = (i & 1) * 2;
              x0[i] = pack2<T>(unpack_lo<T>(x0[i]) * rstd * ga[o], unpack_hi<T>(x0[i]) * rstd * ga[o + 1]);
              x1[i] = pack2<T>(unpack_lo<T>(x1[i]) * rstd * gb[o], unpack_hi<T>(x1[i]) * rstd * gb[o + 1]);
            }
            if (xn_row != nullptr) {
              *reinterpret_cast<u32x4*>(xn_row + kpos) = x0;
              *reinterpret_cast<u32x4*>(xn_row + kpos + 8) = x1;
            }
          }
#pragma unroll
          for (int eb = 0; eb < 4; ++eb) {
            if (eb < neb) {
              u32x4 w0 = {0u, 0u, 0u, 0u}, w1 = {0u, 0u, 0u, 0u};
              if (valid) {
                w0 = *reinterpret_cast<const u32x4*>(wlds + wbase[eb] + kbyte);
                w1 = *reinterpret_cast<const u32x4*>(wlds + wbase[eb] + kbyte + 16);
              }
              acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w0), __builtin_bit_cast(frag_t, x0), acc[eb]);
              acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w1), __builtin_bit_cast(frag_t, x1), acc[eb]);
            }
          }
        }
      }
    }
    }
    if constexpr (KS) {
      // every wave is done with the weights; the parts of a group meet in LDS and part 0 adds them in part order
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      f32x4* red = reinterpret_cast<f32x4*>(wlds + red_at);
      if (part != 0) {
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) red[(wave * 4 + eb) * 64 + lane] = acc[eb];
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (part == 0) {
        for (int p = 1; p < ksplit; ++p) {
#pragma unroll
          for (int eb = 0; eb < 4; ++eb) acc[eb] += red[((wave + p) * 4 + eb) * 64 + lane];
        }
      }
    }
    if (active && part == 0) {
      const int t = grp * 16 + r;
      grp += stride;
      if (!KS && grp < ngroups) open_group(grp);
      router_epilogue<T>(acc, t, t < Trows, q, bias, E, k, logits_out, gates, idx,
                         chunk_hist != nullptr ? whist : nullptr);
    } else {
      grp += stride;
    }
    if (chunk_hist != nullptr) {
      // all counts of this turn are in (LDS only: the x loads already in flight for the next turn stay in flight)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0), vmcnt / expcnt untouched
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      const int chunk = blockIdx.x + turn * gridDim.x;
      for (int e = threadIdx.x; e < E; e += blockDim.x) {
        if (chunk < nchunks) chunk_hist[(size_t)e * nchunks + chunk] = whist[e];
        whist[e] = 0;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
  }
}

// Many tokens, gate weights too large for LDS.  A workgroup of eight waves owns ROUTER_KS_TG groups of 16 tokens;
// wave w takes the 64-wide K steps w, w + 8, ... of all of them (two steps' loads in flight at a time), so a wave
// walks an eighth of the row, and a step's gate-weight fragments serve every group.  The partial logits meet in
// LDS, two groups at a time, and are added in wave order (the logits do not depend on scheduling); waves
// 0 .. ROUTER_KS_TG - 1 then run one group's epilogue each.
#define ROUTER_KS_WAVES 8
#define ROUTER_KS_TG 4
template <typename T>
__global__ __launch_bounds__(ROUTER_KS_WAVES * 64) void router_fused_ksplit_kernel(
    const T* __restrict__ x, const T* __restrict__ gw, const float* __restrict__ bias, int Trows, int H, int E, int k,
    T* __restrict__ logits_out, T* __restrict__ gates, int32_t* __restrict__ idx) {
  typedef typename RMfma<T>::vec frag_t;
  constexpr int TG = ROUTER_KS_TG, NW = ROUTER_KS_WAVES;
  static_assert(TG % 2 == 0 && TG <= NW, "groups are reduced in pairs, one finishing wave per group");
  __shared__ f32x4 red[NW][2][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tok0 = blockIdx.x * (16 * TG);
  const T* xrow[TG];
#pragma unroll
  for (int g = 0; g < TG; ++g) {
    int t = tok0 + g * 16 + r;
    if (t > Trows - 1) t = Trows - 1;
    xrow[g] = x + (size_t)t * H;
  }
  const T* wrow[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    int e = eb * 16 + r;
    if (e > E - 1) e = E - 1;
    wrow[eb] = gw + (size_t)e * H;
  }
  const int neb = (E + 15) >> 4;
  f32x4 acc[4][TG];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb)
#pragma unroll
    for (int g = 0; g < TG; ++g) acc[eb][g] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int k0 = wave * 64; k0 < H; k0 += 2 * NW * 64) {
    u32x4 xa[2][TG][2], wa[2][4][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int kpos = k0 + s * NW * 64 + q * 16;
      const bool valid = kpos < H;  // the MFMA runs on all lanes: out-of-range k contributes zeros
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        xa[s][g][0] = xa[s][g][1] = (u32x4){0u, 0u, 0u, 0u};
        if (valid) {
          xa[s][g][0] = *reinterpret_cast<const u32x4*>(xrow[g] + kpos);
          xa[s][g][1] = *reinterpret_cast<const u32x4*>(xrow[g] + kpos + 8);
        }
      }
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        wa[s][eb][0] = wa[s][eb][1] = (u32x4){0u, 0u, 0u, 0u};
        if (valid && eb < neb) {
          wa[s][eb][0] = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos);
          wa[s][eb][1] = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos + 8);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int eb = 0; eb < 4; ++eb)
          if (eb < neb) {
#pragma unroll
            for (int g = 0; g < TG; ++g)
              acc[eb][g] = RMfma<T>::run(__builtin_bit_cast(frag_t, wa[s][eb][h]),
                                         __builtin_bit_cast(frag_t, xa[s][g][h]), acc[eb][g]);
          }
  }

  f32x4 fin[4];
#pragma unroll
  for (int gp = 0; gp < TG / 2; ++gp) {
    if (gp > 0) __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) red[wave][j][eb][lane] = acc[eb][2 * gp + j];
    __syncthreads();
    if ((wave >> 1) == gp) {
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        f32x4 sum = red[0][wave & 1][eb][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][wave & 1][eb][lane];
        fin[eb] = sum;
      }
    }
  }
  if (wave < TG) {
    const int t = tok0 + wave * 16 + r;
    router_epilogue<T>(fin, t, t < Trows, q, bias, E, k, logits_out, gates, idx);
  }
}

// Few tokens (decode): one workgroup of 16 waves per group of 16 tokens; the waves split K (wave w takes
// the 64-wide K steps w, w+16, ...) and their partial logits meet in LDS, so that the latency of walking
// H is paid once per 16th of the row instead of once per row.
template <typename T>
__global__ __launch_bounds__(1024) void router_fused_small_kernel(const T* __restrict__ x, const T* __restrict__ gw,
                                                                  const float* __restrict__ bias, int Trows, int H,
                                                                  int E, int k, T* __restrict__ logits_out,
                                                                  T* __restrict__ gates, int32_t* __restrict__ idx) {
  typedef typename RMfma<T>::vec frag_t;
  __shared__ f32x4 red[16][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tok0 = blockIdx.x * 16;
  int t = tok0 + r;
  const bool tvalid = t < Trows;
  const T* xrow = x + (size_t)(tvalid ? t : Trows - 1) * H;
  const T* wrow[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    int e = eb * 16 + r;
    if (e > E - 1) e = E - 1;
    wrow[eb] = gw + (size_t)e * H;
  }
  f32x4 acc[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * 64; k0 < H; k0 += 16 * 64) {
    const int kpos = k0 + q * 16;
    const bool valid = kpos < H;  // the MFMA runs on all lanes: out-of-range k contributes zeros
    u32x4 x0 = {0u, 0u, 0u, 0u}, x1 = {0u, 0u, 0u, 0u};
    if (valid) {
      x0 = *reinterpret_cast<const u32x4*>(xrow + kpos);
      x1 = *reinterpret_cast<const u32x4*>(xrow + kpos + 8);
    }
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      u32x4 w0 = {0u, 0u, 0u, 0u}, w1 = {0u, 0u, 0u, 0u};
      if (valid) {
        w0 = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos);
        w1 = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos + 8);
      }
      acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w0), __builtin_bit_cast(frag_t, x0), acc[eb]);
      acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w1), __builtin_bit_cast(frag_t, x1), acc[eb]);
    }
  }
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) red[wave][eb][lane] = acc[eb];
  __syncthreads();
  if (wave == 0) {
    // fixed summation order (wave 0, 1, ..., 15): the logits do not depend on scheduling
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      f32x4 sum = red[0][eb][lane];
      for (int w = 1; w < 16; ++w) sum += red[w][eb][lane];
      acc[eb] = sum;
    }
    router_epilogue<T>(acc, t, tvalid, q, bias, E, k, logits_out, gates, idx);
  }
}

// Few tokens, K split across workgroups.  One workgroup reads at most 26 bytes per clock, and a 16-token group
// needs all of the gate weights (E x H): four workgroups pulling 640 KB each take 20+ us for a 64-token batch.
// Here workgroup (tg, ks) takes K range ks of token group tg (four waves, one 64-wide K step each per
// round) and writes its 16 x 64 partial logits, as raw accumulator registers, to the workspace; a second
// launch adds the partials in a fixed order (the logits do not depend on scheduling) and runs the epilogue.
#define ROUTER_SPLIT_WAVES 4
template <typename T>
__global__ __launch_bounds__(ROUTER_SPLIT_WAVES * 64) void router_splitk_partial_kernel(
    const T* __restrict__ x, const T* __restrict__ gw, int Trows, int H, int E, int steps_per_split,
    f32x4* __restrict__ partial, unsigned* __restrict__ ticket) {
  typedef typename RMfma<T>::vec frag_t;
  __shared__ f32x4 red[ROUTER_SPLIT_WAVES][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // the finish kernel's ticket counter (fused sort) starts at zero: this kernel is complete before that one starts
  if (ticket != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *ticket = 0u;
  const int r = lane & 15, q = lane >> 4;
  const int tg = blockIdx.x, ks = blockIdx.y;
  int t = tg * 16 + r;
  if (t > Trows - 1) t = Trows - 1;
  const T* xrow = x + (size_t)t * H;
  const T* wrow[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    int e = eb * 16 + r;
    if (e > E - 1) e = E - 1;
    wrow[eb] = gw + (size_t)e * H;
  }
  f32x4 acc[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int step0 = ks * steps_per_split;
  for (int st = wave; st < steps_per_split; st += ROUTER_SPLIT_WAVES) {
    const int kpos = (step0 + st) * 64 + q * 16;
    const bool valid = kpos < H;  // the MFMA runs on all lanes: out-of-range k contributes zeros
    u32x4 x0 = {0u, 0u, 0u, 0u}, x1 = {0u, 0u, 0u, 0u};
    u32x4 w0[4], w1[4];
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) w0[eb] = w1[eb] = (u32x4){0u, 0u, 0u, 0u};
    if (valid) {
      x0 = *reinterpret_cast<const u32x4*>(xrow + kpos);
      x1 = *reinterpret_cast<const u32x4*>(xrow + kpos + 8);
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        w0[eb] = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos);
        w1[eb] = *reinterpret_cast<const u32x4*>(wrow[eb] + kpos + 8);
      }
    }
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w0[eb]), __builtin_bit_cast(frag_t, x0), acc[eb]);
      acc[eb] = RMfma<T>::run(__builtin_bit_cast(frag_t, w1[eb]), __builtin_bit_cast(frag_t, x1), acc[eb]);
    }
  }
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) red[wave][eb][lane] = acc[eb];
  __syncthreads();
  if (wave == 0) {
    f32x4* dst = partial + ((size_t)ks * gridDim.x + tg) * 4 * 64;
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      f32x4 sum = red[0][eb][lane];
#pragma unroll
      for (int w = 1; w < ROUTER_SPLIT_WAVES; ++w) sum += red[w][eb][lane];
      dst[eb * 64 + lane] = sum;
    }
  }
}

// Four waves per token group: wave w adds splits w, w + 4, ... (all of its loads in flight at once), wave 0 adds
// the four sums in wave order and runs the epilogue.  The order of additions is fixed by the launch shape alone.
template <typename T>
__global__ __launch_bounds__(256) void router_splitk_finish_kernel(const f32x4* __restrict__ partial, int splits,
                                                                   const float* __restrict__ bias, int Trows, int E, int k,
                                                                   T* __restrict__ logits_out, T* __restrict__ gates,
                                                                   int32_t* __restrict__ idx) {
  __shared__ f32x4 red[4][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tg = blockIdx.x;
  const int t = tg * 16 + r;
  f32x4 acc[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int ks = wave; ks < splits; ks += 4) {
    const f32x4* src = partial + ((size_t)ks * gridDim.x + tg) * 4 * 64;
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) acc[eb] += src[eb * 64 + lane];
  }
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) red[wave][eb][lane] = acc[eb];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    f32x4 sum = red[0][eb][lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) sum += red[w][eb][lane];
    acc[eb] = sum;
  }
  router_epilogue<T>(acc, t, t < Trows, q, bias, E, k, logits_out, gates, idx);
}

// The finish kernel with the expert sort folded in (few tokens, T * k <= SORT_SINGLE_BLOCK_MAX): every workgroup
// publishes its 16 tokens' experts and takes a ticket; the workgroup that draws the last ticket sorts all T * k ids
// in the same launch (the single-block counting sort of routing.hip).  One launch boundary less on a path that is a
// chain of short dependent launches.  `ticket` is a counter in the workspace that the partial kernel has zeroed.
template <typename T>
__global__ __launch_bounds__(256) void router_splitk_finish_sort_kernel(
    const f32x4* __restrict__ partial, int splits, const float* __restrict__ bias, int Trows, int E, int k, int nbits,
    T* __restrict__ logits_out, T* __restrict__ gates, int32_t* __restrict__ idx, unsigned* __restrict__ ticket,
    int32_t* __restrict__ sorted_expert, int32_t* __restrict__ sorted_scattered, int32_t* __restrict__ expert_offsets) {
  __shared__ f32x4 red[4][4][64];
  __shared__ int is_last;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int tg = blockIdx.x;
  const int t = tg * 16 + r;
  f32x4 acc[4];
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) acc[eb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int ks = wave; ks < splits; ks += 4) {
    const f32x4* src = partial + ((size_t)ks * gridDim.x + tg) * 4 * 64;
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) acc[eb] += src[eb * 64 + lane];
  }
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) red[wave][eb][lane] = acc[eb];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      f32x4 sum = red[0][eb][lane];
#pragma unroll
      for (int w = 1; w < 4; ++w) sum += red[w][eb][lane];
      acc[eb] = sum;
    }
    router_epilogue<T>(acc, t, t < Trows, q, bias, E, k, logits_out, gates, idx);
    __threadfence();  // this workgroup's experts are visible device-wide before its ticket is
    if (lane == 0) is_last = atomicAdd(ticket, 1u) == gridDim.x - 1;
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();  // ... and the last workgroup reads what the others published
  sort_single_block(idx, Trows * k, E, nbits, sorted_expert, sorted_scattered, expert_offsets,
                    reinterpret_cast<int*>(&red[0][0][0]));
}

// K splits for the few-token path: one 64-wide K step per wave and round, enough workgroups to occupy the chip
static int router_splits(int T_, int H) {
  const int steps = mi_ceil_div(H, 64);
  int splits = mi_ceil_div(steps, ROUTER_SPLIT_WAVES);
  const int groups = mi_ceil_div(T_, 16);
  while (splits > 1 && (long)splits * groups > 1024) splits = (splits + 1) / 2;
  return splits;
}

// gate weights (16 bits an element) fit in LDS next to the per-expert words of the LDS-resident kernel
static bool router_lds_fits(int H, int E) { return (size_t)E * ((size_t)H * 2 + 16) <= 156u * 1024u; }

// The few-token forms (K split across waves or workgroups) are used up to ROUTER_FEW_TOKENS tokens, and up to 1024
// where the LDS-resident kernel does not take the gate weights.  Every entry point applies the same rule, so that
// the router gives the same bits whichever of them a caller uses.  Measured, router + sort as the layer calls them,
// hidden size 1536, 40 experts, top-8: few-token form 19.2 / 22.5 / 26 / 35 / 43 us at 256 / 384 / 512 / 768 / 1024
// tokens (its one-block sort is what grows), LDS-resident kernel + scan + scatter 21.4 us from 320 to 4096 tokens.
#define ROUTER_FEW_TOKENS 320
static bool router_few_tokens(int T_, int H, int E) { return T_ <= (router_lds_fits(H, E) ? ROUTER_FEW_TOKENS : 1024); }

static size_t router_ws_bytes(int T_, int H, int E) {
  if (T_ <= 0 || !router_few_tokens(T_, H, E)) return 0;
  return (size_t)router_splits(T_, H) * mi_ceil_div(T_, 16) * 4 * 64 * sizeof(f32x4);
}

template <typename T>
static int launch_router_splitk(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                void* logits_out, void* gates, int32_t* idx, void* ws, hipStream_t s) {
  const int splits = router_splits(T_, H);
  const int steps_per_split = mi_ceil_div(mi_ceil_div(H, 64), splits);
  const int groups = mi_ceil_div(T_, 16);
  hipLaunchKernelGGL((router_splitk_partial_kernel<T>), dim3(groups, splits), dim3(ROUTER_SPLIT_WAVES * 64), 0, s,
                     static_cast<const T*>(x), static_cast<const T*>(gw), T_, H, E, steps_per_split,
                     static_cast<f32x4*>(ws), static_cast<unsigned*>(nullptr));
  int rc = mi_launch_status();
  if (rc != MI_MOE_OK) return rc;
  hipLaunchKernelGGL((router_splitk_finish_kernel<T>), dim3(groups), dim3(256), 0, s, static_cast<const f32x4*>(ws),
                     splits, bias, T_, E, k, static_cast<T*>(logits_out), static_cast<T*>(gates), idx);
  return mi_launch_status();
}

// launch shape of the LDS-resident kernel: workgroups and waves per workgroup
static int router_lds_shape(int T_, int* blocks, int* waves) {
  int cus = 0;
  const int rc = mi_cu_count(&cus);
  if (rc != MI_MOE_OK) return rc;
  const int groups = mi_ceil_div(T_, 16);
  *blocks = groups < cus ? groups : cus;
  int w = mi_ceil_div(groups, *blocks);
  *waves = w > ROUTER_LDS_WAVES ? ROUTER_LDS_WAVES : w;
  return MI_MOE_OK;
}

// `lds`: gate weights (+ gamma); the E counters of the chunk histogram come on top
template <typename T, bool NORM>
static int launch_router_lds(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                             void* logits_out, void* gates, int32_t* idx, RouterNorm norm, size_t lds, hipStream_t s,
                             int32_t* chunk_hist = nullptr, int nchunks = 0) {
  int blocks = 0, waves = 0;
  int rc = router_lds_shape(T_, &blocks, &waves);
  if (rc != MI_MOE_OK) return rc;
  // few groups per workgroup (at most four waves would walk one): the idle waves take shares of the K steps
  // (router_fused_lds_kernel, KS); 3 groups leave two waves without a share
  const int ksplit = waves <= 4 ? (waves == 1 ? 8 : (waves == 2 ? 4 : 2)) : 1;
  size_t bytes = lds + (size_t)E * sizeof(int);
  int red_at = 0, ss_at = 0;
  if (NORM && ksplit > 1) {  // 16 partial sums of squares per wave
    ss_at = (int)((bytes + 15) / 16 * 16);
    bytes = (size_t)ss_at + ROUTER_LDS_WAVES * 16 * sizeof(float);
  }
  if (ksplit > 1) {
    constexpr size_t RED_BYTES = (size_t)ROUTER_LDS_WAVES * 4 * 64 * sizeof(f32x4);  // 32 KB
    if ((size_t)E * ((size_t)H * sizeof(T) + 16) < RED_BYTES) {  // small weights: behind everything else
      red_at = (int)((bytes + 15) / 16 * 16);
      bytes = (size_t)red_at + RED_BYTES;
    }
  }
  auto kern = waves > 4 ? router_fused_lds_kernel<T, 3, NORM, false> : router_fused_lds_kernel<T, 6, NORM, true>;
  const int slot = waves > 4 ? 0 : 1;
  static std::atomic<uint64_t> lds_ok[2];  // the LDS size varies with E and H: opt in to the most it can be
  rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), MI_LDS_MAX_BYTES, lds_ok[slot]);
  if (rc != MI_MOE_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(ROUTER_LDS_WAVES * 64), bytes, s, static_cast<const T*>(x),
                     static_cast<const T*>(gw), bias, T_, H, E, k, static_cast<T*>(logits_out), static_cast<T*>(gates), idx,
                     norm, chunk_hist, nchunks, waves, ksplit, red_at, ss_at);
  return mi_launch_status();
}

template <typename T>
static int launch_router(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                         void* logits_out, void* gates, int32_t* idx, hipStream_t s) {
  if (router_few_tokens(T_, H, E)) {  // split K across the waves of a workgroup instead
    hipLaunchKernelGGL((router_fused_small_kernel<T>), dim3(mi_ceil_div(T_, 16)), dim3(1024), 0, s,
                       static_cast<const T*>(x), static_cast<const T*>(gw), bias, T_, H, E, k,
                       static_cast<T*>(logits_out), static_cast<T*>(gates), idx);
    return mi_launch_status();
  }
  // gate weights fit in LDS next to nothing else: the LDS-resident kernel
  const size_t wbytes = (size_t)E * ((size_t)H * sizeof(T) + 16);
  if (wbytes <= 156u * 1024u) {
    const RouterNorm none = {nullptr, nullptr, 0.f};
    return launch_router_lds<T, false>(x, gw, bias, T_, H, E, k, logits_out, gates, idx, none, wbytes, s);
  }
  hipLaunchKernelGGL((router_fused_ksplit_kernel<T>), dim3(mi_ceil_div(T_, 16 * ROUTER_KS_TG)),
                     dim3(ROUTER_KS_WAVES * 64), 0, s, static_cast<const T*>(x), static_cast<const T*>(gw), bias, T_, H,
                     E, k, static_cast<T*>(logits_out), static_cast<T*>(gates), idx);
  return mi_launch_status();
}

// Router + sort in two launches (split K, the finishing launch sorts in its last workgroup).
// [partial logits][ticket, padded to 256 bytes]
static size_t router_sort_ws_bytes(int T_, int H, int E, int k) {
  const size_t base = router_ws_bytes(T_, H, E);
  if (base == 0 || (long)T_ * k > SORT_SINGLE_BLOCK_MAX) return 0;
  return base + 256;
}

template <typename T>
static int launch_router_splitk_sort(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k,
                                     void* logits_out, void* gates, int32_t* idx, int32_t* sorted_expert,
                                     int32_t* sorted_scattered, int32_t* expert_offsets, void* ws, hipStream_t s) {
  const int splits = router_splits(T_, H);
  const int steps_per_split = mi_ceil_div(mi_ceil_div(H, 64), splits);
  const int groups = mi_ceil_div(T_, 16);
  unsigned* ticket = reinterpret_cast<unsigned*>(static_cast<unsigned char*>(ws) + router_ws_bytes(T_, H, E));
  hipLaunchKernelGGL((router_splitk_partial_kernel<T>), dim3(groups, splits), dim3(ROUTER_SPLIT_WAVES * 64), 0, s,
                     static_cast<const T*>(x), static_cast<const T*>(gw), T_, H, E, steps_per_split,
                     static_cast<f32x4*>(ws), ticket);
  int rc = mi_launch_status();
  if (rc != MI_MOE_OK) return rc;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  hipLaunchKernelGGL((router_splitk_finish_sort_kernel<T>), dim3(groups), dim3(256), 0, s,
                     static_cast<const f32x4*>(ws), splits, bias, T_, E, k, nbits, static_cast<T*>(logits_out),
                     static_cast<T*>(gates), idx, ticket, sorted_expert, sorted_scattered, expert_offsets);
  return mi_launch_status();
}

// Many tokens: router (LDS-resident gate weights) with the sort's histogram pass folded in, then the sort's scan
// and scatter passes (routing.hip) on chunks of waves * 16 tokens.
int mi_sort_after_hist(const int32_t* topk_idx, int L, int E, int chunk, int32_t* sorted_expert,
                       int32_t* sorted_scattered, int32_t* expert_offsets, int32_t* ws, hipStream_t s);

static bool router_hist_shape(int T_, int H, int E, int k, int* chunk_tokens, int* nchunks) {
  if (router_few_tokens(T_, H, E) || (long)T_ * k > 0x7fffffffL - 8192) return false;
  if (!router_lds_fits(H, E)) return false;
  int blocks = 0, waves = 0;
  if (router_lds_shape(T_, &blocks, &waves) != MI_MOE_OK) return false;
  *chunk_tokens = waves * 16;
  *nchunks = mi_ceil_div(T_, *chunk_tokens);
  return true;
}

extern "C" size_t mi_moe_router_fused_sort_workspace_bytes(int T, int H, int E, int k) {
  if (T < 1 || H < 1 || k < 1 || E < 1) return 0;
  const size_t small = router_sort_ws_bytes(T, H, E, k);
  if (small) return small;
  int chunk_tokens = 0, nchunks = 0;
  if (E > 64 || k > ROUTER_KMAX || H % 16 != 0 || !router_hist_shape(T, H, E, k, &chunk_tokens, &nchunks)) return 0;
  return ((size_t)E * nchunks + (size_t)E) * sizeof(int32_t);
}

extern "C" int mi_moe_router_fused_sort(const void* x, const void* gate_w, const float* bias, int T, int H, int E, int k,
                                        int dtype, void* logits_out, void* gates_out, int32_t* idx_out,
                                        int32_t* sorted_expert, int32_t* sorted_scattered, int32_t* expert_offsets,
                                        void* ws, size_t ws_bytes, mi_moe_stream_t stream) {
  if (T < 1 || H < 1 || E < 1 || k < 1 || k > E) return MI_MOE_ESHAPE;
  if (E > 64 || k > ROUTER_KMAX || H % 16 != 0) return MI_MOE_EUNSUPPORTED;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  const size_t need = mi_moe_router_fused_sort_workspace_bytes(T, H, E, k);
  if (need == 0) return MI_MOE_EUNSUPPORTED;  // neither the few-token form nor the LDS-resident form takes the shape
  if (!x || !gate_w || !gates_out || !idx_out || !sorted_expert || !sorted_scattered || !expert_offsets) return MI_MOE_ENULL;
  if (!ws || ws_bytes < need) return MI_MOE_EWORKSPACE;
  if (!mi_aligned(x, 16) || !mi_aligned(gate_w, 16) || !mi_aligned(ws, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (router_sort_ws_bytes(T, H, E, k) != 0) {
    if (dtype == MI_MOE_BF16)
      return launch_router_splitk_sort<bf16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out,
                                               sorted_expert, sorted_scattered, expert_offsets, ws, s);
    return launch_router_splitk_sort<f16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, sorted_expert,
                                            sorted_scattered, expert_offsets, ws, s);
  }
  int chunk_tokens = 0, nchunks = 0;
  router_hist_shape(T, H, E, k, &chunk_tokens, &nchunks);
  const RouterNorm none = {nullptr, nullptr, 0.f};
  const size_t wbytes = (size_t)E * ((size_t)H * 2 + 16);
  int32_t* hist = static_cast<int32_t*>(ws);
  const int rc = dtype == MI_MOE_BF16
                     ? launch_router_lds<bf16_t, false>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out,
                                                        none, wbytes, s, hist, nchunks)
                     : launch_router_lds<f16_t, false>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out,
                                                       none, wbytes, s, hist, nchunks);
  if (rc != MI_MOE_OK) return rc;
  return mi_sort_after_hist(idx_out, T * k, E, chunk_tokens * k, sorted_expert, sorted_scattered, expert_offsets, hist, s);
}

// Many tokens and more than 64 experts (16-bit, no bias): the logits are a product of a size that wants the
// grouped GEMM's tile kernels -- the general kernel re-reads all gate weights from L2 for every 16 tokens.  With
// a workspace the router runs that kernel with ONE expert that owns every row (x rows in place, gate_w as its
// (1, E, H) weight: fp32 accumulation, one rounding, as F.linear), then the top-k kernel on the logits -- in
// logits_out when the caller wants them, else in the workspace.  Measured, 32768 tokens: 128 experts, hidden
// 2048, 177 -> 47 us; 256 experts, hidden 7168, 951 -> 194 us; the crossover is near T * E = 2^20.
static bool router_gemm_form(int T_, int H, int E, int k, int dtype, const float* bias) {
  return dtype != MI_MOE_F32 && bias == nullptr && E > 64 && (long)T_ * E >= (1L << 20) && H % 16 == 0;
}
static size_t router_gemm_form_bytes(int T_, int E) { return ((size_t)T_ * E * 2 + 255) / 256 * 256 + 256; }

__global__ void router_one_expert_offsets_kernel(int32_t* offsets, int rows) {
  if (threadIdx.x == 0 && blockIdx.x == 0) offsets[0] = rows;
}

size_t mi_router_general_ws_bytes(int T_, int H, int E);  // router_general.hip

extern "C" size_t mi_moe_router_fused_workspace_bytes(int T, int H, int E) {
  if (T < 0 || H < 1 || E < 1) return 0;
  if (E > 64) {  // the general kernel's two forms that take a workspace: many tokens / few tokens
    const size_t many = router_gemm_form(T, H, E, 1, MI_MOE_BF16, nullptr) ? router_gemm_form_bytes(T, E) : 0;
    const size_t few = mi_router_general_ws_bytes(T, H, E);
    return many > few ? many : few;
  }
  return router_ws_bytes(T, H, E);
}

// router_general.hip: fp32, 65 .. 256 experts, k up to 64
int mi_router_general_ok(int H, int E, int k, int dtype);
int mi_router_general(const void* x, const void* gw, const float* bias, int T_, int H, int E, int k, int dtype,
                      void* logits_out, void* gates, int32_t* idx, void* ws, hipStream_t s);
size_t mi_router_general_ws_bytes(int T_, int H, int E);

extern "C" int mi_moe_router_fused(const void* x, const void* gate_w, const float* bias, int T, int H, int E, int k,
                                   int dtype, void* logits_out, void* gates_out, int32_t* idx_out, void* ws,
                                   size_t ws_bytes, mi_moe_stream_t stream) {
  if (T < 0 || H < 1 || E < 1 || k < 1 || k > E) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16 && dtype != MI_MOE_F32) return MI_MOE_EDTYPE;
  const bool streaming = dtype != MI_MOE_F32 && E <= 64 && k <= ROUTER_KMAX && H % 16 == 0;
  if (!streaming && !mi_router_general_ok(H, E, k, dtype)) return MI_MOE_EUNSUPPORTED;
  if (T == 0) return MI_MOE_OK;
  if (!x || !gate_w || !gates_out || !idx_out) return MI_MOE_ENULL;
  if (!mi_aligned(x, 16) || !mi_aligned(gate_w, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!streaming) {
    if (ws != nullptr && router_gemm_form(T, H, E, k, dtype, bias)) {
      if (ws_bytes < router_gemm_form_bytes(T, E)) return MI_MOE_EWORKSPACE;
      if (!mi_aligned(ws, 16)) return MI_MOE_EALIGN;
      unsigned char* base = static_cast<unsigned char*>(ws);
      int32_t* offsets = reinterpret_cast<int32_t*>(base + router_gemm_form_bytes(T, E) - 256);
      void* logits = logits_out != nullptr ? logits_out : static_cast<void*>(base);
      hipLaunchKernelGGL(router_one_expert_offsets_kernel, dim3(1), dim3(64), 0, s, offsets, T);
      const int rc = mi_moe_scattered_gemm_ws(x, gate_w, logits, nullptr, offsets, T, H, E, 1, 1, 1, 1, dtype, -1, nullptr,
                                              0, stream);
      if (rc == MI_MOE_OK) return mi_moe_router_topk_softmax(logits, T, E, k, dtype, gates_out, idx_out, stream);
      // a shape the tile kernels do not take (refused before anything of theirs was launched): the general kernel
      if (rc != MI_MOE_EUNSUPPORTED && rc != MI_MOE_EALIGN) return rc;
    }
    void* gws = nullptr;  // few tokens and more than 64 experts: the contraction cut into ranges
    if (ws != nullptr && mi_router_general_ws_bytes(T, H, E) > 0) {
      if (ws_bytes < mi_router_general_ws_bytes(T, H, E)) return MI_MOE_EWORKSPACE;
      if (!mi_aligned(ws, 16)) return MI_MOE_EALIGN;
      gws = ws;
    }
    return mi_router_general(x, gate_w, bias, T, H, E, k, dtype, logits_out, gates_out, idx_out, gws, s);
  }
  const size_t need = router_ws_bytes(T, H, E);
  if (ws != nullptr && need > 0) {  // few tokens and a workspace: K split across workgroups
    if (ws_bytes < need) return MI_MOE_EWORKSPACE;
    if (!mi_aligned(ws, 16)) return MI_MOE_EALIGN;
    if (dtype == MI_MOE_BF16)
      return launch_router_splitk<bf16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, ws, s);
    return launch_router_splitk<f16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, ws, s);
  }
  if (dtype == MI_MOE_BF16) return launch_router<bf16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, s);
  return launch_router<f16_t>(x, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, s);
}

static size_t rmsnorm_router_lds_bytes(int H, int E, size_t elt) {
  return (size_t)E * ((size_t)H * elt + 16) + (size_t)H * sizeof(float);
}

extern "C" int mi_moe_rmsnorm_router_fused_supported(int H, int E, int k, int dtype) {
  if (H < 1 || E < 1 || E > 64 || k < 1 || k > ROUTER_KMAX || k > E || H % 16 != 0) return 0;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return 0;
  return rmsnorm_router_lds_bytes(H, E, 2) <= 156u * 1024u;
}

extern "C" int mi_moe_rmsnorm_router_fused(const void* h, const void* ln_weight, float eps, const void* gate_w,
                                           const float* bias, int T, int H, int E, int k, int dtype,
                                           void* x_norm_out, void* logits_out, void* gates_out, int32_t* idx_out,
                                           mi_moe_stream_t stream) {
  if (T < 0 || H < 1 || E < 1 || k < 1 || k > E) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (!mi_moe_rmsnorm_router_fused_supported(H, E, k, dtype)) return MI_MOE_EUNSUPPORTED;
  if (T == 0) return MI_MOE_OK;
  if (!h || !gate_w || !x_norm_out || !gates_out || !idx_out) return MI_MOE_ENULL;
  if (!mi_aligned(h, 16) || !mi_aligned(gate_w, 16) || !mi_aligned(x_norm_out, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RouterNorm norm = {ln_weight, x_norm_out, eps};
  const size_t lds = rmsnorm_router_lds_bytes(H, E, 2);
  if (dtype == MI_MOE_BF16)
    return launch_router_lds<bf16_t, true>(h, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, norm, lds, s);
  return launch_router_lds<f16_t, true>(h, gate_w, bias, T, H, E, k, logits_out, gates_out, idx_out, norm, lds, s);
}
