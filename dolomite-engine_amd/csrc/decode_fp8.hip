// Decode-shape (few rows per expert) grouped GEMM with fp8 e4m3fn expert weights and one fp32 scale
// per output channel:   out[orow(i), n] = scale[e_i, n] * sum_k in[irow(i), k] * Wq[e_i, n, k]
// optionally with the SwiGLU epilogue (weight rows [0,N) "up", [N,2N) "gate").
//
// The reference has no fp8 expert path (lm_engine/fp8.py:63-73 converts nn.Linear only); the
// semantics are "dequantise, then lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:273-290".
//
// The shape is weight-streaming bound: with ~6 rows per expert every weight byte is used once, so
// the kernel is organised around the weight stream.
//   * grid = experts x column-tile groups; an expert with no rows exits at once, so only the weights
//     of touched experts are read, each exactly once (row groups beyond 16 re-read from L2).
//   * a wavefront owns 16 output channels (x2 for SwiGLU): lane (r = l%16, q = l/16) streams weight
//     row r, 16 consecutive fp8 per load (one dwordx4), i.e. each 64-wide K step is one fully used
//     128-byte line per weight row.  The bytes are widened to bf16/f16 in registers (exact) and used as
//     the A operand of v_mfma_f32_16x16x32; the B operand is the matching 16-row activation slice.
//     A and B use the same lane->k assignment, so no shuffle is needed to match the MFMA's own k order.
//   * KSPLIT wavefronts of a workgroup share one column tile and split K between them (more loads in
//     flight per weight row); partial sums meet in LDS.
//   * the per-channel scale, SwiGLU and the 8-byte packed store happen in the epilogue.
#include "common.h"


template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // 8 fp8 (two dwords) -> 8 bf16; exact, e4m3 fits in bf16
  static __device__ __forceinline__ vec widen(uint32_t lo, uint32_t hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
    bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
    bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
    bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
    vec v = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    return v;
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec widen(uint32_t lo, uint32_t hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 p0 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false);
    f32x2 p1 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
    f32x2 p2 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
    f32x2 p3 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
    vec v = {(f16_t)p0[0], (f16_t)p0[1], (f16_t)p1[0], (f16_t)p1[1],
             (f16_t)p2[0], (f16_t)p2[1], (f16_t)p3[0], (f16_t)p3[1]};
    return v;
  }
};

struct DecodeArgs {
  const void* in;
  const uint8_t* wq;
  const float* scale;
  void* out;
  const int32_t* sorted_scattered;
  const int32_t* expert_offsets;
  int L, K, N, E, kdiv;
  int gather, scatter;
  int groups_per_expert;  // workgroups per expert (streaming kernel: wave units per expert)
  int tiled;              // weights are in the streamed-tile layout (streaming kernel only)
};

template <typename T, bool GLU, int KSPLIT>
__global__ __launch_bounds__(256) void decode_fp8_kernel(DecodeArgs a) {
  constexpr int NTB = 4 / KSPLIT;  // 16-channel column tiles per workgroup
  constexpr int WR = GLU ? 2 : 1;
  typedef typename Mfma16<T>::vec frag_t;
  __shared__ f32x4 red[4][2][64];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int expert = blockIdx.x / a.groups_per_expert;
  const int grp = blockIdx.x - expert * a.groups_per_expert;
  const int row_begin = expert ? a.expert_offsets[expert - 1] : 0;
  const int row_end = a.expert_offsets[expert];
  if (row_begin >= row_end) return;  // whole workgroup: nothing routed here, weights stay untouched

  const int ks = wave % KSPLIT;
  const int n0 = (grp * NTB + wave / KSPLIT) * 16;
  int wrow = n0 + r;
  if (wrow > a.N - 1) wrow = a.N - 1;  // column tail re-reads the last channel; never stored
  const uint8_t* __restrict__ wu = a.wq + ((size_t)expert * WR * a.N + wrow) * a.K;
  const uint8_t* __restrict__ wg = wu + (size_t)a.N * a.K;

  const int ksteps = (a.K + 63) >> 6;
  const int per = (ksteps + KSPLIT - 1) / KSPLIT;
  const int s_begin = ks * per;
  int s_end = s_begin + per;
  if (s_end > ksteps) s_end = ksteps;

  const T* __restrict__ xin = static_cast<const T*>(a.in);
  T* __restrict__ out = static_cast<T*>(a.out);

  for (int g0 = row_begin; g0 < row_end; g0 += 16) {
    int srow = g0 + r;
    if (srow > row_end - 1) srow = row_end - 1;  // short group re-reads the last row; never stored
    const int slot = (a.gather || a.scatter) ? a.sorted_scattered[srow] : 0;
    const int src = a.gather ? slot / a.kdiv : srow;
    const T* __restrict__ xp = xin + (size_t)src * a.K;

    f32x4 acc_u = {0.f, 0.f, 0.f, 0.f}, acc_g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = s_begin; s < s_end; ++s) {
      const int kpos = s * 64 + q * 16;
      u32x4 wub = {0u, 0u, 0u, 0u}, wgb = {0u, 0u, 0u, 0u}, x0 = {0u, 0u, 0u, 0u}, x1 = {0u, 0u, 0u, 0u};
      if (kpos < a.K) {
        wub = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wu + kpos));
        if (GLU) wgb = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wg + kpos));
        x0 = *reinterpret_cast<const u32x4*>(xp + kpos);
        x1 = *reinterpret_cast<const u32x4*>(xp + kpos + 8);
      }
      const frag_t b0 = __builtin_bit_cast(frag_t, x0), b1 = __builtin_bit_cast(frag_t, x1);
      acc_u = Mfma16<T>::run(Mfma16<T>::widen(wub[0], wub[1]), b0, acc_u);
      acc_u = Mfma16<T>::run(Mfma16<T>::widen(wub[2], wub[3]), b1, acc_u);
      if (GLU) {
        acc_g = Mfma16<T>::run(Mfma16<T>::widen(wgb[0], wgb[1]), b0, acc_g);
        acc_g = Mfma16<T>::run(Mfma16<T>::widen(wgb[2], wgb[3]), b1, acc_g);
      }
    }

    if (KSPLIT > 1) {
      if (ks != 0) {
        red[wave][0][lane] = acc_u;
        if (GLU) red[wave][1][lane] = acc_g;
      }
      __syncthreads();
      if (ks == 0) {
#pragma unroll
        for (int o = 1; o < KSPLIT; ++o) {
          f32x4 pu = red[wave + o][0][lane];
          acc_u += pu;
          if (GLU) {
            f32x4 pg = red[wave + o][1][lane];
            acc_g += pg;
          }
        }
      }
      __syncthreads();
    }

    // acc[i]: output channel n0 + 4q + i, row g0 + r
    const int col = n0 + 4 * q;
    if (ks == 0 && g0 + r < row_end && col < a.N) {
      const float* su = a.scale + (size_t)expert * WR * a.N + col;
      const f32x4 scu = *reinterpret_cast<const f32x4*>(su);
      float v[4];
      if (GLU) {
        const f32x4 scg = *reinterpret_cast<const f32x4*>(su + a.N);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (acc_u[i] * scu[i]) * silu_f32(acc_g[i] * scg[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = acc_u[i] * scu[i];
      }
      const int orow = a.scatter ? slot : g0 + r;
      u32x2 p = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
      *reinterpret_cast<u32x2*>(out + (size_t)orow * a.N + col) = p;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Streaming variant: weights and activations reach the matrix cores through per-wave LDS rings filled
// by DMA (global_load_lds_dwordx4).
//
// In the kernel above the lane -> address map is dictated by the MFMA operand layout (lane = 16*q + r
// reads row r): neighbouring lanes touch different rows, every 16-byte access is its own cache-line
// lookup, and the address path, not HBM, sets the pace.  Here the global side is laid out for the
// memory system -- 8 neighbouring lanes read one full 128-byte line of a weight row, 16 neighbouring
// lanes 256 bytes of an activation row -- and the MFMA layout is recovered by where the ds_reads look.
//
//   wave       = 32 weight rows over the whole K (SwiGLU: 16 up + 16 gate rows -> 16 output channels);
//                the four waves of a workgroup are independent: no barrier, no cross-wave sum, and two
//                workgroups fit on a CU
//   ring       = NS stages per wave; stage = [32 rows][128 B] fp8 weights + [XT rows][256 B] activations
//   stage      : lane (r, q) takes k [32q, 32q+32) of the stage: per 16-row block two 16-byte weight
//                reads and four MFMA 16x16x32, plus four 16-byte activation reads
//   activations: an expert with at most 8 rows (the decode case) runs one pass with XT = 8 and a
//                three-stage ring (MFMA columns 8..15 mirror 0..7 and are never stored); more rows run
//                passes of 16 with a two-stage ring.  Only ceil(rows/4)*4 rows are fetched.
// Measured against an empty kernel that merely streams the same bytes through the same ring (no LDS reads,
// no MFMA; 6.7 - 6.8 TB/s with non-temporal DMA) this kernel is within 5 - 10 %.
// Needs K % 128 == 0; other shapes take the kernel above.
// ------------------------------------------------------------------------------------------------

// LDS per wave: three stages of [32 x 128] weights + [8 x 256] activations (= two stages with 16 rows)
#define DEC_WAVE_LDS (3 * (32 * 128 + 8 * 256))
// Cache policy of the weight DMA (auxiliary operand of global_load_lds; 1 = sc0, 2 = nt, 16 = sc1).  Every weight
// byte is used once, and non-temporal loads stream measurably faster on this part: up-projection of the 64-token
// shape 131 -> 120 us, down-projection 70 -> 67 us (a plain register-load stream of the same bytes: 6.0 -> 6.9
// TB/s).  sc0 / sc1, alone or with nt, change nothing.
#define DEC_W_POLICY 2

__device__ __forceinline__ constexpr int dec_waitcnt(int vm, int lgkm) {
  return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}

template <int V> struct dec_int { static constexpr int value = V; };

// LDS chunk swizzles of a ring stage.  A ds_read_b128 is served in four passes of 16 lanes -- lanes
// [8p, 8p+8) together with [16+8p, 24+8p) -- i.e. 8 consecutive rows x 2 of a lane row's chunks.  For the
// weight rows (128 B: two rows span the 64 banks) the two chunks differ by 2, for the activation rows (256 B)
// by 4; the XOR masks below put the 16 accesses of every pass in 16 different 16-byte bank groups.
__device__ __forceinline__ int dec_wswz(int t) { return ((t >> 1) & 1) | (((t >> 2) & 1) << 2); }
__device__ __forceinline__ int dec_xswz(int r) { return (r & 3) | ((r & 4) << 1); }

// TILED: the weights are stored as the kernel streams them -- [expert][wave unit][K stage][4 KB], each 4 KB block
// being the LDS image of one ring stage (32 rows x 128 B, chunk slots already swizzled).  A wave then reads one
// contiguous 128 KB run instead of 32 rows 4 KB apart: 5.1 -> 6.1 TB/s for an empty kernel streaming this
// workload's up-projection weights.  (Row-major weights keep working; the module tiles them when it quantises.)
// The launch decides how many waves form a workgroup: they never synchronise.
template <typename T, bool GLU, bool TILED>
__global__ __launch_bounds__(256) void decode_fp8_stream_kernel(DecodeArgs a) {
  constexpr int KCH = 128;                       // k per ring stage
  constexpr int WR = GLU ? 2 : 1;
  constexpr int CHW = GLU ? 16 : 32;             // output channels per wave
  constexpr int NWI = 4;                         // weight DMA instructions per stage (8 rows x 128 B each)
  constexpr int W_BYTES = 32 * KCH;
  constexpr int NM = KCH / 32;                   // MFMA k-steps per stage
  typedef typename Mfma16<T>::vec frag_t;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* glb_ptr_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char dsm[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, q = lane >> 4;
  // a.groups_per_expert = wave units (CHW channels each) per expert; blockDim.x / 64 units share a workgroup
  const int unit = blockIdx.x * (int)(blockDim.x >> 6) + wave;
  const int expert = unit / a.groups_per_expert;
  if (expert >= a.E) return;
  const int row_begin = expert ? a.expert_offsets[expert - 1] : 0;
  const int row_end = a.expert_offsets[expert];
  if (row_begin >= row_end) return;  // nothing routed here: the expert's weights stay untouched
  const int n0 = (unit - expert * a.groups_per_expert) * CHW;
  if (n0 >= a.N) return;             // (waves do not synchronise)

  unsigned char* ring = dsm + wave * DEC_WAVE_LDS;

  // weight DMA: instruction j fills ring rows [8j, 8j+8): lane -> row 8j + lane/8, slot lane%8 holding
  // logical chunk slot ^ dec_wswz(row)
  const unsigned char* wexp = a.wq + (size_t)expert * WR * a.N * a.K;
  uint32_t woff[NWI];
#pragma unroll
  for (int j = 0; j < NWI; ++j) {
    const int t = 8 * j + (lane >> 3);                      // ring row 0..31
    int ch;                                                 // weight row inside the expert
    if (GLU) {
      ch = t < 16 ? n0 + t : a.N + n0 + (t - 16);
      const int lim = (t < 16 ? a.N : 2 * a.N) - 1;
      if (ch > lim) ch = lim;                               // channel tail re-reads the last row; never stored
    } else {
      ch = n0 + t;
      if (ch > a.N - 1) ch = a.N - 1;
    }
    woff[j] = (uint32_t)ch * (uint32_t)a.K + ((lane & 7) ^ dec_wswz(t)) * 16;
  }

  const int nst = a.K / KCH;
  // tiled weights: this unit's K stages are consecutive 4 KB blocks
  const unsigned char* wtile = a.wq + (size_t)unit * nst * W_BYTES + lane * 16;
  const T* __restrict__ xin = static_cast<const T*>(a.in);
  T* __restrict__ out = static_cast<T*>(a.out);

  // One pass over K for the activation rows [g0, g0 + XT): ring of NS stages, NX activation DMA
  // instructions per stage (4 rows each).
  auto pass = [&](int g0, auto xt_tag, auto ns_tag, auto nx_tag) {
    constexpr int XT = decltype(xt_tag)::value;
    constexpr int NS = decltype(ns_tag)::value;
    constexpr int NX = decltype(nx_tag)::value;
    constexpr int STAGE = W_BYTES + XT * KCH * 2;
    constexpr int NDMA = NWI + NX;
    static_assert(NS * STAGE <= DEC_WAVE_LDS, "ring does not fit");
    // activation DMA: instruction j fills ring rows [4j, 4j+4): lane -> row 4j + lane/16, slot lane%16
    // holding logical chunk slot ^ dec_xswz(row)
    const T* xsrc[NX];
#pragma unroll
    for (int j = 0; j < NX; ++j) {
      const int t = 4 * j + (lane >> 4);
      int srow = g0 + t;
      if (srow > row_end - 1) srow = row_end - 1;           // short pass re-reads the last row; never stored
      const int src = a.gather ? a.sorted_scattered[srow] / a.kdiv : srow;
      xsrc[j] = xin + (size_t)src * a.K + (((lane & 15) ^ dec_xswz(t)) * 8);
    }
    auto dma_stage = [&](int st, int slot) {
      const int stc = st < nst ? st : nst - 1;               // surplus rounds re-fetch the last stage
      unsigned char* dst = ring + slot * STAGE;
      if (TILED) {
        const unsigned char* wk = wtile + (size_t)stc * W_BYTES;
#pragma unroll
        for (int j = 0; j < NWI; ++j)
          __builtin_amdgcn_global_load_lds((glb_ptr_t)(wk + j * 1024), (lds_ptr_t)(dst + j * 1024), 16, 0, DEC_W_POLICY);
      } else {
        const unsigned char* wk = wexp + (size_t)stc * KCH;
#pragma unroll
        for (int j = 0; j < NWI; ++j)
          __builtin_amdgcn_global_load_lds((glb_ptr_t)(wk + woff[j]), (lds_ptr_t)(dst + j * 1024), 16, 0, DEC_W_POLICY);
      }
#pragma unroll
      for (int j = 0; j < NX; ++j)
        __builtin_amdgcn_global_load_lds((glb_ptr_t)(xsrc[j] + (size_t)stc * KCH),
                                         (lds_ptr_t)(dst + W_BYTES + j * 1024), 16, 0, 0);
    };

    // What the epilogue needs from memory -- this lane's output row and channel scales -- is requested first, ahead
    // of the ring's DMA: by the end of the pass it has long arrived, and the pass does not end on a load's latency.
    // (Being the oldest requests of the wave, they also retire first: the ring's counted waits stay as they are.)
    const bool store_lane = r < XT && g0 + r < row_end;
    int orow = g0 + r;
    f32x4 sc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};   // SwiGLU: up / gate; else: channel blocks 0 / 1
    if (store_lane) {
      if (a.scatter) orow = a.sorted_scattered[g0 + r];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int col = GLU ? n0 + 4 * q : n0 + 16 * b + 4 * q;
        if (col < a.N)
          sc[b] = *reinterpret_cast<const f32x4*>(a.scale + (size_t)expert * WR * a.N + (GLU ? b * a.N : 0) + col);
      }
    }

    f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const int xr = r & (XT - 1);                             // XT = 8: columns 8..15 mirror 0..7
#pragma unroll
    for (int p = 0; p < NS; ++p) dma_stage(p, p);
    int slot = 0;
    // stage i: wait until at most VM younger DMA instructions are in flight, move the stage to registers, refill
    // its slot (ISSUE) and run the matrix instructions
    auto step = [&](auto vm_tag, auto issue_tag, int i) {
      constexpr int VM = decltype(vm_tag)::value;
      constexpr bool ISSUE = decltype(issue_tag)::value != 0;
      __builtin_amdgcn_s_waitcnt(dec_waitcnt(VM, 15));               // stage i has landed
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      const unsigned char* ws = ring + slot * STAGE;
      const unsigned char* xs = ws + W_BYTES;
      frag_t xb[NM];
#pragma unroll
      for (int m = 0; m < NM; ++m)
        xb[m] = __builtin_bit_cast(frag_t,
                                   *reinterpret_cast<const u32x4*>(xs + xr * (KCH * 2) + (((q * NM + m) ^ dec_xswz(xr)) * 16)));
      // the whole stage goes to registers first, so that its slot can be refilled before the arithmetic
      u32x4 wv[2][NM / 2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int t = 16 * b + r;
#pragma unroll
        for (int h = 0; h < NM / 2; ++h)
          wv[b][h] = *reinterpret_cast<const u32x4*>(ws + t * KCH + (((q * (NM / 2) + h) ^ dec_wswz(t)) * 16));
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(dec_waitcnt(63, 0));                // my reads of this slot are done
      if (ISSUE) dma_stage(i + NS, slot);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int h = 0; h < NM / 2; ++h) {
          acc[b] = Mfma16<T>::run(Mfma16<T>::widen(wv[b][h][0], wv[b][h][1]), xb[2 * h], acc[b]);
          acc[b] = Mfma16<T>::run(Mfma16<T>::widen(wv[b][h][2], wv[b][h][3]), xb[2 * h + 1], acc[b]);
        }
      slot = slot + 1 == NS ? 0 : slot + 1;
    };
    static_assert(NS == 2 || NS == 3, "the unrolled tail below");
    if (nst >= NS) {
      for (int i = 0; i < nst - NS; ++i) step(dec_int<(NS - 1) * NDMA>{}, dec_int<1>{}, i);
      // the last NS stages are all requested: nothing is issued any more and the waits count down
      if constexpr (NS == 3) step(dec_int<2 * NDMA>{}, dec_int<0>{}, 0);
      step(dec_int<NDMA>{}, dec_int<0>{}, 0);
      step(dec_int<0>{}, dec_int<0>{}, 0);
    } else {
      // fewer stages than the ring has slots: the prologue's surplus requests re-fetched the last stage
      for (int i = 0; i < nst; ++i) step(dec_int<(NS - 1) * NDMA>{}, dec_int<1>{}, i);
      __builtin_amdgcn_s_waitcnt(dec_waitcnt(0, 0));                 // surplus DMA must not outlive the wave's LDS
    }

    // acc[b][i]: weight row 16b + 4q + i of this wave, activation row g0 + r
    if (store_lane) {
      if (GLU) {
        const int col = n0 + 4 * q;
        if (col < a.N) {
          float v[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = (acc[0][i] * sc[0][i]) * silu_f32(acc[1][i] * sc[1][i]);
          const u32x2 p = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
          *reinterpret_cast<u32x2*>(out + (size_t)orow * a.N + col) = p;
        }
      } else {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int col = n0 + 16 * b + 4 * q;
          if (col < a.N) {
            const u32x2 p = {pack2<T>(acc[b][0] * sc[b][0], acc[b][1] * sc[b][1]),
                             pack2<T>(acc[b][2] * sc[b][2], acc[b][3] * sc[b][3])};
            *reinterpret_cast<u32x2*>(out + (size_t)orow * a.N + col) = p;
          }
        }
      }
    }
  };

  const int n_rows = row_end - row_begin;
  if (n_rows <= 4) {
    pass(row_begin, dec_int<8>{}, dec_int<3>{}, dec_int<1>{});
  } else if (n_rows <= 8) {
    pass(row_begin, dec_int<8>{}, dec_int<3>{}, dec_int<2>{});
  } else {
    for (int g0 = row_begin; g0 < row_end; g0 += 16) pass(g0, dec_int<16>{}, dec_int<2>{}, dec_int<4>{});
  }
}

template <typename T, bool GLU>
static int launch_decode_stream(DecodeArgs a, hipStream_t s) {
  constexpr int CHW = GLU ? 16 : 32;
  a.groups_per_expert = mi_ceil_div(a.N, CHW);
  const long units = (long)a.E * a.groups_per_expert;
  // one wave per workgroup: units are dispatched one by one as waves retire (measured 6.1 vs 5.6 TB/s for the
  // contiguous stream with four-wave workgroups); eight fit a CU by LDS
  const int waves = a.tiled ? 1 : 4;
  const int lds = waves * DEC_WAVE_LDS;
  auto kern = a.tiled ? decode_fp8_stream_kernel<T, GLU, true> : decode_fp8_stream_kernel<T, GLU, false>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_ok[2];  // one mask per kernel of this instantiation (tiled / row-major)
    const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), lds, lds_ok[a.tiled ? 1 : 0]);
    if (rc != MI_MOE_OK) return rc;
  }
  const long grid = (units + waves - 1) / waves;
  if (grid > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(waves * 64), lds, s, a);
  return mi_launch_status();
}

template <typename T, bool GLU, int KSPLIT>
static int launch_decode(DecodeArgs a, hipStream_t s) {
  constexpr int NTB = 4 / KSPLIT;
  a.groups_per_expert = mi_ceil_div(a.N, 16 * NTB);
  long grid = (long)a.E * a.groups_per_expert;
  if (grid > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL((decode_fp8_kernel<T, GLU, KSPLIT>), dim3((unsigned)grid), dim3(256), 0, s, a);
  return mi_launch_status();
}

template <typename T, bool GLU>
static int dispatch_decode(const DecodeArgs& a, hipStream_t s) {
  // the streaming kernel needs whole 128-wide K stages and 32-bit weight offsets inside one expert
  if (a.K % 128 == 0 && (a.K >= 512 || a.tiled) && (double)(GLU ? 2 : 1) * a.N * a.K < 4.0e9)
    return launch_decode_stream<T, GLU>(a, s);
  if (a.tiled) return MI_MOE_EUNSUPPORTED;  // the tile layout exists for whole 128-wide K stages only
  if (a.K >= 2048) return launch_decode<T, GLU, 4>(a, s);
  if (a.K >= 1024) return launch_decode<T, GLU, 2>(a, s);
  return launch_decode<T, GLU, 1>(a, s);
}

// grouped_gemm.hip: the same product on the register-staged tile kernels, fp8 bytes widened on their way into LDS
int mi_gemm_fp8_tiled(const void* in, const void* wq, const float* scale, void* out, const int32_t* sorted_scattered,
                      const int32_t* expert_offsets, int L, int K, int N, int E, int kdiv, int gather, int scatter,
                      int glu, int w_tiled, int dtype, hipStream_t s);

// Rows per expert (on average) from which the tile kernels take over: the streaming kernels read an expert's
// weights once per 16 of its rows, a tile kernel once per row tile.  Measured on 64 experts of 2 x 1408 x 4096 and
// 4096 x 1408 weights, top-6, both projections: 12 rows per expert 224 us streaming / 266 us tiles, 18 rows 339 / 273,
// 48 rows 762 / 383, 96 rows 1448 / 410.
#define FP8_TILED_MIN_ROWS 16

static int run_decode(DecodeArgs a, int dtype, bool glu, hipStream_t s, int form) {
  if (a.L < 0 || a.K < 1 || a.N < 1 || a.E < 1 || a.kdiv < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (a.L == 0) return MI_MOE_OK;
  if (!a.in || !a.wq || !a.scale || !a.out || !a.expert_offsets) return MI_MOE_ENULL;
  if ((a.gather || a.scatter) && !a.sorted_scattered) return MI_MOE_ENULL;
  if (a.K % 16 != 0 || a.N % 4 != 0) return MI_MOE_EUNSUPPORTED;
  // form: 0 by the batch, 1 the streaming kernels, 2 the tile kernels
  if (form == 2 || (form == 0 && (long)a.L >= (long)FP8_TILED_MIN_ROWS * a.E))
    return mi_gemm_fp8_tiled(a.in, a.wq, a.scale, a.out, a.sorted_scattered, a.expert_offsets, a.L, a.K, a.N, a.E,
                             a.kdiv, a.gather, a.scatter, glu ? 1 : 0, a.tiled ? 1 : 0, dtype, s);
  if (!mi_aligned(a.in, 16) || !mi_aligned(a.wq, 16) || !mi_aligned(a.scale, 16) || !mi_aligned(a.out, 8))
    return MI_MOE_EALIGN;
  if (dtype == MI_MOE_BF16) return glu ? dispatch_decode<bf16_t, true>(a, s) : dispatch_decode<bf16_t, false>(a, s);
  return glu ? dispatch_decode<f16_t, true>(a, s) : dispatch_decode<f16_t, false>(a, s);
}

extern "C" size_t mi_moe_fp8_tiled_bytes(int E, int N, int K, int glu) {
  if (E < 1 || N < 1 || K < 128 || K % 128 != 0) return 0;
  const int chw = glu ? 16 : 32;
  return (size_t)E * mi_ceil_div(N, chw) * (size_t)(K / 128) * 4096;
}

// cfg: -1 picks by the batch (tile kernels from FP8_TILED_MIN_ROWS rows per expert on average), 0 the streaming
// kernels, 1 the tile kernels
static int fp8_form(int cfg) { return cfg < 0 ? 0 : (cfg == 0 ? 1 : 2); }

extern "C" int mi_moe_up_swiglu_fp8_cfg(const void* x, const void* w_fc_q, const float* w_fc_scale, void* act_out,
                                        const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int H,
                                        int I, int E, int k, int dtype, int w_tiled, int cfg, mi_moe_stream_t stream) {
  if (cfg < -1 || cfg > 1) return MI_MOE_EUNSUPPORTED;
  DecodeArgs a;
  a.in = x; a.wq = static_cast<const uint8_t*>(w_fc_q); a.scale = w_fc_scale; a.out = act_out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = H; a.N = I; a.E = E; a.kdiv = k; a.gather = 1; a.scatter = 0; a.groups_per_expert = 0;
  a.tiled = w_tiled != 0;
  return run_decode(a, dtype, true, static_cast<hipStream_t>(stream), fp8_form(cfg));
}

extern "C" int mi_moe_up_swiglu_fp8(const void* x, const void* w_fc_q, const float* w_fc_scale, void* act_out,
                                    const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int H,
                                    int I, int E, int k, int dtype, int w_tiled, mi_moe_stream_t stream) {
  return mi_moe_up_swiglu_fp8_cfg(x, w_fc_q, w_fc_scale, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype,
                                  w_tiled, -1, stream);
}

extern "C" int mi_moe_down_fp8_cfg(const void* act, const void* w_proj_q, const float* w_proj_scale, void* o_out,
                                   const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int I, int H,
                                   int E, int dtype, int w_tiled, int cfg, mi_moe_stream_t stream) {
  if (cfg < -1 || cfg > 1) return MI_MOE_EUNSUPPORTED;
  DecodeArgs a;
  a.in = act; a.wq = static_cast<const uint8_t*>(w_proj_q); a.scale = w_proj_scale; a.out = o_out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = I; a.N = H; a.E = E; a.kdiv = 1; a.gather = 0; a.scatter = 1; a.groups_per_expert = 0;
  a.tiled = w_tiled != 0;
  return run_decode(a, dtype, false, static_cast<hipStream_t>(stream), fp8_form(cfg));
}

extern "C" int mi_moe_down_fp8(const void* act, const void* w_proj_q, const float* w_proj_scale, void* o_out,
                               const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int I, int H,
                               int E, int dtype, int w_tiled, mi_moe_stream_t stream) {
  return mi_moe_down_fp8_cfg(act, w_proj_q, w_proj_scale, o_out, sorted_scattered, expert_offsets, L, I, H, E, dtype,
                             w_tiled, -1, stream);
}

// ---- fp8 weights -> 16-bit weights with the channel scale folded in ----------------------------------------------
// The kernels above stream an expert's weights once per 16 of its rows: right for decode, linear in the batch
// beyond that.  For batches with many rows per expert the caller widens the weights once per call (w * scale in
// fp32, one rounding) into a scratch tensor of the activation dtype and runs the tiled 16-bit grouped GEMM on it.
// One thread per 16-byte piece of a weight row; reads either layout, writes (E, rows, K) row-major.
template <typename T>
__global__ __launch_bounds__(256) void fp8_dequant_kernel(const uint8_t* __restrict__ wq, const float* __restrict__ scale,
                                                          T* __restrict__ out, long pieces, int N, int K, int glu,
                                                          int tiled) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= pieces) return;
  const int ppr = K >> 4;                // pieces per row
  const long grow = id / ppr;            // row over all experts
  const int c16 = (int)(id - grow * ppr);
  size_t src = (size_t)id * 16;
  if (tiled) {
    const int R = glu ? 2 * N : N;
    const long e = grow / R;
    const int row = (int)(grow - e * R);
    const int half = (glu && row >= N) ? 1 : 0;
    const int n = row - half * N;
    const int chw = glu ? 16 : 32;
    const int U = (N + chw - 1) / chw;
    const int u = n / chw;
    const int t = n - u * chw + 16 * half;  // row inside the 32-row stage image
    const int stage = c16 >> 3, c = c16 & 7;
    const int slot = c ^ (((t >> 1) & 1) | (((t >> 2) & 1) << 2));
    src = (((((size_t)e * U + u) * (size_t)(K >> 7) + stage) * 32 + t) * 8 + slot) * 16;
  }
  const u32x4 v = *reinterpret_cast<const u32x4*>(wq + src);
  const float sc = scale[grow];
  u32x4 o[2];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(v[d], false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(v[d], true);
    // the product is rounded to fp32 and then to T, as `(w.float() * scale).to(T)` does: left alone, the compiler
    // fuses product and conversion to fp16 into one fma with a zero addend (one rounding, and -0 becomes +0)
    float p[4] = {lo[0] * sc, lo[1] * sc, hi[0] * sc, hi[1] * sc};
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(p[i]));
    o[d >> 1][(d & 1) * 2] = pack2<T>(p[0], p[1]);
    o[d >> 1][(d & 1) * 2 + 1] = pack2<T>(p[2], p[3]);
  }
  u32x4* dst = reinterpret_cast<u32x4*>(out + (size_t)id * 16);
  dst[0] = o[0];
  dst[1] = o[1];
}

extern "C" int mi_moe_fp8_dequant(const void* w_q, const float* w_scale, void* w_out, int E, int out, int in, int glu,
                                  int w_tiled, int dtype, mi_moe_stream_t stream) {
  if (E < 1 || out < 1 || in < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (in % 16 != 0 || (w_tiled && in % 128 != 0)) return MI_MOE_EUNSUPPORTED;
  if (!w_q || !w_scale || !w_out) return MI_MOE_ENULL;
  if (!mi_aligned(w_q, 16) || !mi_aligned(w_out, 16)) return MI_MOE_EALIGN;
  const long rows = (long)E * (glu ? 2 : 1) * out;
  const long pieces = rows * (in / 16);
  const long blocks = (pieces + 255) / 256;
  if (blocks > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MI_MOE_BF16)
    hipLaunchKernelGGL((fp8_dequant_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const uint8_t*>(w_q), w_scale, static_cast<bf16_t*>(w_out), pieces, out, in, glu,
                       w_tiled);
  else
    hipLaunchKernelGGL((fp8_dequant_kernel<f16_t>), dim3((unsigned)blocks), dim3(256), 0, s,
                       static_cast<const uint8_t*>(w_q), w_scale, static_cast<f16_t*>(w_out), pieces, out, in, glu,
                       w_tiled);
  return mi_launch_status();
}
