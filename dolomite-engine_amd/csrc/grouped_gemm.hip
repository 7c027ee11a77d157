// Grouped ("scatter2scatter") GEMM of the scattered-MoE forward on gfx950 matrix cores.
//
//   out[orow(i), :] = in[irow(i), :] @ W[e_i]^T        for every row i of the expert-sorted order
//
// with an optional SwiGLU epilogue (W rows [0,N) are "up", [N,2N) "gate"; out = up * silu(gate)).
// Stands in for the external scattered_experts op called at
// lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:91-101 (call sites moe.py:273-290) and for
// GLUActivation (activations/glu.py:42-43) when fused.
//
// Kernels in this file, in order:
//   grouped_gemm_kernel             register-staged tiles (any K that is a multiple of one 16-byte chunk; bf16, fp16
//                                   and fp32): the design notes below
//   grouped_gemm_dma_kernel         the same tile with the operands brought to LDS by DMA, one tile per workgroup
//   grouped_gemm_persistent_kernel  one workgroup per CU walking a list of 256 x 256 tiles, two wave groups in
//                                   ping-pong (large expert loads; its notes stand in front of it), with
//   grouped_gemm_split_finish_kernel  for the tiles of a last round that were cut along K
//   grouped_gemm_naive_kernel       one thread per output element, only on request (cfg 3)
//
// Design
//   * One workgroup computes a BM x BN output tile of ONE expert.  The tile list is not built on the
//     host (that would need the per-expert counts, i.e. a device->host sync): every workgroup derives
//     "its" (expert, row-tile, column-tile) from the E inclusive offsets with a short scalar scan.  The
//     grid is the host-side upper bound floor(L/BM)+min(E,L) row tiles; surplus workgroups exit.
//   * Workgroup ids are re-mapped so that each of the 8 XCDs (ids are dealt round-robin to XCDs)
//     works on a contiguous range of tiles: neighbouring tiles share the gathered activation rows
//     (column tiles of one row tile) and the expert's weight matrix, which then stay in that XCD's L2.
//   * Both operands are K-contiguous in HBM (activations (rows, K), weights (E, N, K)), so both are
//     fetched as 16-byte chunks, staged in LDS with an XOR swizzle (conflict-free ds_write_b128 /
//     ds_read_b128) and fed to v_mfma_f32_32x32x16 as the A (weights) and B (activations) operands.
//     With the weights as operand A each lane ends up with 4 consecutive output columns of one row,
//     so the epilogue packs 4 results into one 8-byte store.
//   * Two LDS stages: the global loads of K-tile i+1 are issued before the MFMAs of tile i and
//     written to the other stage afterwards; one barrier per K-tile.
#include "common.h"

#include <type_traits>

template <typename T> struct Mfma32;
template <> struct Mfma32<bf16_t> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma32<f16_t> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// fp32 operands: a 16-byte chunk holds four k values; the lane halves (lane / 32) hold different chunks, so four
// 32x32x2 instructions -- element i of both operands -- consume the eight k values of a chunk pair.  Which k a
// lane contributes in which step does not matter as long as both operands use the same assignment.
template <> struct Mfma32<float> {
  typedef f32x4 vec;
  static __device__ __forceinline__ f32x16 run(vec a, vec b, f32x16 c) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i], c, 0, 0, 0);
    return c;
  }
};

// 16x16x32: half the flops per instruction and the same rate, but a quarter of the accumulator traffic
// per flop.  Under the chip's power limit (random operands) it sustains about 30 % more throughput than
// 32x32x16, so the persistent ping-pong kernel uses it.
template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x4 run(vec a, vec b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct GemmArgs {
  const void* in;
  const void* w;
  void* out;
  const int32_t* sorted_scattered;
  const int32_t* expert_offsets;
  int L;        // rows of the sorted order
  int K;        // contraction length
  int N;        // output columns (SwiGLU: I, with 2N weight rows per expert)
  int E;
  int kdiv;     // gather divisor (top-k) for scattered inputs
  int kshift;   // log2(kdiv) if kdiv is a power of two, else -1 (set by launch_persistent)
  int n_tiles;  // column tiles per row tile
  int gather;   // input row of sorted row i is sorted_scattered[i] / kdiv (else i)
  int scatter;  // output row of sorted row i is sorted_scattered[i] (else i)
  int remap;    // XCD-aware tile order
  void* ws;     // persistent kernel: workspace for splitting the last round of tiles along K (or null)
  void* pre;    // persistent SwiGLU kernel: (L, 2N) pre-activation output next to the activation (or null)
  int out_nt;   // persistent kernel: store the output non-temporal (set in run_gemm)
  // fp8 weights (register-staged kernel, W8 form): w holds e4m3fn bytes, row-major (E, rows, K) or in the streamed-tile
  // layout of decode_fp8.hip; wscale (E, rows) fp32 is applied to the accumulators in the epilogue
  const float* wscale;
  int w_tiled;
};

// 8 fp8 e4m3fn values (two dwords) -> 8 values of a 16-bit type (exact: e4m3 fits in either)
template <typename T> struct Widen8;
template <> struct Widen8<bf16_t> {
  static __device__ __forceinline__ u32x4 run(uint32_t lo, uint32_t hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
    const bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
    const bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
    const bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
    return (u32x4){__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1), __builtin_bit_cast(uint32_t, p2),
                   __builtin_bit_cast(uint32_t, p3)};
  }
};
template <> struct Widen8<f16_t> {
  static __device__ __forceinline__ u32x4 run(uint32_t lo, uint32_t hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 p0 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false), p1 = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
    const f32x2 p2 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false), p3 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
    return (u32x4){pack2<f16_t>(p0[0], p0[1]), pack2<f16_t>(p1[0], p1[1]), pack2<f16_t>(p2[0], p2[1]),
                   pack2<f16_t>(p3[0], p3[1])};
  }
};
template <> struct Widen8<float> {  // (not used: fp32 activations have no fp8 form)
  static __device__ __forceinline__ u32x4 run(uint32_t, uint32_t) { return (u32x4){0u, 0u, 0u, 0u}; }
};


// Tile -> (expert, row range, column tile).  Row tiles are numbered expert by expert (expert e has
// ceil(n_e / BM) of them), column tiles innermost.  The walk over the E inclusive offsets is done by
// one wavefront 64 experts at a time (one coalesced load + a shuffle scan) instead of E dependent
// scalar loads; every wave of the workgroup does it redundantly, so no LDS or barrier is involved.
// With `remap` the workgroup ids (dealt round-robin to the 8 XCDs) are permuted so that each XCD
// owns a contiguous range of tiles.  Returns false for surplus workgroups.
struct TileCoord {
  int expert, row_begin, row_end, nt;
};

template <int BM>
__device__ __forceinline__ bool decode_tile(const int32_t* __restrict__ off, int E, int n_tiles, int remap,
                                            TileCoord& tc) {
  const int lane = threadIdx.x & 63;
  // pass 1: total number of row tiles
  int total_m = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int end = e < E ? off[e] : 0;
    const int prev = (e < E && e > 0) ? off[e - 1] : 0;
    int t = e < E ? (end - prev + BM - 1) / BM : 0;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) t += __shfl_xor(t, o, 64);
    total_m += t;
  }
  const int total = total_m * n_tiles;
  int tile;
  if (remap & 1) {
    const int per = (total + 7) >> 3;
    const int local = blockIdx.x >> 3;
    if (local >= per) return false;
    tile = (blockIdx.x & 7) * per + local;
  } else {
    tile = blockIdx.x;
  }
  if (tile >= total) return false;
  const int mt = tile / n_tiles;
  tc.nt = tile - mt * n_tiles;
  // pass 2: the expert whose row tiles contain mt
  int carry = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int end = e < E ? off[e] : 0;
    const int prev = (e < E && e > 0) ? off[e - 1] : 0;
    const int t = e < E ? (end - prev + BM - 1) / BM : 0;
    int incl = t;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    incl += carry;
    const uint64_t hit = __ballot(incl > mt);
    if (hit) {
      const int src = __ffsll((long long)hit) - 1;
      const int first_tile = __shfl(incl - t, src, 64);
      const int p = __shfl(prev, src, 64);
      tc.expert = e0 + src;
      tc.row_begin = p + (mt - first_tile) * BM;
      tc.row_end = __shfl(end, src, 64);
      return true;
    }
    carry = __shfl(incl, 63, 64);
  }
  return false;
}

// scheduling-group masks of __builtin_amdgcn_sched_group_barrier
#define SG_MFMA 0x008
#define SG_VMEM_RD 0x020
#define SG_DS_RD 0x100
#define SG_DS_WR 0x200

// W8: the weights are fp8 e4m3fn bytes with one fp32 scale per weight row (a.wscale); a thread fetches the 8 bytes
// of its chunk and widens them on their way into LDS, the scale meets the accumulators in the epilogue.  For batches
// between decode (decode_fp8.hip streams an expert's weights once per 16 rows) and the sizes where widening all
// weights first pays (mi_moe_fp8_dequant).
template <typename T, int BM, int BNW, int WM, int WN, bool GLU, bool KTAIL, bool W8 = false>
__global__ __launch_bounds__(WM* WN * 64) void grouped_gemm_kernel(GemmArgs a) {
  static_assert(!W8 || sizeof(T) == 2, "fp8 weights go with 16-bit activations");
  constexpr int CE = 16 / sizeof(T);        // elements per 16-byte chunk (8 for the 16-bit types, 4 for fp32)
  constexpr int BK = 8 * CE;                // K tile: 128 bytes per row
  constexpr int NT = WM * WN * 64;
  constexpr int CPR = BK / CE;              // 16-byte chunks per tile row
  constexpr int RS = NT / CPR;              // tile rows covered by one pass of the workgroup
  constexpr int XCH = BM * CPR / NT;        // chunks per thread, activation tile
  constexpr int WCH = BNW * CPR / NT;       // chunks per thread, weight tile
  constexpr int BN = GLU ? BNW / 2 : BNW;   // output columns per tile
  constexpr int WTM = BM / WM;              // wave tile, rows
  constexpr int WTN = BNW / WN;             // wave tile, weight rows
  constexpr int MB = WTM / 32, NB = WTN / 32;
  constexpr int STAGE_ELEMS = (BM + BNW) * BK;
  constexpr int NMFMA = MB * NB;            // MFMAs per 16-wide k step
  constexpr int NRD = MB + NB;              // fragment reads per k step
  constexpr int NWR = XCH + WCH;            // LDS chunk writes per K tile
  constexpr int RD_PER = (NRD + NMFMA - 1) / NMFMA;
  constexpr int WR_PER = (NWR + 2 * NMFMA - 1) / (2 * NMFMA);
  constexpr int LD_PER = (NWR + NMFMA - 1) / NMFMA;
  static_assert(RS % 16 == 0 && BM % RS == 0 && BNW % RS == 0, "tile/thread shape");
  static_assert(!GLU || NB % 2 == 0, "SwiGLU needs an even number of column blocks per wave");
  typedef typename Mfma32<T>::vec frag_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;

  TileCoord tc;
  if (!decode_tile<BM>(a.expert_offsets, a.E, a.n_tiles, a.remap, tc)) return;
  const int expert = tc.expert, row_begin = tc.row_begin, row_end = tc.row_end, nt = tc.nt;

  // ---- per-thread global sources ---------------------------------------------------------------
  const int c = tid % CPR;   // chunk within a tile row
  const int r0 = tid / CPR;  // first tile row of this thread
  constexpr int WROWS_MUL = GLU ? 2 : 1;
  const T* __restrict__ xbase = static_cast<const T*>(a.in);
  const T* __restrict__ wbase = static_cast<const T*>(a.w) + (W8 ? 0 : (size_t)expert * WROWS_MUL * a.N * a.K);
  // W8: byte address of the expert's weights; woff[j] is a byte offset (row-major: of the row's chunk c; tiled: of
  // the row inside stage 0 of its unit) and wfx[j] the row's slot swizzle in the tiled layout
  const uint8_t* __restrict__ wbase8 = nullptr;
  if constexpr (W8) {
    const size_t expert_bytes =
        a.w_tiled ? (size_t)mi_ceil_div_dev(a.N, GLU ? 16 : 32) * (size_t)(a.K >> 7) * 4096 : (size_t)WROWS_MUL * a.N * a.K;
    wbase8 = static_cast<const uint8_t*>(a.w) + (size_t)expert * expert_bytes;
  }
  int wfx[WCH];

  uint32_t xoff[XCH], woff[WCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int srow = row_begin + r0 + j * RS;
    if (srow > row_end - 1) srow = row_end - 1;  // tail rows re-read the last valid row; never stored
    int src = a.gather ? a.sorted_scattered[srow] / a.kdiv : srow;
    xoff[j] = (uint32_t)src * (uint32_t)a.K + c * CE;
  }
#pragma unroll
  for (int j = 0; j < WCH; ++j) {
    int r = r0 + j * RS;
    int col, half = 0;
    if (GLU) {
      half = r >= BN;
      col = nt * BN + (half ? r - BN : r);
    } else {
      col = nt * BN + r;
    }
    if (col > a.N - 1) col = a.N - 1;  // column tail re-reads the last weight row; never stored
    woff[j] = (uint32_t)(half * a.N + col) * (uint32_t)a.K + c * CE;
    wfx[j] = 0;
    if constexpr (W8) {
      if (a.w_tiled) {
        // unit u = 16 up + 16 gate channels (GLU) or 32 channels; row t of the unit's 32-row stage image
        const int u = GLU ? col >> 4 : col >> 5;
        const int t = GLU ? (col & 15) + 16 * half : (col & 31);
        woff[j] = (uint32_t)u * (uint32_t)(a.K >> 7) * 4096u + (uint32_t)t * 128u;
        wfx[j] = ((t >> 1) & 1) | (((t >> 2) & 1) << 2);
      }
    }
  }

  // LDS tile layout: row r holds its eight 16-byte chunks at slots  chunk ^ swz(r),
  // swz(r) = (r & 7) ^ ((r >> 3) & 1): any 8 consecutive rows AND any 16 consecutive rows of one
  // logical chunk fall into distinct bank groups (row parity selects the upper / lower 32 banks).
  // RS % 16 == 0, so all chunks of a thread share one swizzle.
  const int sw_c = c ^ ((r0 & 7) ^ ((r0 >> 3) & 1));
  const int st_x = (r0 * CPR + sw_c) * CE;              // element offset inside the X tile
  const int st_w = BM * BK + (r0 * CPR + sw_c) * CE;    // ... inside the W tile (after the X tile)

  u32x4 xreg[XCH], wreg[WCH];
  u32x2 wraw[W8 ? WCH : 1];  // W8: the chunk's 8 bytes as loaded (widened when they go to LDS)
  const int nk = (a.K + BK - 1) / BK;
  // W8: byte offset of this thread's 8-byte chunk of the K tile that starts at k0 (tiled: K % 128 == 0, so every
  // chunk exists and kc = k0 + 8 c < K)
  auto w8_at = [&](int j, int k0) -> uint32_t {
    if (!a.w_tiled) return woff[j] + (uint32_t)k0;
    const int kc = k0 + c * CE;
    return woff[j] + (uint32_t)(kc >> 7) * 4096u + (uint32_t)((((kc & 127) >> 4) ^ wfx[j]) << 4) + (uint32_t)(kc & 8);
  };

  auto load_global = [&](int kt) {
    int k0 = kt * BK;
    if (KTAIL) {
      // the last K tile may be partial: out-of-range chunks re-read chunk 0 of the row and are zeroed
      const bool kvalid = (k0 + c * CE) < a.K;
      const int koff = kvalid ? k0 : -(c * CE);
#pragma unroll
      for (int j = 0; j < XCH; ++j) {
        u32x4 v = *reinterpret_cast<const u32x4*>(xbase + xoff[j] + koff);
        xreg[j] = kvalid ? v : (u32x4){0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int j = 0; j < WCH; ++j) {
        if constexpr (W8) {
          // (a partial K tile only exists with row-major weights: the tiled layout has whole 128-wide stages)
          const u32x2 v = *reinterpret_cast<const u32x2*>(wbase8 + woff[j] + koff);
          wraw[j] = kvalid ? v : (u32x2){0u, 0u};
        } else {
          u32x4 v = *reinterpret_cast<const u32x4*>(wbase + woff[j] + koff);
          wreg[j] = kvalid ? v : (u32x4){0u, 0u, 0u, 0u};
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < XCH; ++j) xreg[j] = *reinterpret_cast<const u32x4*>(xbase + xoff[j] + k0);
#pragma unroll
      for (int j = 0; j < WCH; ++j) {
        if constexpr (W8) wraw[j] = *reinterpret_cast<const u32x2*>(wbase8 + w8_at(j, k0));
        else wreg[j] = *reinterpret_cast<const u32x4*>(wbase + woff[j] + k0);
      }
    }
  };
  // chunk writes [first, first + count) of this thread's NWR chunks (X chunks first, then W chunks)
  auto store_lds = [&](int stage, int first, int count) {
    T* s = smem + stage * STAGE_ELEMS;
#pragma unroll
    for (int j = 0; j < NWR; ++j) {
      if (j < first || j >= first + count) continue;
      if (j < XCH)
        *reinterpret_cast<u32x4*>(s + st_x + j * RS * BK) = xreg[j];
      else if constexpr (W8)
        *reinterpret_cast<u32x4*>(s + st_w + (j - XCH) * RS * BK) = Widen8<T>::run(wraw[j - XCH][0], wraw[j - XCH][1]);
      else
        *reinterpret_cast<u32x4*>(s + st_w + (j - XCH) * RS * BK) = wreg[j - XCH];
    }
  };

  // ---- fragment reads ---------------------------------------------------------------------------
  // lane l reads tile row (block_row0 + l%32), logical chunk 2*kk + l/32
  const int frow = lane & 31, fhalf = lane >> 5;
  const int fswz = (frow & 7) ^ ((frow >> 3) & 1);  // block_row0 is a multiple of 32
  int frag_x_off[MB], frag_w_off[NB];                // element offsets of the row inside a stage
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) frag_x_off[mb] = (wm * WTM + mb * 32 + frow) * BK;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    int r;
    if (GLU) {
      constexpr int HB = NB / 2;  // blocks per half
      int h = nb >= HB;
      r = h * BN + wn * (WTN / 2) + (h ? nb - HB : nb) * 32 + frow;
    } else {
      r = wn * WTN + nb * 32 + frow;
    }
    frag_w_off[nb] = BM * BK + r * BK;
  }
  int chunk_off[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) chunk_off[kk] = ((kk * 2 + fhalf) ^ fswz) * CE;

  frag_t xf[2][MB], wf[2][NB];
  auto read_frags = [&](int stage, int kk, int buf) {
    const T* s = smem + stage * STAGE_ELEMS + chunk_off[kk];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[buf][nb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_w_off[nb]));
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      xf[buf][mb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_x_off[mb]));
  };

  f32x16 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][mb][i] = 0.f;

  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = Mfma32<T>::run(wf[buf][nb], xf[buf][mb], acc[nb][mb]);
  };

  // ---- software pipeline ------------------------------------------------------------------------
  // Per K tile (4 k-steps of two chunks each), with LDS stages cur / nxt and fragment buffers 0 / 1:
  //   step 0: MFMA(buf0) | read frags(step1, cur) -> buf1
  //   step 1: MFMA(buf1) | read frags(step2, cur) -> buf0 | write first half of tile kt+1 -> nxt
  //   step 2: MFMA(buf0) | read frags(step3, cur) -> buf1 | write second half            -> nxt
  //   barrier            (nxt complete; everybody has fetched its last fragments of cur)
  //   step 3: MFMA(buf1) | read frags(step0, nxt) -> buf0 | global loads of tile kt+2 -> registers
  // The sched_group_barrier sequences ask the backend to issue the LDS / global instructions in the
  // shadow of the MFMAs (one wave per SIMD: nothing else hides their issue slots).
  load_global(0);
  store_lds(0, 0, NWR);
  __syncthreads();
  load_global(nk > 1 ? 1 : 0);
  read_frags(0, 0, 0);

  // The last round stages a surplus tile (a re-read of the last one) that nobody consumes; keeping the
  // loop body uniform keeps the accumulators in place (no peeled copy of the 256 accumulator registers).
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    read_frags(cur, 1, 1);
    mfma_step(0);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    read_frags(cur, 2, 0);
    store_lds(nxt, 0, NWR / 2);
    mfma_step(1);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_WR, WR_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    read_frags(cur, 3, 1);
    store_lds(nxt, NWR / 2, NWR - NWR / 2);
    mfma_step(0);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_WR, WR_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    read_frags(nxt, 0, 0);
    load_global(kt + 2 < nk ? kt + 2 : nk - 1);  // the surplus load of the last round is never used
    mfma_step(1);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
      __builtin_amdgcn_sched_group_barrier(SG_VMEM_RD, LD_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // ---- epilogue ---------------------------------------------------------------------------------
  // acc[nb][mb][i]: weight row (output column) = 8*(i/4) + 4*(lane/32) + i%4 of block nb,
  //                 activation row             = lane%32 of block mb
  T* __restrict__ out = static_cast<T*>(a.out);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = row_begin + wm * WTM + mb * 32 + frow;
    if (row >= row_end) continue;
    const int orow = a.scatter ? a.sorted_scattered[row] : row;
    T* orow_ptr = out + (size_t)orow * a.N;
    constexpr int OB = GLU ? NB / 2 : NB;
#pragma unroll
    for (int nb = 0; nb < OB; ++nb) {
      const int col0 = nt * BN + (GLU ? wn * (WTN / 2) : wn * WTN) + nb * 32 + fhalf * 4;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = col0 + g * 8;
        if (col >= a.N) continue;
        float v[4];
        f32x4 su = {1.f, 1.f, 1.f, 1.f}, sg = {1.f, 1.f, 1.f, 1.f};
        if constexpr (W8) {  // (N % 4 == 0 and col % 4 == 0: the four columns exist together)
          const float* sc = a.wscale + (size_t)expert * WROWS_MUL * a.N + col;
          su = *reinterpret_cast<const f32x4*>(sc);
          if (GLU) sg = *reinterpret_cast<const f32x4*>(sc + a.N);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (GLU) {
            float up = acc[nb][mb][g * 4 + i];
            float gt = acc[nb + NB / 2][mb][g * 4 + i];
            if constexpr (W8) {
              up *= su[i];
              gt *= sg[i];
            }
            v[i] = up * silu_f32(gt);
          } else {
            v[i] = acc[nb][mb][g * 4 + i];
            if constexpr (W8) v[i] *= su[i];
          }
        }
        if constexpr (sizeof(T) == 4) {
          *reinterpret_cast<f32x4*>(orow_ptr + col) = (f32x4){v[0], v[1], v[2], v[3]};
        } else {
          u32x2 p = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
          *reinterpret_cast<u32x2*>(orow_ptr + col) = p;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Main kernel: global -> LDS by DMA (global_load_lds_dwordx4), 4 LDS stages of 32 k each.
//
// The register-staged kernel above keeps only one K tile in flight; under load the L2 -> CU latency
// exceeds one tile's worth of MFMA time and the matrix cores idle.  Here the tiles never pass through
// VGPRs: every wave issues 16-byte-per-lane DMA loads whose destination is a contiguous 1 KiB run of
// LDS (lane i -> base + 16*i).  Three tiles are in flight while a fourth is consumed.
//
//   stage layout   (BM + BNW) rows x 32 k, 64 bytes per row = 4 slots of 16 bytes;
//                  slot of logical chunk c in row r:  c ^ ((r >> 2) & 3)   (ds_read_b128 conflict-free)
//   DMA mapping    one wave instruction fills 16 rows: lane l -> row l/4, slot l%4, so the lane fetches
//                  logical chunk (l%4) ^ ((row >> 2) & 3) of its row: the swizzle is applied on the
//                  global side, 4 lanes still cover one contiguous 64-byte piece of a row
//   iteration kt   (stage cur = kt % 4, fragment buffers 0/1, two k-steps of 16)
//       A: MFMA(step 0, buf0)      | ds_read step 1 of cur -> buf1
//       s_waitcnt vmcnt(2 tiles)   : my share of tile kt+1 has landed;  lgkmcnt(0): my reads of cur are done
//       s_barrier                  : tile kt+1 complete, stage cur free
//       B: MFMA(step 1, buf1)      | ds_read step 0 of tile kt+1 -> buf0 | DMA tile kt+4 -> stage cur
// The waits are explicit (s_waitcnt immediates); a fence-carrying __syncthreads would drain all DMA.
// ------------------------------------------------------------------------------------------------

__device__ __forceinline__ constexpr int waitcnt_imm(int vm, int lgkm) {
  // gfx9 encoding: vmcnt = {imm[15:14], imm[3:0]}, expcnt = imm[6:4] (7 = no wait), lgkmcnt = imm[11:8]
  return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}

// One DMA instruction: every lane moves 16 bytes from (scalar base + its 32-bit byte offset) to LDS; the
// 64 destinations are the contiguous run starting at the LDS byte address in M0.  Written as inline
// assembly on purpose: for the builtin the compiler assumes that any later LDS read may alias the DMA write
// and puts "s_waitcnt vmcnt(0)" in front of it, which drains the prefetch ring every K slice.  Here the
// ordering is done by hand (s_waitcnt immediates before the barrier that publishes a stage).
// The offset register is read when the instruction issues, but the compiler treats a register named by an
// assembly statement as busy until vmcnt reaches 0 and waits before overwriting it: callers pass offsets
// that live in registers of their own for a whole tile, never a per-slice temporary.  TAG keeps otherwise
// identical statements in the two arms of a branch from being merged back into one with a selected
// (temporary) operand.
template <int TAG>
__device__ __forceinline__ void dma16_to_lds(const void* base, uint32_t byte_off, uint32_t lds_addr) {
  if (TAG == 0)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(byte_off), "s"(base)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 ; next tile" : : "s"(lds_addr), "v"(byte_off), "s"(base)
                 : "memory", "m0");
}

template <typename T, int BM, int BNW, int WM, int WN, bool GLU>
__global__ __launch_bounds__(WM* WN * 64) void grouped_gemm_dma_kernel(GemmArgs a) {
  constexpr int BK = 32;
  constexpr int NSTAGE = 4;
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr int ROWS = BM + BNW;
  constexpr int STAGE_BYTES = ROWS * BK * 2;
  constexpr int NLD = ROWS / 16 / NW;       // DMA instructions per wave per tile
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr int WTM = BM / WM, WTN = BNW / WN;
  constexpr int MB = WTM / 32, NB = WTN / 32;
  constexpr int NMFMA = MB * NB;
  constexpr int NRD = MB + NB;
  constexpr int RD_PER = (NRD + NMFMA - 1) / NMFMA;
  constexpr int LD_PER = (NLD + NMFMA - 1) / NMFMA;
  static_assert(ROWS % (16 * NW) == 0 && BM % 16 == 0, "tile/wave shape");
  static_assert(!GLU || NB % 2 == 0, "SwiGLU needs an even number of column blocks per wave");
  static_assert(3 * NLD <= 63, "vmcnt range");
  typedef typename Mfma32<T>::vec frag_t;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* glb_ptr_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;

  TileCoord tc;
  if (!decode_tile<BM>(a.expert_offsets, a.E, a.n_tiles, a.remap, tc)) return;
  const int expert = tc.expert, row_begin = tc.row_begin, row_end = tc.row_end, nt = tc.nt;

  // ---- DMA sources: instruction j of this wave fills stage rows [(j*NW + wave)*16, +16) -----------
  constexpr int WROWS_MUL = GLU ? 2 : 1;
  const T* __restrict__ xbase = static_cast<const T*>(a.in);
  const T* __restrict__ wbase = static_cast<const T*>(a.w) + (size_t)expert * WROWS_MUL * a.N * a.K;
  const int lchunk = (lane & 3) ^ ((lane >> 4) & 3);  // (row >> 2) & 3 == (lane >> 4) & 3: groups are 16-row aligned
  const T* src[NLD];
#pragma unroll
  for (int j = 0; j < NLD; ++j) {
    const int r = (j * NW + wave) * 16 + (lane >> 2);  // stage row
    if (r < BM) {
      int srow = row_begin + r;
      if (srow > row_end - 1) srow = row_end - 1;  // tail rows re-read the last valid row; never stored
      const int s = a.gather ? a.sorted_scattered[srow] / a.kdiv : srow;
      src[j] = xbase + (size_t)s * a.K + lchunk * 8;
    } else {
      const int wr = r - BM;
      int col, half = 0;
      if (GLU) {
        half = wr >= BN;
        col = nt * BN + (half ? wr - BN : wr);
      } else {
        col = nt * BN + wr;
      }
      if (col > a.N - 1) col = a.N - 1;  // column tail re-reads the last weight row; never stored
      src[j] = wbase + ((size_t)half * a.N + col) * a.K + lchunk * 8;
    }
  }
  const int nk = a.K / BK;
  auto dma_tile = [&](int kt, int stage) {
    const int k0 = (kt < nk ? kt : nk - 1) * BK;  // surplus rounds re-fetch the last tile; never consumed
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
      unsigned char* dst = smem_raw + stage * STAGE_BYTES + (j * NW + wave) * 1024;
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(src[j] + k0), (lds_ptr_t)dst, 16, 0, 0);
    }
  };

  // ---- fragment reads --------------------------------------------------------------------------------
  const int frow = lane & 31, fhalf = lane >> 5;
  const int fswz = (frow >> 2) & 3;  // block rows start at multiples of 32
  int frag_x_off[MB], frag_w_off[NB];  // byte offset of the fragment row inside a stage
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) frag_x_off[mb] = (wm * WTM + mb * 32 + frow) * (BK * 2);
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    int r;
    if (GLU) {
      constexpr int HB = NB / 2;
      int h = nb >= HB;
      r = h * BN + wn * (WTN / 2) + (h ? nb - HB : nb) * 32 + frow;
    } else {
      r = wn * WTN + nb * 32 + frow;
    }
    frag_w_off[nb] = (BM + r) * (BK * 2);
  }
  const int chunk_byte[2] = {((0 + fhalf) ^ fswz) * 16, ((2 + fhalf) ^ fswz) * 16};

  frag_t xf[2][MB], wf[2][NB];
  auto read_frags = [&](int stage, int kk, int buf) {
    const unsigned char* s = smem_raw + stage * STAGE_BYTES + chunk_byte[kk];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[buf][nb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_w_off[nb]));
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      xf[buf][mb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_x_off[mb]));
  };

  f32x16 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][mb][i] = 0.f;

  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = Mfma32<T>::run(wf[buf][nb], xf[buf][mb], acc[nb][mb]);
  };

  // ---- pipeline ----------------------------------------------------------------------------------------
  dma_tile(0, 0);
  dma_tile(1, 1);
  dma_tile(2, 2);
  dma_tile(3, 3);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(3 * NLD, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_frags(0, 0, 0);

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & (NSTAGE - 1), nxt = (kt + 1) & (NSTAGE - 1);
    read_frags(cur, 1, 1);
    mfma_step(0);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * NLD, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    read_frags(nxt, 0, 0);
    dma_tile(kt + 4, cur);
    mfma_step(1);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      __builtin_amdgcn_sched_group_barrier(SG_DS_RD, RD_PER, 0);
      __builtin_amdgcn_sched_group_barrier(SG_VMEM_RD, LD_PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));  // surplus DMA must not outlive the workgroup's LDS

  // ---- epilogue ---------------------------------------------------------------------------------
  T* __restrict__ out = static_cast<T*>(a.out);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = row_begin + wm * WTM + mb * 32 + frow;
    if (row >= row_end) continue;
    const int orow = a.scatter ? a.sorted_scattered[row] : row;
    T* orow_ptr = out + (size_t)orow * a.N;
    constexpr int OB = GLU ? NB / 2 : NB;
#pragma unroll
    for (int nb = 0; nb < OB; ++nb) {
      const int col0 = nt * BN + (GLU ? wn * (WTN / 2) : wn * WTN) + nb * 32 + fhalf * 4;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = col0 + g * 8;
        if (col >= a.N) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (GLU) {
            float up = acc[nb][mb][g * 4 + i];
            float gt = acc[nb + NB / 2][mb][g * 4 + i];
            v[i] = up * silu_f32(gt);
          } else {
            v[i] = acc[nb][mb][g * 4 + i];
          }
        }
        u32x2 p = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
        *reinterpret_cast<u32x2*>(orow_ptr + col) = p;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Persistent variant of the DMA kernel: one workgroup per CU walks a list of tiles and the 4-stage
// LDS ring runs straight through the tile boundaries.
//
// A workgroup that handles one tile pays, per tile, for a launch, the tile lookup, the row-index
// loads, an empty pipeline (three stages of DMA latency) and an epilogue during which nothing is in
// flight; with K = 1536 that is as long as the MFMA work itself.  Here
//   * the DMA for the first four K slices of tile i+1 is issued during the last four slices of tile i,
//   * the lookup of tile i+2 comes from a per-expert table in LDS (no global loads) and its row-index
//     loads are issued before the epilogue of tile i and consumed after it,
//   * the epilogue stages each 32 x 64 block of results through a per-wave LDS scratch so that global
//     stores are 16 bytes per lane and 128 contiguous bytes per row.
// Tile order: workgroup b serves XCD b % 8 (hardware deals workgroup ids round-robin to the XCDs); the
// XCD's contiguous tile range is dealt to its workgroups in turn, so at any moment the CUs of one XCD
// work on neighbouring tiles (same expert weights, shared activation rows) out of one L2.
//
// The eight waves form two groups that alternate between a memory phase and a matrix phase (see pp_slice).  With
// all waves in one phase and one barrier per K slice, the two waves of a SIMD stall together (barrier, LDS latency,
// DMA issue) and the matrix pipe idles: measured on the 32768-token Granite-3B shape, about 65 % matrix-pipe
// occupancy in cycles inside the K loop against about 80 % for the alternating form, with 32-wide as with 64-wide
// K slices.  (With random operands the chip then lowers its clock to stay inside its power limit, so wall time
// improves less than the cycle count.)
// ------------------------------------------------------------------------------------------------

#define PERSIST_MAX_E 256

// Splitting the last round along K.  A workgroup's tiles all take the same time, so when the tiles of an XCD do not
// fill its last round, the workgroups without a tile wait for one tile time.  With a workspace, the `rem` tiles of
// that round are cut into `parts` = min(slots / rem, PERSIST_SPLIT_MAX) ranges of K slices, one per workgroup; a
// part writes its fp32 accumulators to the workspace instead of running the epilogue, and a second, small launch
// (grouped_gemm_split_finish_kernel) adds the parts of every split tile in part order and runs the epilogue, so
// the result does not depend on timing.  A round is only split if that shortens it by at least
// PERSIST_SPLIT_MIN_SAVED slices: the partial tiles' trip through memory and the second launch cost 40-80 us
// (measured), about 100 slices' worth.
#define PERSIST_SPLIT_MAX 4
#define PERSIST_SPLIT_MIN_SAVED 120
#define PERSIST_SPLIT_MIN_SLICES 32
#define PERSIST_WS_TILE_BYTES (256 * 256 * 4)

// whether a contraction of length K can be shortened by PERSIST_SPLIT_MIN_SAVED slices at all (launch_persistent
// applies the same rule, plus one on the grid)
static bool persistent_may_split(int K) {
  const int nk = K / 32;
  return nk - nk / PERSIST_SPLIT_MAX >= PERSIST_SPLIT_MIN_SAVED;
}

// Which tiles a workgroup runs.  Workgroup b sits on XCD b % 8 (the hardware deals workgroup ids round-robin to the
// XCDs) in slot b / 8.  Two ways of dealing the band-ordered tile list to them:
//   * contiguous (the default): XCD x owns the x-th eighth of the list and deals it to its slots in turn, so the
//     CUs of an XCD work on neighbouring tiles out of one L2 and an XCD stays with its experts;
//   * interleaved (PERSIST_REMAP_INTERLEAVE): round r of the whole chip is the tiles [r * grid, (r + 1) * grid), XCD
//     x taking the x-th run of grid / 8 of them.  All XCDs then work on neighbouring tiles at the same time.  When
//     an expert has more column tiles than a band is wide (intermediate size 14336: 112 column tiles, bands of 8),
//     consecutive bands read the same activation rows, and the XCDs share them through the memory-side cache
//     instead of each fetching them from HBM in its own time: Mixtral-shape layer 5.02 -> 4.73 ms.  With few
//     column tiles (the band is the whole row) it changes little either way (-1.3 % on the Granite-1B shape,
//     +1.1 % on the Granite-3B shape), so the host asks for it only from 8 column tiles on.
// Either way the tiles that do not fill the last round can be cut along K (see PERSIST_SPLIT_MAX).
#define PERSIST_REMAP_INTERLEAVE 2
#define PERSIST_REMAP_FIXED 4  // the caller chose the form (cfg 8 / 9): the host does not apply its own rule

struct SplitPlan {
  int base, stride;  // tile of this workgroup in round i < full_rounds: base + i * stride
  int full_rounds;   // rounds in which every slot has a tile
  int rem;           // tiles of the last round, the first of them being rem_base
  int rem_base;
  int parts;         // K ranges each of them is cut into (1: not split)
  int lslot;         // this workgroup's slot in the last round: part lslot / rem of tile rem_base + lslot % rem
  int ws_base;       // first partial-tile slot of the last round's tiles in the workspace
};

// xcd / slot of the workgroup (slot < nslot); for the finishing kernel, slot is the tile of the last round it adds up
__device__ __forceinline__ SplitPlan persist_split_plan(int total, int xcd, int slot, int nslot, int nk, bool have_ws,
                                                        bool interleave) {
  SplitPlan sp;
  int cap;  // slots that share one last round
  if (interleave) {
    cap = nslot * 8;
    sp.lslot = xcd * nslot + slot;
    sp.base = sp.lslot;
    sp.stride = cap;
    sp.full_rounds = total / cap;
    sp.rem = total - sp.full_rounds * cap;
    sp.rem_base = sp.full_rounds * cap;
    sp.ws_base = 0;
  } else {
    cap = nslot;
    const int per = (total + 7) >> 3;
    int n_x = total - xcd * per;
    n_x = n_x < 0 ? 0 : (n_x < per ? n_x : per);
    sp.lslot = slot;
    sp.base = xcd * per + slot;
    sp.stride = nslot;
    sp.full_rounds = n_x / nslot;
    sp.rem = n_x - sp.full_rounds * nslot;
    sp.rem_base = xcd * per + sp.full_rounds * nslot;
    sp.ws_base = xcd * nslot;
  }
  sp.parts = 1;
  if (have_ws && sp.rem > 0) {
    int p = cap / sp.rem;
    if (p > PERSIST_SPLIT_MAX) p = PERSIST_SPLIT_MAX;
    if (p >= 2 && nk / p >= PERSIST_SPLIT_MIN_SLICES && nk - nk / p >= PERSIST_SPLIT_MIN_SAVED) sp.parts = p;
  }
  return sp;
}

// etab[2e] = row tiles of experts 0..e, etab[2e+1] = offsets[e]; filled by the calling wave (all 64 lanes)
template <int BM>
__device__ __forceinline__ void persist_expert_table(const int32_t* __restrict__ off, int E, int* etab) {
  const int lane = threadIdx.x & 63;
  int carry = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int end = e < E ? off[e] : 0;
    const int prev = (e < E && e > 0) ? off[e - 1] : 0;
    const int t = e < E ? (end - prev + BM - 1) / BM : 0;
    int incl = t;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    incl += carry;
    if (e < E) {
      etab[2 * e] = incl;
      etab[2 * e + 1] = end;
    }
    carry = __shfl(incl, 63, 64);
  }
}

// tile id -> coordinates, from the LDS table (wave-uniform result).  An expert's tiles are numbered band
// by band: a band is up to 8 column tiles wide and runs over all of the expert's row tiles, row tile
// slowest.  The 32 workgroups of an XCD, which take 32 consecutive tiles at a time, then cover about
// 4 row tiles x 8 column tiles: 12 operand slabs for 32 tiles, and each weight slab is fetched once per
// band instead of once per row tile (with many column tiles -- intermediate 14336 -- a plain row-major
// order re-streams all of an expert's weights from HBM for every row tile).  Up to 8 column tiles the band
// is the whole row, so that complete output rows are written at about the same time.
template <int BM>
__device__ __forceinline__ void persist_locate(const int* etab, int E, int n_tiles, int tile, TileCoord& tc) {
  const int lane = threadIdx.x & 63;
  const int tile_band = n_tiles < 8 ? n_tiles : 8;
  const int q = tile / n_tiles;  // experts own contiguous tile ranges: (row tiles before) * n_tiles
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int incl = e < E ? etab[2 * e] : 0x7fffffff;
    const uint64_t hit = __ballot(incl > q);
    if (hit) {
      const int ex = e0 + __ffsll((long long)hit) - 1;
      const int first_tile = ex > 0 ? etab[2 * (ex - 1)] : 0;
      const int prev = ex > 0 ? etab[2 * (ex - 1) + 1] : 0;
      const int row_tiles = etab[2 * ex] - first_tile;
      const int local = tile - first_tile * n_tiles;
      const int band = local / (row_tiles * tile_band);
      const int rem = local - band * row_tiles * tile_band;
      const int left = n_tiles - band * tile_band;
      const int width = left < tile_band ? left : tile_band;
      const int mt = rem / width;
      tc.expert = ex;
      tc.nt = band * tile_band + rem - mt * width;
      tc.row_begin = prev + mt * BM;
      tc.row_end = etab[2 * ex + 1];
      return;
    }
  }
  tc.expert = 0; tc.nt = 0; tc.row_begin = 0; tc.row_end = 1;  // unreachable for a valid tile id
}

template <typename T, int BM, int BNW, int WM, int WN, bool GLU, bool WT = false, bool KEEP_PRE = false>
__global__ __launch_bounds__(WM* WN * 64) void grouped_gemm_persistent_kernel(GemmArgs a) {
  // KEEP_PRE: the SwiGLU form that also writes the pre-activation (a.pre), for training
  static_assert(!KEEP_PRE || GLU, "the pre-activation belongs to the SwiGLU form");
  // WT: the expert weights are (K, N) row-major ("x @ W" with W as stored, the form both data gradients of the
  // backward take).  A K slice of them is 32 rows of 512 bytes; it is staged as it lies in HBM and the fragments
  // are read with the transposing LDS read (see read_frags).
  static_assert(!WT || (!GLU && BNW == 256), "transposed-weight form");
  constexpr int BK = 32;                     // K slice per ring stage = one 16x16x32 matrix instruction deep
  constexpr int NSTAGE = 4;                  // ring of 128 KiB
  constexpr int RPI = 16;                    // stage rows filled by one DMA instruction (1 KiB)
  constexpr int LROW_SHIFT = 2;              // lane -> row within the instruction's rows
  constexpr int NW = WM * WN;
  constexpr int ROWS = BM + BNW;
  constexpr int STAGE_BYTES = ROWS * BK * 2;
  constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
  // per-wave epilogue scratch: 32 rows x 64 columns, in the ring stage that is free at a tile boundary.  64 columns
  // make every store a run of whole 128-byte lines per row (measured: 64-byte pieces write at 4.4-4.6 TB/s
  // chip-wide, 128-byte ones at 5.0-5.3).
  constexpr int EPI_COLS = 64;
  constexpr int EPI_BYTES = 32 * EPI_COLS * 2;
  constexpr int EPI_CPR = EPI_COLS / 8;      // 16-byte chunks per scratch row
  constexpr int NLD = ROWS / RPI / NW;       // DMA instructions per wave per K slice
  constexpr int NXLD = BM / RPI / NW;        // ... of which activation rows (the first NXLD)
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr int WTM = BM / WM, WTN = BNW / WN;
  constexpr int MT = 16;                     // edge of one accumulator block (v_mfma_f32_16x16x32)
  constexpr int MB = WTM / MT, NB = WTN / MT;
  constexpr int OB = GLU ? NB / 2 : NB;      // output column blocks per wave
  constexpr int EPI_MB = 32 / MT;            // accumulator row blocks per 32-row epilogue pass
  constexpr int EPI_NB = EPI_COLS / MT;      // accumulator column blocks per epilogue pass
  static_assert(BM % (16 * NW) == 0 && BNW % (16 * NW) == 0 && NW % 2 == 0, "tile/wave shape");
  static_assert(OB % EPI_NB == 0 && MB % EPI_MB == 0, "epilogue pass shape");
  static_assert((NSTAGE - 1) * NLD <= 63, "vmcnt range");
  typedef typename Mfma16<T>::vec frag_t;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  // [ring][expert table: E x (tiles inclusive, row end)]
  int* etab = reinterpret_cast<int*>(smem_raw + RING_BYTES);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;

  // ---- per-expert table: etab[2e] = row tiles of experts 0..e, etab[2e+1] = offsets[e] ---------------
  if (wave == 0) persist_expert_table<BM>(a.expert_offsets, a.E, etab);
  __syncthreads();
  const int total = etab[2 * (a.E - 1)] * a.n_tiles;
  const int xcd = blockIdx.x & 7, slot0 = blockIdx.x >> 3, nslot = gridDim.x >> 3;
  const int nk = a.K / BK;  // >= NSTAGE (host-checked)
  // full_rounds rounds in which every slot has a tile, then `rem` tiles, each cut into `parts` K ranges
  const SplitPlan sp =
      persist_split_plan(total, xcd, slot0, nslot, nk, a.ws != nullptr, (a.remap & PERSIST_REMAP_INTERLEAVE) != 0);
  const int my_part = sp.parts > 1 ? sp.lslot / sp.rem : 0, my_rem_tile = sp.rem > 0 ? sp.lslot % sp.rem : 0;

  // i-th tile of this workgroup, or -1
  auto tile_of = [&](int i) -> int {
    if (i < sp.full_rounds) return sp.base + i * sp.stride;
    if (i > sp.full_rounds || sp.lslot >= sp.rem * sp.parts) return -1;
    return sp.rem_base + my_rem_tile;
  };
  // K slices [k0, k0 + len) of the i-th item
  auto item_k = [&](int i, int& k0, int& len) {
    if (i == sp.full_rounds && sp.parts > 1) {
      k0 = my_part * nk / sp.parts;
      len = (my_part + 1) * nk / sp.parts - k0;
    } else {
      k0 = 0;
      len = nk;
    }
  };
  auto locate = [&](int tile, TileCoord& tc) { persist_locate<BM>(etab, a.E, a.n_tiles, tile, tc); };

  // ---- DMA sources -----------------------------------------------------------------------------------
  // A tile's sources are NLD 32-bit byte offsets per lane (activation rows relative to the input
  // matrix, weight rows relative to the expert's weight matrix) plus the expert's scalar base; the K
  // position is added on the scalar side, so a DMA instruction is "scalar base + lane offset".
  constexpr int WROWS_MUL = GLU ? 2 : 1;
  const unsigned char* __restrict__ xbase = static_cast<const unsigned char*>(a.in);
  const unsigned char* __restrict__ wall = static_cast<const unsigned char*>(a.w);
  const size_t expert_bytes = (size_t)WROWS_MUL * a.N * a.K * sizeof(T);
  // logical 16-byte chunk this lane fetches so that it lands in its swizzled slot (see read_frags): row =
  // 16*grp + lane/4, slot = lane%4, swizzle (row >> 1) & 3 -- the one that reads the 16 rows x 4 chunks of a
  // fragment without bank conflicts (measured; (row >> 2) & 3 costs about 20 % of the LDS read rate there)
  const int lchunk = (lane & 3) ^ ((lane >> 3) & 3);
  struct TileSrc {
    uint32_t off[NLD];
    const unsigned char* wbase;
  };
  // sorted-order row of the activation rows this lane fetches (clamped into the tile's expert)
  auto load_rows = [&](const TileCoord& tc, int (&raw)[NXLD]) {
#pragma unroll
    for (int j = 0; j < NXLD; ++j) {
      int srow = tc.row_begin + (j * NW + wave) * RPI + (lane >> LROW_SHIFT);
      if (srow > tc.row_end - 1) srow = tc.row_end - 1;  // tail rows re-read the last valid row; never stored
      raw[j] = a.gather ? a.sorted_scattered[srow] : srow;
    }
  };
  auto make_src = [&](const TileCoord& tc, const int (&raw)[NXLD], TileSrc& ts) {
    ts.wbase = wall + (size_t)tc.expert * expert_bytes;
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
      if (j < NXLD) {
        // (top-k is a power of two in every configuration of the reference: a shift instead of a division per lane
        // and tile; launch_persistent sets kshift to -1 otherwise)
        const int s = !a.gather ? raw[j] : (a.kshift >= 0 ? raw[j] >> a.kshift : raw[j] / a.kdiv);
        ts.off[j] = ((uint32_t)s * (uint32_t)a.K + lchunk * 8) * (uint32_t)sizeof(T);
      } else if constexpr (WT) {
        // DMA instruction = two K rows of the slice; LDS piece lane % 32 of row krow holds the logical 16-byte
        // piece whose 32-byte group is (piece / 2) ^ f(krow): the swizzle the transposing reads expect
        const int krow = 2 * ((j - NXLD) * NW + wave) + (lane >> 5);
        const int f = (krow & 3) | (((krow >> 3) & 3) << 2);
        const int piece = lane & 31;
        int col = tc.nt * BN + ((((piece >> 1) ^ f) & 15) << 4) + (piece & 1) * 8;
        if (col > a.N - 8) col = a.N - 8;  // column tail re-reads the last piece of the row; never stored
        ts.off[j] = ((uint32_t)krow * (uint32_t)a.N + col) * (uint32_t)sizeof(T);
      } else {
        const int wr = ((j - NXLD) * NW + wave) * RPI + (lane >> LROW_SHIFT);
        int col, half = 0;
        if (GLU) {
          half = wr >= BN;
          col = tc.nt * BN + (half ? wr - BN : wr);
        } else {
          col = tc.nt * BN + wr;
        }
        if (col > a.N - 1) col = a.N - 1;  // column tail re-reads the last weight row; never stored
        ts.off[j] = ((uint32_t)(half * a.N + col) * (uint32_t)a.K + lchunk * 8) * (uint32_t)sizeof(T);
      }
    }
  };
  // slice kt of tile `cur`, or (from_next) of tile `next`, into ring stage `stage`
  auto dma_slice = [&](const TileSrc& cur, const TileSrc& next, bool from_next, int kt, int stage) {
    const size_t kbytes = (size_t)kt * BK * sizeof(T);
    const unsigned char* xs = xbase + kbytes;
    const unsigned char* ws = (from_next ? next.wbase : cur.wbase) + (WT ? kbytes * a.N : kbytes);
    const uint32_t stage_lds = (uint32_t)(size_t)(lds_ptr_t)smem_raw + stage * STAGE_BYTES;
    // activation rows fill stage rows [0, BM), weight rows [BM, BM + BNW)
    auto grp = [&](int j) { return j < NXLD ? (j * NW + wave) : (BM / RPI + (j - NXLD) * NW + wave); };
    if (from_next) {
#pragma unroll
      for (int j = 0; j < NLD; ++j) dma16_to_lds<1>(j < NXLD ? xs : ws, next.off[j], stage_lds + grp(j) * 1024);
    } else {
#pragma unroll
      for (int j = 0; j < NLD; ++j) dma16_to_lds<0>(j < NXLD ? xs : ws, cur.off[j], stage_lds + grp(j) * 1024);
    }
  };

  // ---- fragment reads ----------------------------------------------------------------------------------
  // lane -> (row of its 16-row block, k chunk): the instruction takes k = 8 * (lane / 16) + [0, 8) of the slice
  const int frow = lane % MT, fhalf = lane / MT;
  const int fswz = (frow >> 1) & 3;
  int frag_x_off[MB], frag_w_off[NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) frag_x_off[mb] = (wm * WTM + mb * MT + frow) * (BK * 2);
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    int r;
    if (GLU) {
      constexpr int HB = NB / 2;
      int h = nb >= HB;
      r = h * BN + wn * (WTN / 2) + (h ? nb - HB : nb) * MT + frow;
    } else {
      r = wn * WTN + nb * MT + frow;
    }
    frag_w_off[nb] = (BM + r) * (BK * 2);
  }
  const int chunk_byte = (fhalf ^ fswz) * 16;
  frag_t xf[MB], wf[NB];
  // WT: ds_read_b64_tr_b16 transposes 4 rows x 16 columns across 16 lanes: lane i of the group supplies the
  // address of (row i / 4, columns 4 (i % 4) ..) and receives column i of the four rows.  Lane group q reads rows
  // 8q .. 8q + 3 and, 2 KiB further, 8q + 4 .. 8q + 7: together the 8 contraction values the matrix instruction
  // wants from lane (column, q).
  typedef short tr_s16x4 __attribute__((ext_vector_type(4)));
  const int tr_i = lane & 15, tr_q = lane >> 4;
  const uint32_t tr_base = (8 * tr_q + (tr_i >> 2)) * (BNW * 2) + ((((tr_i >> 2) | (tr_q << 2))) << 5) + (tr_i & 3) * 8;
  const uint32_t lds_base = (uint32_t)(size_t)(lds_ptr_t)smem_raw;
  auto read_frags = [&](int stage) {
    const unsigned char* s = smem_raw + stage * STAGE_BYTES + chunk_byte;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if constexpr (WT) {
        typedef __attribute__((address_space(3))) tr_s16x4* tr_ptr_t;
        const uint32_t addr = lds_base + stage * STAGE_BYTES + BM * BK * 2 + (tr_base ^ ((uint32_t)(wn * NB + nb) << 5));
        const tr_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(size_t)addr);
        const tr_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(size_t)(addr + 4 * BNW * 2));
        wf[nb] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      } else {
        wf[nb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_w_off[nb]));
      }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      xf[mb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(s + frag_x_off[mb]));
  };

  // accumulator block (nb, mb): register i of a lane is output column 16 * nb + 4 * fhalf + i (weight row) of
  // token row 16 * mb + frow
  f32x4 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[nb][mb][i] = 0.f;

  // eight instructions in a row share the activation operand.  The first slice of a tile multiplies onto a zero
  // operand instead of the accumulators (an inline constant of the instruction), so that the accumulators need not
  // be cleared between tiles: 128 moves per wave and tile, issued when the matrix pipe has nothing else to do.
  auto mfma_step = [&](auto first_tag) {
    constexpr bool FIRST = decltype(first_tag)::value;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb][mb] = Mfma16<T>::run(wf[nb], xf[mb], FIRST ? zero : acc[nb][mb]);
  };

  int g = 0;  // running K-slice count; slice g lives in ring stage g % NSTAGE
  // One K slice.  The waves with wn == 0 and those with
  // wn == 1 -- one of each per SIMD -- run this same code one phase apart (see the tile loop): while one group
  // issues its NB * MB matrix instructions back to back out of registers, the other reads its fragments of the
  // slice from LDS and issues its share of the DMA for slice g + 3 into the stage both groups have finished
  // reading.  Every phase ends in a workgroup barrier; at each barrier one group has just issued its last MFMA
  // and the other has its operands in registers, so the matrix pipe of the SIMD never waits for LDS, DMA or the
  // barrier itself.
  auto pp_slice = [&](auto first_tag, const TileSrc& tcur, const TileSrc& tnext, bool from_next, int kload) {
    const int cur = g & (NSTAGE - 1), fill = (g + NSTAGE - 1) & (NSTAGE - 1);
    read_frags(cur);
    dma_slice(tcur, tnext, from_next, kload, fill);
    asm volatile("" ::: "memory");
    // own DMA of slice g + 1 has landed (slices g + 2 and g + 3 stay in flight); fragments are in registers
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((NSTAGE - 2) * NLD, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // (Signalling the second barrier a few matrix instructions early, so that they cover its release
    // latency, measured slower: the group's next memory phase then starts late and becomes the long one.)
    mfma_step(first_tag);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    ++g;
  };

  // ---- epilogue of one tile: acc -> (SwiGLU) -> LDS scratch -> 16-byte row-contiguous stores -----------
  T* __restrict__ out = static_cast<T*>(a.out);
  static_assert(NW * EPI_BYTES <= STAGE_BYTES, "epilogue scratch must fit the free ring stage");
  constexpr int RPP = 64 / EPI_CPR;  // rows per read-back pass
  static_assert(RPP == 8, "read-back row order below");
  // Row of the 32-row block that read-back instruction `it` takes for this lane: instruction 0 the even rows of
  // the first sixteen, instruction 1 the odd ones, then the second sixteen.  All rows of an instruction have the
  // same parity, which is what lets the epilogue's writes use both 8-byte halves of a 16-byte chunk (see there).
  auto rb_row = [&](int it) { return 16 * (it >> 1) + 2 * (lane / EPI_CPR) + (it & 1); };
  constexpr int MP = MB / EPI_MB;    // 32-row passes over the wave's token rows
  // Destination rows of everything this lane will store in a tile's epilogue.  With scattered output they are
  // fetched one tile ahead (next to the gather indices of the tile after), so that the epilogue does not start
  // with a memory latency.
  struct OutRows {
    int r[MP][32 / RPP];
  };
  auto load_out_rows = [&](const TileCoord& tc, OutRows& o) {
    // (rows past the expert's end are never stored: with scattered output they read the index of its last row, so
    // that the loads need no predicates)
    const int row0 = tc.row_begin + wm * WTM;
    if (a.scatter) {
#pragma unroll
      for (int mp = 0; mp < MP; ++mp)
#pragma unroll
        for (int it = 0; it < 32 / RPP; ++it) {
          const int row = row0 + mp * 32 + rb_row(it);
          o.r[mp][it] = a.sorted_scattered[row < tc.row_end ? row : tc.row_end - 1];
        }
    } else {
#pragma unroll
      for (int mp = 0; mp < MP; ++mp)
#pragma unroll
        for (int it = 0; it < 32 / RPP; ++it) o.r[mp][it] = row0 + mp * 32 + rb_row(it);
    }
  };
  // INTERIOR: every row and column of the tile exists (all tiles but an expert's last row tile and a ragged last
  // column tile), so the stores need no predicates; NT: non-temporal stores (see persistent_out_nt).  Both are
  // compile-time forms of one body: the tile boundary is bound by instruction issue (no matrix work covers it),
  // and a predicate, an exec-mask save / restore and a branch on the store's cache policy around each of a wave's
  // 16 stores were a sixth of its instructions.
  // WHAT: 0 the kernel's result (with SwiGLU: up * silu(gate)); 1 / 2 (SwiGLU kernel keeping the pre-activation):
  // the up / the gate half of h, into a.pre.  KEEP: the result is formed from the ROUNDED halves, as the separate
  // activation kernel forms it from the stored h (swiglu_forward_kernel).
  auto epilogue_as = [&](auto what_tag, auto interior_tag, auto nt_tag, auto keep_tag, const TileCoord& tc,
                         const OutRows& orows) {
    constexpr int WHAT = decltype(what_tag)::value;
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    constexpr bool NT = decltype(nt_tag)::value;
    constexpr bool KEEP = decltype(keep_tag)::value;
    constexpr int OBX = WHAT == 0 ? OB : NB / 2;  // output column blocks of this form
    static_assert(OBX % EPI_NB == 0, "epilogue pass shape");
    T* __restrict__ dst_base = WHAT == 0 ? out : static_cast<T*>(a.pre);
    const int ld = WHAT == 0 ? a.N : 2 * a.N;
    // the ring stage consumed last is free until the next tile's first memory phase refills it (the tile loop
    // puts a barrier between this epilogue and that refill)
    unsigned char* scratch = smem_raw + ((g + NSTAGE - 1) & (NSTAGE - 1)) * STAGE_BYTES + wave * EPI_BYTES;
    // Scratch row r (128 bytes: the full width of the 32 banks) keeps its 16-byte chunks at slots chunk ^ swz(r),
    // and odd rows keep the two 8-byte halves of every chunk swapped: the sixteen lanes that write together hold
    // sixteen different rows and the same 8 bytes of each, and land in sixteen different bank pairs (with the chunk
    // swizzle alone rows 2j and 2j + 1 collided on every write: 1000 conflict cycles per plain tile, now 500 --
    // off the critical path either way, the layer's time did not move).
    // The read-back takes rows of one parity per instruction and swaps the halves of the odd ones by naming.
    auto swz = [](int r) { return (r >> 1) & 7; };
    const auto& orow_of = orows.r;
#pragma unroll
    for (int mp = 0; mp < MP; ++mp) {
#pragma unroll
      for (int og = 0; og < OBX / EPI_NB; ++og) {
        // write the 32 x EPI_COLS block: a lane holds, per accumulator block, token row frow and the four
        // output columns 4 * fhalf + [0, 4)
#pragma unroll
        for (int mbb = 0; mbb < EPI_MB; ++mbb) {
          const int mb = mp * EPI_MB + mbb;
          const int srow = mbb * MT + frow;
#pragma unroll
          for (int ob = 0; ob < EPI_NB; ++ob) {
            const int nb = og * EPI_NB + ob;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (WHAT == 1) {
                v[i] = acc[nb][mb][i];
              } else if (WHAT == 2) {
                v[i] = acc[nb + NB / 2][mb][i];
              } else if (GLU) {
                float up = acc[nb][mb][i];
                float gt = acc[nb + NB / 2][mb][i];
                if (KEEP) {
                  up = Elt<T>::round(up);
                  gt = Elt<T>::round(gt);
                }
                v[i] = up * gt * __builtin_amdgcn_rcpf(1.0f + __expf(-gt));
              } else {
                v[i] = acc[nb][mb][i];
              }
            }
            const int colp = ob * MT + fhalf * 4;  // column inside the pass
            const u32x2 p = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
            *reinterpret_cast<u32x2*>(scratch + srow * (EPI_COLS * 2) + (((colp >> 3) ^ swz(srow)) * 16) +
                                      (((colp >> 2) ^ srow) & 1) * 8) = p;
          }
        }
        // read back: lane -> row rb_row(it), 16-byte chunk lane%EPI_CPR
        const int cchunk = lane % EPI_CPR;
        // column of the result (the predicate's), and of what this form writes
        const int col = tc.nt * BN + (GLU ? wn * (WTN / 2) : wn * WTN) + og * EPI_COLS + cchunk * 8;
        const int dcol = WHAT == 2 ? a.N + col : col;
        // two reads at a time in front of their stores (one LDS latency for both): left alone, the compiler sinks
        // each read into its store's predicated region and waits for it there; all four at once do not fit next
        // to the accumulators
        constexpr int RB = 2;
        static_assert((32 / RPP) % RB == 0, "read-back batches");
#pragma unroll
        for (int it0 = 0; it0 < 32 / RPP; it0 += RB) {
          __builtin_amdgcn_sched_barrier(0);  // (one batch's addresses and values live at a time)
          u32x4 vals[RB];
#pragma unroll
          for (int j = 0; j < RB; ++j) {
            const int r = rb_row(it0 + j);
            const u32x4 v = *reinterpret_cast<const u32x4*>(scratch + r * (EPI_COLS * 2) + ((cchunk ^ swz(r)) * 16));
            vals[j] = ((it0 + j) & 1) ? u32x4{v[2], v[3], v[0], v[1]} : v;
          }
#pragma unroll
          for (int j = 0; j < RB; ++j) asm volatile("" : "+v"(vals[j]));
#pragma unroll
          for (int j = 0; j < RB; ++j) {
            const int it = it0 + j;
            const int r = rb_row(it);
            const int row = tc.row_begin + wm * WTM + mp * 32 + r;
            if (INTERIOR || (row < tc.row_end && col < a.N)) {
              int orow = orow_of[mp][it];
              asm volatile("" : "+v"(orow));  // (the address is formed here, not once per row and kept in registers)
              u32x4* dst = reinterpret_cast<u32x4*>(dst_base + (size_t)orow * ld + dcol);
              if constexpr (NT) __builtin_nontemporal_store(vals[j], dst);
              else *dst = vals[j];
            }
          }
        }
      }
    }
  };
  typedef std::integral_constant<int, 0> what_result;
  typedef std::integral_constant<int, 1> what_up;
  typedef std::integral_constant<int, 2> what_gate;
  auto epilogue = [&](const TileCoord& tc, const OutRows& orows) {
    const bool interior = tc.row_begin + BM <= tc.row_end && (tc.nt + 1) * BN <= a.N;
    if constexpr (KEEP_PRE) {
      {
        // the activation and both halves of the pre-activation (plain stores: the backward reads them again)
        if (interior) {
          epilogue_as(what_result{}, std::true_type{}, std::false_type{}, std::true_type{}, tc, orows);
          epilogue_as(what_up{}, std::true_type{}, std::false_type{}, std::true_type{}, tc, orows);
          epilogue_as(what_gate{}, std::true_type{}, std::false_type{}, std::true_type{}, tc, orows);
        } else {
          epilogue_as(what_result{}, std::false_type{}, std::false_type{}, std::true_type{}, tc, orows);
          epilogue_as(what_up{}, std::false_type{}, std::false_type{}, std::true_type{}, tc, orows);
          epilogue_as(what_gate{}, std::false_type{}, std::false_type{}, std::true_type{}, tc, orows);
        }
        return;
      }
    }
    if (interior) {
      if (a.out_nt) epilogue_as(what_result{}, std::true_type{}, std::true_type{}, std::false_type{}, tc, orows);
      else epilogue_as(what_result{}, std::true_type{}, std::false_type{}, std::false_type{}, tc, orows);
    } else {
      if (a.out_nt) epilogue_as(what_result{}, std::false_type{}, std::true_type{}, std::false_type{}, tc, orows);
      else epilogue_as(what_result{}, std::false_type{}, std::false_type{}, std::false_type{}, tc, orows);
    }
  };

  // ---- a part of a split tile: accumulators -> workspace (one partial tile per (XCD, slot), fp32) -----------------
  // Vector j of thread t lies at [j][t]: every store instruction writes 8 KB in a row.  The address is a uniform
  // base that moves from vector to vector plus one per-thread offset (the accumulators leave no registers for an
  // address per vector).
  auto store_part = [&]() {
    constexpr size_t PART_VECS = (size_t)NB * MB * NW * 64;  // f32x4 per partial tile
    unsigned t = tid;
    asm volatile("" : "+v"(t));  // (keeps the offset from being computed ahead of the tile loop and held through it)
    f32x4* base = static_cast<f32x4*>(a.ws) + ((size_t)sp.ws_base + (size_t)my_rem_tile * sp.parts + my_part) * PART_VECS;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) (base + (nb * MB + mb) * (NW * 64))[t] = acc[nb][mb];
  };

  // ---- tile loop -------------------------------------------------------------------------------------------
  int t0 = tile_of(0);
  if (t0 < 0) return;
  TileCoord c0, c1;
  locate(t0, c0);
  int t1 = tile_of(1);
  if (t1 >= 0) locate(t1, c1); else c1 = c0;
  int k0_cur, nk_cur, k0_next, nk_next;
  item_k(0, k0_cur, nk_cur);
  if (t1 >= 0) item_k(1, k0_next, nk_next); else { k0_next = k0_cur; nk_next = nk_cur; }
  TileSrc src_cur, src_next;
  {
    int raw0[NXLD], raw1[NXLD];
    load_rows(c0, raw0);
    load_rows(c1, raw1);
    make_src(c0, raw0, src_cur);
    make_src(c1, raw1, src_next);
  }
  OutRows out_cur, out_next;
  load_out_rows(c0, out_cur);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  constexpr int AHEAD = NSTAGE - 1;  // slices in flight ahead of the one being consumed
  static_assert(WN == 2, "two wave groups");
#pragma unroll
  for (int st = 0; st < AHEAD; ++st) dma_slice(src_cur, src_cur, false, k0_cur + st, st);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm((AHEAD - 1) * NLD, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  for (int i = 0;; ++i) {
    // the ring runs on into the next tile: the last AHEAD slices refill with its first AHEAD.
    // group wn == 1 runs one phase behind group wn == 0 inside a tile; both leave the tile together
    if (wn == 1) __builtin_amdgcn_s_barrier();
    // (a tile or a part of one has at least NSTAGE slices: the first is never among the last AHEAD)
    pp_slice(std::true_type{}, src_cur, src_next, false, k0_cur + AHEAD);
    for (int kt = 1; kt < nk_cur; ++kt) {
      const bool from_next = kt >= nk_cur - AHEAD;
      pp_slice(std::false_type{}, src_cur, src_next, from_next,
               from_next ? k0_next + kt + AHEAD - nk_cur : k0_cur + kt + AHEAD);
    }
    if (wn == 0) __builtin_amdgcn_s_barrier();
    if (nk_cur != nk) {
      // a part of a split tile, always a workgroup's last item: the finishing launch adds the parts up
      store_part();
      break;
    }
    const int t2 = tile_of(i + 2);
    TileCoord c2 = c1;
    if (t2 >= 0) locate(t2, c2);
    int raw2[NXLD];
    load_rows(c2, raw2);
    load_out_rows(c1, out_next);
    epilogue(c0, out_cur);
    // every wave is done with its scratch before any wave's DMA of the next tile lands in that stage
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (t1 < 0) {
      // The compiler folds this exit into the loop's back edge and then assumes, inside the slice loop, that
      // the row-index loads above may still be in flight (nobody consumes them on this path): it would drain
      // the DMA ring with vmcnt(0) at the top of every K slice.  Retiring them here keeps that path clean.
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
      break;
    }
    c0 = c1;
    c1 = c2;
    t1 = t2;
    src_cur = src_next;
    out_cur = out_next;
    k0_cur = k0_next;
    nk_cur = nk_next;
    if (t2 >= 0) item_k(i + 2, k0_next, nk_next);  // else: the surplus DMA of the last item re-reads its own slices
    make_src(c2, raw2, src_next);
    // Retire every load the compiler knows about (row indices, epilogue traffic) here, once per tile:
    // otherwise it re-checks them with vmcnt(0) inside the slice loop and drains the DMA ring there.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));  // surplus DMA must not outlive the workgroup's LDS
}

// The tiles the persistent kernel cut along K (see PERSIST_SPLIT_MAX): one workgroup per (XCD, tile of its last
// round) recomputes the same plan, adds the tile's partial accumulators in part order and writes the tile the way
// the persistent kernel's epilogue does (same arithmetic, same rounding; thread t holds what thread t of a part
// held).  Workgroups whose tile does not exist or was not split return at once.
template <typename T, int BM, int BNW, int WM, int WN, bool GLU>
__global__ __launch_bounds__(WM* WN * 64) void grouped_gemm_split_finish_kernel(GemmArgs a, int nslot) {
  constexpr int NW = WM * WN;
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr int WTM = BM / WM, WTN = BNW / WN;
  constexpr int MT = 16;
  constexpr int MB = WTM / MT, NB = WTN / MT;
  constexpr int OB = GLU ? NB / 2 : NB;
  constexpr size_t PART_VECS = (size_t)NB * MB * NW * 64;
  __shared__ int etab[2 * PERSIST_MAX_E];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;
  if (wave == 0) persist_expert_table<BM>(a.expert_offsets, a.E, etab);
  __syncthreads();
  const int total = etab[2 * (a.E - 1)] * a.n_tiles;
  // contiguous: workgroup b adds up tile b / 8 of XCD b % 8's last round; interleaved: tile b of the chip's last round
  const bool interleave = (a.remap & PERSIST_REMAP_INTERLEAVE) != 0;
  const int xcd = interleave ? 0 : (int)(blockIdx.x & 7), j = interleave ? (int)blockIdx.x : (int)(blockIdx.x >> 3);
  const SplitPlan sp = persist_split_plan(total, xcd, 0, nslot, a.K / 32, true, interleave);
  if (sp.parts == 1 || j >= sp.rem) return;
  TileCoord tc;
  persist_locate<BM>(etab, a.E, a.n_tiles, sp.rem_base + j, tc);

  // vector j of thread t of a part lies at [j][t]
  const f32x4* part = static_cast<const f32x4*>(a.ws) + ((size_t)sp.ws_base + (size_t)j * sp.parts) * PART_VECS + tid;
  f32x4 sum[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) sum[nb][mb] = __builtin_nontemporal_load(part + (nb * MB + mb) * (NW * 64));
  for (int p = 1; p < sp.parts; ++p) {
    part += PART_VECS;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const f32x4 v = __builtin_nontemporal_load(part + (nb * MB + mb) * (NW * 64));
#pragma unroll
        for (int c = 0; c < 4; ++c) sum[nb][mb][c] += v[c];
      }
  }

  // accumulator block (nb, mb): register i of a lane is output column 16 * nb + 4 * fhalf + i of the wave's
  // columns, token row 16 * mb + frow of the wave's rows; with SwiGLU block nb + NB / 2 holds the gate of block nb
  const int frow = lane % MT, fhalf = lane / MT;
  T* __restrict__ out = static_cast<T*>(a.out);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = tc.row_begin + wm * WTM + mb * MT + frow;
    if (row >= tc.row_end) continue;
    const int orow = a.scatter ? a.sorted_scattered[row] : row;
#pragma unroll
    for (int nb = 0; nb < OB; ++nb) {
      const int col = tc.nt * BN + (GLU ? wn * (WTN / 2) : wn * WTN) + nb * MT + fhalf * 4;
      if (col >= a.N) continue;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (GLU) {
          const float up = sum[nb][mb][i];
          const float gt = sum[nb + NB / 2][mb][i];
          v[i] = up * gt * __builtin_amdgcn_rcpf(1.0f + __expf(-gt));
        } else {
          v[i] = sum[nb][mb][i];
        }
      }
      const u32x2 p2 = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
      *reinterpret_cast<u32x2*>(out + (size_t)orow * a.N + col) = p2;
    }
  }
}

// ---- any-shape / any-dtype fallback (one thread per output element) ------------------------------
// Used for fp32 and for shapes the tiled kernel does not take (K % 8 != 0, N % 4 != 0, unaligned
// pointers).  Correct, not fast.
template <typename T, bool GLU>
__global__ __launch_bounds__(256) void grouped_gemm_naive_kernel(GemmArgs a) {
  const int col = blockIdx.y * 64 + (threadIdx.x & 63);
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.L || col >= a.N) return;
  int expert = 0;
  while (expert < a.E - 1 && a.expert_offsets[expert] <= row) ++expert;
  const int src = a.gather ? a.sorted_scattered[row] / a.kdiv : row;
  const int orow = a.scatter ? a.sorted_scattered[row] : row;
  const T* x = static_cast<const T*>(a.in) + (size_t)src * a.K;
  const T* w = static_cast<const T*>(a.w) + ((size_t)expert * (GLU ? 2 : 1) * a.N + col) * a.K;
  float up = 0.f, gt = 0.f;
  for (int k = 0; k < a.K; ++k) {
    float xv = Elt<T>::load(x + k);
    up = fmaf(xv, Elt<T>::load(w + k), up);
    if (GLU) gt = fmaf(xv, Elt<T>::load(w + (size_t)a.N * a.K + k), gt);
  }
  float r = GLU ? up * silu_f32(gt) : up;
  Elt<T>::store(static_cast<T*>(a.out) + (size_t)orow * a.N + col, r);
}

// ---- host side ------------------------------------------------------------------------------------

template <typename T, int BM, int BNW, int WM, int WN, bool GLU, bool KTAIL, bool W8 = false>
static int launch_tiled_k(GemmArgs a, hipStream_t s) {
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr size_t lds = 2ull * (BM + BNW) * 128;  // two stages of 128-byte rows
  auto kern = grouped_gemm_kernel<T, BM, BNW, WM, WN, GLU, KTAIL, W8>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_ok{0};
    const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok);
    if (rc != MI_MOE_OK) return rc;
  }
  a.n_tiles = mi_ceil_div(a.N, BN);
  long max_m = (long)a.L / BM + (a.E < a.L ? a.E : a.L);
  long grid = max_m * a.n_tiles;
  grid = (grid + 7) / 8 * 8;
  if (grid > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), lds, s, a);
  return mi_launch_status();
}

template <typename T, int BM, int BNW, int WM, int WN, bool GLU>
static int launch_tiled(GemmArgs a, hipStream_t s) {
  if (a.K % (128 / (int)sizeof(T)) == 0) return launch_tiled_k<T, BM, BNW, WM, WN, GLU, false>(a, s);
  return launch_tiled_k<T, BM, BNW, WM, WN, GLU, true>(a, s);
}

// fp8 weights (K tiles of 64 values: 64 bytes of a weight row)
template <typename T, int BM, int BNW, int WM, int WN, bool GLU>
static int launch_tiled_w8(GemmArgs a, hipStream_t s) {
  if (a.K % 64 == 0) return launch_tiled_k<T, BM, BNW, WM, WN, GLU, false, true>(a, s);
  return launch_tiled_k<T, BM, BNW, WM, WN, GLU, true, true>(a, s);
}

template <typename T, int BM, int BNW, int WM, int WN, bool GLU>
static int launch_dma(GemmArgs a, hipStream_t s) {
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr size_t lds = 4ull * (BM + BNW) * 32 * sizeof(T);
  auto kern = grouped_gemm_dma_kernel<T, BM, BNW, WM, WN, GLU>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_ok{0};
    const int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok);
    if (rc != MI_MOE_OK) return rc;
  }
  a.n_tiles = mi_ceil_div(a.N, BN);
  long max_m = (long)a.L / BM + (a.E < a.L ? a.E : a.L);
  long grid = max_m * a.n_tiles;
  grid = (grid + 7) / 8 * 8;
  if (grid > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), lds, s, a);
  return mi_launch_status();
}

template <typename T, int BM, int BNW, int WM, int WN, bool GLU, bool WT = false, bool KEEP_PRE = false>
static int launch_persistent(GemmArgs a, hipStream_t s) {
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr int NW = WM * WN;
  static_assert(BM * BNW * 4 == PERSIST_WS_TILE_BYTES, "size of a partial tile in the workspace");
  const size_t lds = 4ull * (BM + BNW) * 32 * sizeof(T) + (size_t)a.E * 8;
  auto kern = grouped_gemm_persistent_kernel<T, BM, BNW, WM, WN, GLU, WT, KEEP_PRE>;
  static std::atomic<uint64_t> lds_ok{0};  // the expert table makes lds vary with E: opt in to the most it can be
  int rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), MI_LDS_MAX_BYTES, lds_ok);
  if (rc != MI_MOE_OK) return rc;
  a.n_tiles = mi_ceil_div(a.N, BN);
  a.kshift = -1;
  if (a.kdiv > 0 && (a.kdiv & (a.kdiv - 1)) == 0)
    for (a.kshift = 0; (1 << a.kshift) < a.kdiv;) ++a.kshift;
  if (!(a.remap & PERSIST_REMAP_FIXED) && a.n_tiles >= 8) a.remap |= PERSIST_REMAP_INTERLEAVE;  // (see there)
  int cus = 0;
  if ((rc = mi_cu_count(&cus)) != MI_MOE_OK) return rc;
  long max_tiles = ((long)a.L / BM + (a.E < a.L ? a.E : a.L)) * a.n_tiles;
  long grid = cus < max_tiles ? cus : max_tiles;
  grid = (grid + 7) / 8 * 8;
  // no contraction length that a split could shorten by PERSIST_SPLIT_MIN_SAVED slices, or one slot per XCD
  if (!persistent_may_split(a.K) || grid < 16 || a.pre != nullptr) a.ws = nullptr;  // (the finishing launch writes the result only)
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), lds, s, a);
  if ((rc = mi_launch_status()) != MI_MOE_OK || a.ws == nullptr) return rc;
  // the tiles that were cut: at most half of the slots of a round that was split hold tiles (rounded up: an odd
  // number of slots per XCD)
  const int nslot = (int)(grid / 8);
  hipLaunchKernelGGL((grouped_gemm_split_finish_kernel<T, BM, BNW, WM, WN, GLU>), dim3(8u * (unsigned)((nslot + 1) / 2)),
                     dim3(NW * 64), 0, s, a, nslot);
  return mi_launch_status();
}

// fp8 expert weights on the register-staged tiles: out[orow(i)] = scale[e_i] * (in[irow(i)] @ Wq[e_i]^T), with SwiGLU
// over the [up ; gate] halves when glu.  Called by decode_fp8.hip for batches beyond a few rows per expert (the
// streaming kernels there read an expert's weights once per 16 of its rows).  Shapes: K % 16 == 0, N % 4 == 0,
// w_tiled only with K % 128 == 0; MI_MOE_EUNSUPPORTED otherwise.
template <typename T, bool GLU>
static int dispatch_w8(const GemmArgs& a, hipStream_t s) {
  const long avg = a.E > 0 ? (long)a.L / a.E : a.L;
  if (avg >= 512) return launch_tiled_w8<T, 256, 256, 2, 2, GLU>(a, s);
  if (avg >= 48) return launch_tiled_w8<T, 128, 128, 2, 2, GLU>(a, s);
  return launch_tiled_w8<T, 32, 128, 1, 2, GLU>(a, s);
}

int mi_gemm_fp8_tiled(const void* in, const void* wq, const float* scale, void* out, const int32_t* sorted_scattered,
                      const int32_t* expert_offsets, int L, int K, int N, int E, int kdiv, int gather, int scatter,
                      int glu, int w_tiled, int dtype, hipStream_t s) {
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (L == 0) return MI_MOE_OK;
  if (K % 16 != 0 || N % 4 != 0 || (w_tiled && K % 128 != 0)) return MI_MOE_EUNSUPPORTED;
  // 32-bit element offsets into the activations, 32-bit byte offsets inside one expert's weights
  const double in_rows = gather ? (double)L / (kdiv > 0 ? kdiv : 1) : (double)L;
  if (in_rows * K >= 2147483648.0) return MI_MOE_EUNSUPPORTED;
  const double wrows = w_tiled ? (double)mi_ceil_div(N, glu ? 16 : 32) * 32 : (double)(glu ? 2 : 1) * N;
  if (wrows * K >= 2147483648.0) return MI_MOE_EUNSUPPORTED;
  if (!mi_aligned(in, 16) || !mi_aligned(wq, 16) || !mi_aligned(scale, 16) || !mi_aligned(out, 8)) return MI_MOE_EALIGN;
  GemmArgs a;
  a.in = in; a.w = wq; a.out = out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = K; a.N = N; a.E = E; a.kdiv = kdiv > 0 ? kdiv : 1; a.kshift = -1; a.n_tiles = 0;
  a.gather = gather; a.scatter = scatter; a.remap = 1; a.ws = nullptr; a.pre = nullptr; a.out_nt = 0;
  a.wscale = scale; a.w_tiled = w_tiled;
  if (dtype == MI_MOE_BF16) return glu ? dispatch_w8<bf16_t, true>(a, s) : dispatch_w8<bf16_t, false>(a, s);
  return glu ? dispatch_w8<f16_t, true>(a, s) : dispatch_w8<f16_t, false>(a, s);
}

// workspace of the persistent kernel: one fp32 partial tile per workgroup of the largest grid
extern "C" size_t mi_moe_grouped_gemm_workspace_bytes(void) {
  int cus = 0;
  if (mi_cu_count(&cus) != MI_MOE_OK) return 0;
  return (size_t)((cus + 7) / 8 * 8) * PERSIST_WS_TILE_BYTES;
}

extern "C" int mi_moe_grouped_gemm_splits(int K, int dtype) {
  return (dtype == MI_MOE_BF16 || dtype == MI_MOE_F16) && K > 0 && K % 32 == 0 && persistent_may_split(K);
}

static int check_ws(const void* ws, size_t ws_bytes) {
  if (ws == nullptr) return MI_MOE_OK;
  const size_t need = mi_moe_grouped_gemm_workspace_bytes();
  if (need == 0 || ws_bytes < need) return MI_MOE_EWORKSPACE;
  return mi_aligned(ws, 16) ? MI_MOE_OK : MI_MOE_EALIGN;
}

static bool persistent_ok(const GemmArgs& a) {
  return a.K % 32 == 0 && a.K >= 128 && a.N % 8 == 0 && a.E <= PERSIST_MAX_E && mi_aligned(a.out, 16);
}

template <typename T, bool GLU>
static int launch_naive(GemmArgs a, hipStream_t s) {
  dim3 grid(mi_ceil_div(a.L, 4), mi_ceil_div(a.N, 64));
  if (grid.y > 65535u) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL((grouped_gemm_naive_kernel<T, GLU>), grid, dim3(256), 0, s, a);
  return mi_launch_status();
}

// tile configurations
//   0 / 1 / 2  register-staged 256x256 / 128x128 / 32x256 (any K % 8 == 0)
//   3          one thread per output element (any shape, any dtype)
//   4          DMA-staged 128x128, one tile per workgroup (K % 32 == 0)
//   7          persistent DMA-staged 256x256, 8 waves, 32-wide K slices, two wave groups in ping-pong
template <typename T, bool GLU>
static int dispatch_cfg(GemmArgs a, int cfg, hipStream_t s) {
  switch (cfg) {
    case 0: return launch_tiled<T, 256, 256, 2, 2, GLU>(a, s);
    case 1: return launch_tiled<T, 128, 128, 2, 2, GLU>(a, s);
    case 2: return launch_tiled<T, 32, 256, 1, 4, GLU>(a, s);
    case 5: return launch_tiled<T, 32, 128, 1, 2, GLU>(a, s);
    case 4: return a.K % 32 == 0 ? launch_dma<T, 128, 128, 2, 2, GLU>(a, s) : MI_MOE_EUNSUPPORTED;
    case 7: return persistent_ok(a) ? launch_persistent<T, 256, 256, 4, 2, GLU>(a, s) : MI_MOE_EUNSUPPORTED;
    case 8:  // the persistent kernel with the tile order fixed: XCDs own contiguous ranges ...
      a.remap |= PERSIST_REMAP_FIXED;
      return persistent_ok(a) ? launch_persistent<T, 256, 256, 4, 2, GLU>(a, s) : MI_MOE_EUNSUPPORTED;
    case 9:  // ... or take consecutive blocks of one chip-wide round
      a.remap |= PERSIST_REMAP_FIXED | PERSIST_REMAP_INTERLEAVE;
      return persistent_ok(a) ? launch_persistent<T, 256, 256, 4, 2, GLU>(a, s) : MI_MOE_EUNSUPPORTED;
    default: return MI_MOE_EUNSUPPORTED;
  }
}

// fp32 runs on the register-staged kernels only (32x32x2 matrix instructions)
template <bool GLU>
static int dispatch_cfg_f32(GemmArgs a, int cfg, hipStream_t s) {
  switch (cfg) {
    case 0: return launch_tiled<float, 256, 256, 2, 2, GLU>(a, s);
    case 1: return launch_tiled<float, 128, 128, 2, 2, GLU>(a, s);
    case 2: return launch_tiled<float, 32, 256, 1, 4, GLU>(a, s);
    case 5: return launch_tiled<float, 32, 128, 1, 2, GLU>(a, s);
    default: return MI_MOE_EUNSUPPORTED;
  }
}

// Shapes the matrix-core kernels take: 16-byte chunks along K (8 elements of a 16-bit type, 4 of fp32), four
// results per output piece, 32-bit element offsets inside one operand.
static bool tiled_shape_ok(const GemmArgs& a, int in_rows_bound, bool glu, int elt_bytes) {
  if (a.K % (16 / elt_bytes) != 0 || a.N % 4 != 0) return false;
  if ((double)in_rows_bound * a.K >= 2147483648.0) return false;
  if ((double)(glu ? 2 : 1) * a.N * a.K >= 2147483648.0) return false;
  return true;
}
static bool tiled_aligned(const GemmArgs& a, int elt_bytes) {
  return mi_aligned(a.in, 16) && mi_aligned(a.w, 16) && mi_aligned(a.out, 4 * elt_bytes);
}

static int pick_cfg(const GemmArgs& a) {
  const long avg = a.E > 0 ? (long)a.L / a.E : a.L;  // rows per expert if the load were uniform
  if (avg >= 192 && persistent_ok(a)) return 7;
  if (avg >= 512) return 0;
  if (avg >= 48) return a.K % 32 == 0 ? 4 : 1;
  // A few rows per expert: every weight byte is used once and the kernel is a weight stream, which wants many
  // workgroups.  Measured at 8 - 256 tokens (kernel times, up / down projection): hidden 1536, 40 experts -- 32 x 256
  // tiles 29 - 31 / 13.5 - 17 us, 32 x 128 tiles 23 - 27 / 12 - 17 us, DMA-staged 128 x 128 tiles 28 - 30 / 13 - 16 us;
  // hidden 1024, 32 experts -- 20 - 22 / 12 - 15, 16 - 21 / 9 - 13, 15 - 16 / 9 - 11 us.  A very long contraction
  // (the down-projection of an intermediate size of 14336: 226 against 188 us at 64 tokens) wants the deeper ring of
  // the DMA-staged kernel too.
  return (a.K % 32 == 0 && (a.K <= 1024 || a.K >= 8192)) ? 4 : 5;
}

// cfg < 0 picks a matrix-core kernel from the shape.  Nothing drops to the one-thread-per-output kernel on its own:
// a problem the matrix-core kernels cannot take is refused (MI_MOE_EALIGN for a misaligned pointer,
// MI_MOE_EUNSUPPORTED for the shape) and the caller asks for cfg 3 explicitly if it wants the slow kernel.
// Cache policy of the persistent kernel's output stores.  The plain form's output -- the (slots, hidden) rows the
// combine streams once -- is stored non-temporal, so that it does not push the operands out of the caches:
// down-projection of the 16384-token, 32-expert shape 0.169 -> 0.146 ms (its combine 0.048 -> 0.053 ms), little
// either way on the other shapes.  The SwiGLU form's output is the next GEMM's operand: up to about the size the
// memory-side cache can hold next to the weights it stays cached (134 MB on that shape: non-temporal stores would
// make the GEMM that reads it back 8 % slower); beyond that it would not survive until it is read and only evicts
// the operands on its way (268 MB on the 32768-token, 40-expert shape: both GEMMs 1 % faster non-temporal).
static int persistent_out_nt(const GemmArgs& a, bool glu, int elt) {
  if (!glu) return 1;
  return (double)a.L * a.N * elt > 192.0 * 1024 * 1024;
}

static int run_gemm(GemmArgs a, int dtype, bool glu, int cfg, int in_rows_bound, hipStream_t s) {
  a.out_nt = persistent_out_nt(a, glu, dtype == MI_MOE_F32 ? 4 : 2);
  if (a.L == 0) return MI_MOE_OK;
  if (dtype != MI_MOE_F32 && dtype != MI_MOE_F16 && dtype != MI_MOE_BF16) return MI_MOE_EDTYPE;
  if (cfg == 3) {
    switch (dtype) {
      case MI_MOE_F32: return glu ? launch_naive<float, true>(a, s) : launch_naive<float, false>(a, s);
      case MI_MOE_F16: return glu ? launch_naive<f16_t, true>(a, s) : launch_naive<f16_t, false>(a, s);
      default: return glu ? launch_naive<bf16_t, true>(a, s) : launch_naive<bf16_t, false>(a, s);
    }
  }
  const int elt = dtype == MI_MOE_F32 ? 4 : 2;
  if (!tiled_shape_ok(a, in_rows_bound, glu, elt)) return MI_MOE_EUNSUPPORTED;
  if (!tiled_aligned(a, elt)) return MI_MOE_EALIGN;
  if (dtype == MI_MOE_F32) {
    if (cfg < 0) {
      // fp32 matrix instructions are slow enough that what matters is how many CUs have a tile.  Measured (up /
      // down projection, us): 128 x 128 tiles beat 256 x 256 at every size tried (262144 rows, 40 experts, hidden
      // 1536: 3240 / 1678 against 3359 / 1690; 65536 rows, 32 experts: 1136 / 585 against 1338 / 686), and below
      // about two 128 x 128 tiles per CU the 32 x 256 tiles win (the reference's correctness configuration, 1024
      // rows in 8 experts: 15 / 24 against 23 / 37; 4096 rows: 38 / 25 against 43 / 38 and, for 256 x 256, 73 / 127).
      const long avg = a.E > 0 ? (long)a.L / a.E : a.L;
      const long tiles128 = ((long)a.L / 128 + a.E / 2 + 1) * mi_ceil_div((glu ? 2 : 1) * a.N, 128);
      cfg = avg < 48 ? 5 : ((avg >= 512 && tiles128 >= 512) ? 1 : 2);
    }
    return glu ? dispatch_cfg_f32<true>(a, cfg, s) : dispatch_cfg_f32<false>(a, cfg, s);
  }
  if (cfg < 0) cfg = pick_cfg(a);
  if (dtype == MI_MOE_BF16) return glu ? dispatch_cfg<bf16_t, true>(a, cfg, s) : dispatch_cfg<bf16_t, false>(a, cfg, s);
  return glu ? dispatch_cfg<f16_t, true>(a, cfg, s) : dispatch_cfg<f16_t, false>(a, cfg, s);
}

static int check_common(const void* in, const void* w, void* out, const int32_t* ss, const int32_t* off, int L, int K,
                        int N, int E, int k, int dtype, bool need_ss) {
  if (L < 0 || K < 1 || N < 1 || E < 1 || E > 65536 || k < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_F32 && dtype != MI_MOE_F16 && dtype != MI_MOE_BF16) return MI_MOE_EDTYPE;
  if (L == 0) return MI_MOE_OK;
  if (!in || !w || !out || !off) return MI_MOE_ENULL;
  if (need_ss && !ss) return MI_MOE_ENULL;
  return MI_MOE_OK;
}

extern "C" int mi_moe_scattered_gemm_ws(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                                        const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                        int grouped_in, int grouped_out, int dtype, int cfg, void* ws,
                                        size_t ws_bytes, mi_moe_stream_t stream) {
  int rc = check_common(in, w, out, sorted_scattered, expert_offsets, L, K, N, E, k, dtype,
                        !grouped_in || !grouped_out);
  if (rc != MI_MOE_OK) return rc;
  if ((rc = check_ws(ws, ws_bytes)) != MI_MOE_OK) return rc;
  GemmArgs a;
  a.in = in; a.w = w; a.out = out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = K; a.N = N; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = !grouped_in; a.scatter = !grouped_out; a.remap = 1; a.ws = ws; a.pre = nullptr;
  return run_gemm(a, dtype, false, cfg, L, static_cast<hipStream_t>(stream));
}

extern "C" int mi_moe_scattered_gemm_cfg(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                                         const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                         int grouped_in, int grouped_out, int dtype, int cfg,
                                         mi_moe_stream_t stream) {
  return mi_moe_scattered_gemm_ws(in, w, out, sorted_scattered, expert_offsets, L, K, N, E, k, grouped_in,
                                  grouped_out, dtype, cfg, nullptr, 0, stream);
}

extern "C" int mi_moe_scattered_gemm_wt_ws(const void* in, const void* w_kn, void* out,
                                           const int32_t* sorted_scattered, const int32_t* expert_offsets, int L,
                                           int K, int N, int E, int k, int grouped_in, int grouped_out, int dtype,
                                           void* ws, size_t ws_bytes, mi_moe_stream_t stream) {
  int rc = check_common(in, w_kn, out, sorted_scattered, expert_offsets, L, K, N, E, k, dtype,
                        !grouped_in || !grouped_out);
  if (rc != MI_MOE_OK) return rc;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if ((rc = check_ws(ws, ws_bytes)) != MI_MOE_OK) return rc;
  if (L == 0) return MI_MOE_OK;
  GemmArgs a;
  a.in = in; a.w = w_kn; a.out = out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = K; a.N = N; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = !grouped_in; a.scatter = !grouped_out; a.remap = 1; a.ws = ws; a.pre = nullptr;
  a.out_nt = persistent_out_nt(a, false, 2);
  if (!tiled_shape_ok(a, L, false, 2) || !persistent_ok(a)) return MI_MOE_EUNSUPPORTED;
  if (!tiled_aligned(a, 2)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MI_MOE_BF16) return launch_persistent<bf16_t, 256, 256, 4, 2, false, true>(a, s);
  return launch_persistent<f16_t, 256, 256, 4, 2, false, true>(a, s);
}

extern "C" int mi_moe_scattered_gemm_wt(const void* in, const void* w_kn, void* out, const int32_t* sorted_scattered,
                                        const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                        int grouped_in, int grouped_out, int dtype, mi_moe_stream_t stream) {
  return mi_moe_scattered_gemm_wt_ws(in, w_kn, out, sorted_scattered, expert_offsets, L, K, N, E, k, grouped_in,
                                     grouped_out, dtype, nullptr, 0, stream);
}

extern "C" int mi_moe_scattered_gemm(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                                     const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                     int grouped_in, int grouped_out, int dtype, mi_moe_stream_t stream) {
  return mi_moe_scattered_gemm_cfg(in, w, out, sorted_scattered, expert_offsets, L, K, N, E, k, grouped_in,
                                   grouped_out, dtype, -1, stream);
}

extern "C" int mi_moe_up_swiglu_ws(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                                   const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                                   int cfg, void* ws, size_t ws_bytes, mi_moe_stream_t stream) {
  int rc = check_common(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, true);
  if (rc != MI_MOE_OK) return rc;
  if ((rc = check_ws(ws, ws_bytes)) != MI_MOE_OK) return rc;
  GemmArgs a;
  a.in = x; a.w = w_fc; a.out = act_out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = H; a.N = I; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = 1; a.scatter = 0; a.remap = 1; a.ws = ws; a.pre = nullptr;
  return run_gemm(a, dtype, true, cfg, L, static_cast<hipStream_t>(stream));
}

extern "C" int mi_moe_up_swiglu_keep(const void* x, const void* w_fc, void* act_out, void* pre_out,
                                     const int32_t* sorted_scattered, const int32_t* expert_offsets, int L, int H, int I,
                                     int E, int k, int dtype, mi_moe_stream_t stream) {
  int rc = check_common(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, true);
  if (rc != MI_MOE_OK) return rc;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (L == 0) return MI_MOE_OK;
  if (!pre_out) return MI_MOE_ENULL;
  if (!mi_aligned(pre_out, 16)) return MI_MOE_EALIGN;
  GemmArgs a;
  a.in = x; a.w = w_fc; a.out = act_out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = H; a.N = I; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = 1; a.scatter = 0; a.remap = 1; a.ws = nullptr; a.pre = pre_out;
  // only the persistent kernel writes the pre-activation: shapes it does not take, and loads for which another
  // kernel would be picked, are the caller's two-call path
  if (!persistent_ok(a) || pick_cfg(a) != 7) return MI_MOE_EUNSUPPORTED;
  if (!tiled_shape_ok(a, L, true, 2)) return MI_MOE_EUNSUPPORTED;
  if (!tiled_aligned(a, 2)) return MI_MOE_EALIGN;
  a.out_nt = 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MI_MOE_BF16) return launch_persistent<bf16_t, 256, 256, 4, 2, true, false, true>(a, s);
  return launch_persistent<f16_t, 256, 256, 4, 2, true, false, true>(a, s);
}

extern "C" int mi_moe_up_swiglu_cfg(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                                    const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                                    int cfg, mi_moe_stream_t stream) {
  return mi_moe_up_swiglu_ws(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, cfg, nullptr, 0,
                             stream);
}

extern "C" int mi_moe_up_swiglu(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                                const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                                mi_moe_stream_t stream) {
  return mi_moe_up_swiglu_cfg(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, -1, stream);
}
