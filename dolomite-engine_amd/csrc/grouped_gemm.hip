// Grouped ("scatter2scatter") GEMM of the scattered-MoE forward on gfx950 matrix cores.
//
//   out[orow(i), :] = in[irow(i), :] @ W[e_i]^T        for every row i of the expert-sorted order
//
// with an optional SwiGLU epilogue (W rows [0,N) are "up", [N,2N) "gate"; out = up * silu(gate)).
// Stands in for the external scattered_experts op called at
// lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:91-101 (call sites moe.py:273-290) and for
// GLUActivation (activations/glu.py:42-43) when fused.
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
  int n_tiles;  // column tiles per row tile
  int gather;   // input row of sorted row i is sorted_scattered[i] / kdiv (else i)
  int scatter;  // output row of sorted row i is sorted_scattered[i] (else i)
  int remap;    // XCD-aware tile order
};

template <typename T, int BM, int BNW, int BK, int WM, int WN, bool GLU>
__global__ __launch_bounds__(WM* WN * 64) void grouped_gemm_kernel(GemmArgs a) {
  constexpr int NT = WM * WN * 64;
  constexpr int CPR = BK / 8;               // 16-byte chunks per tile row
  constexpr int RS = NT / CPR;              // tile rows covered by one pass of the workgroup
  constexpr int XCH = BM * CPR / NT;        // chunks per thread, activation tile
  constexpr int WCH = BNW * CPR / NT;       // chunks per thread, weight tile
  constexpr int BN = GLU ? BNW / 2 : BNW;   // output columns per tile
  constexpr int WTM = BM / WM;              // wave tile, rows
  constexpr int WTN = BNW / WN;             // wave tile, weight rows
  constexpr int MB = WTM / 32, NB = WTN / 32;
  constexpr int STAGE_ELEMS = (BM + BNW) * BK;
  static_assert(BK == 64 || BK == 32, "BK");
  static_assert(RS % 8 == 0 && BM % RS == 0 && BNW % RS == 0, "tile/thread shape");
  static_assert(!GLU || NB % 2 == 0, "SwiGLU needs an even number of column blocks per wave");
  typedef typename Mfma32<T>::vec frag_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;
  const int32_t* __restrict__ off = a.expert_offsets;

  // ---- which tile is mine --------------------------------------------------------------------
  int total_m = 0;
  {
    int prev = 0;
    for (int e = 0; e < a.E; ++e) {
      int end = off[e];
      total_m += (end - prev + BM - 1) / BM;
      prev = end;
    }
  }
  const int total = total_m * a.n_tiles;
  int tile;
  if (a.remap) {
    const int per = (total + 7) >> 3;
    const int local = blockIdx.x >> 3;
    if (local >= per) return;
    tile = (blockIdx.x & 7) * per + local;
  } else {
    tile = blockIdx.x;
  }
  if (tile >= total) return;
  const int mt = tile / a.n_tiles, nt = tile - mt * a.n_tiles;
  int expert = 0, row_begin = 0, row_end = 0;
  {
    int prev = 0, acc = 0;
    for (int e = 0; e < a.E; ++e) {
      int end = off[e];
      int tiles = (end - prev + BM - 1) / BM;
      if (mt < acc + tiles) {
        expert = e;
        row_begin = prev + (mt - acc) * BM;
        row_end = end;
        break;
      }
      acc += tiles;
      prev = end;
    }
  }

  // ---- per-thread global sources ---------------------------------------------------------------
  const int c = tid % CPR;   // chunk within a tile row
  const int r0 = tid / CPR;  // first tile row of this thread
  constexpr int WROWS_MUL = GLU ? 2 : 1;
  const T* __restrict__ xbase = static_cast<const T*>(a.in);
  const T* __restrict__ wbase = static_cast<const T*>(a.w) + (size_t)expert * WROWS_MUL * a.N * a.K;

  uint32_t xoff[XCH], woff[WCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    int srow = row_begin + r0 + j * RS;
    if (srow > row_end - 1) srow = row_end - 1;  // tail rows re-read the last valid row; never stored
    int src = a.gather ? a.sorted_scattered[srow] / a.kdiv : srow;
    xoff[j] = (uint32_t)src * (uint32_t)a.K + c * 8;
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
    woff[j] = (uint32_t)(half * a.N + col) * (uint32_t)a.K + c * 8;
  }

  // swizzled LDS chunk slot of this thread's chunks (same for all its rows because RS % 8 == 0)
  const int sw_c = (BK == 64) ? (c ^ (r0 & 7)) : (c ^ ((r0 >> 1) & 3));
  const int st_x = (r0 * CPR + sw_c) * 8;              // element offset inside the X tile
  const int st_w = BM * BK + (r0 * CPR + sw_c) * 8;    // ... inside the W tile (after the X tile)

  u32x4 xreg[XCH], wreg[WCH];
  const int nk = (a.K + BK - 1) / BK;

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
    const bool kvalid = (k0 + c * 8) < a.K;
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (kvalid) v = *reinterpret_cast<const u32x4*>(xbase + xoff[j] + k0);
      xreg[j] = v;
    }
#pragma unroll
    for (int j = 0; j < WCH; ++j) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (kvalid) v = *reinterpret_cast<const u32x4*>(wbase + woff[j] + k0);
      wreg[j] = v;
    }
  };
  auto store_lds = [&](int stage) {
    T* s = smem + stage * STAGE_ELEMS;
#pragma unroll
    for (int j = 0; j < XCH; ++j) *reinterpret_cast<u32x4*>(s + st_x + j * RS * BK) = xreg[j];
#pragma unroll
    for (int j = 0; j < WCH; ++j) *reinterpret_cast<u32x4*>(s + st_w + j * RS * BK) = wreg[j];
  };

  // ---- fragment read addresses ----------------------------------------------------------------------
  // lane l reads tile row (block_row0 + l%32), logical chunk 2*kk + l/32
  const int frow = lane & 31, fhalf = lane >> 5;
  int frag_x_row[MB], frag_w_row[NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) frag_x_row[mb] = wm * WTM + mb * 32 + frow;
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
    frag_w_row[nb] = r;
  }

  f32x16 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][mb][i] = 0.f;

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk) load_global(kt + 1);
    const T* sx = smem + (kt & 1) * STAGE_ELEMS;
    const T* sw = sx + BM * BK;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int chunk = kk * 2 + fhalf;
      frag_t xf[MB], wf[NB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        int r = frag_x_row[mb];
        int pc = (BK == 64) ? (chunk ^ (r & 7)) : (chunk ^ ((r >> 1) & 3));
        xf[mb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(sx + (r * CPR + pc) * 8));
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        int r = frag_w_row[nb];
        int pc = (BK == 64) ? (chunk ^ (r & 7)) : (chunk ^ ((r >> 1) & 3));
        wf[nb] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4*>(sw + (r * CPR + pc) * 8));
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = Mfma32<T>::run(wf[nb], xf[mb], acc[nb][mb]);
    }
    if (kt + 1 < nk) store_lds((kt + 1) & 1);
    __syncthreads();
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

template <typename T, int BM, int BNW, int BK, int WM, int WN, bool GLU>
static int launch_tiled(GemmArgs a, hipStream_t s) {
  constexpr int BN = GLU ? BNW / 2 : BNW;
  constexpr size_t lds = 2ull * (BM + BNW) * BK * sizeof(T);
  auto kern = grouped_gemm_kernel<T, BM, BNW, BK, WM, WN, GLU>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  a.n_tiles = mi_ceil_div(a.N, BN);
  long max_m = (long)a.L / BM + (a.E < a.L ? a.E : a.L);
  long grid = max_m * a.n_tiles;
  grid = (grid + 7) / 8 * 8;
  if (grid > 0x7fffffffL) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WM * WN * 64), lds, s, a);
  return mi_launch_status();
}

template <typename T, bool GLU>
static int launch_naive(GemmArgs a, hipStream_t s) {
  dim3 grid(mi_ceil_div(a.L, 4), mi_ceil_div(a.N, 64));
  if (grid.y > 65535u) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL((grouped_gemm_naive_kernel<T, GLU>), grid, dim3(256), 0, s, a);
  return mi_launch_status();
}

// tile configurations: 0 = 256x256 (4 waves), 1 = 128x128 (4 waves), 2 = 32x128 (4 waves), 3 = naive
template <typename T, bool GLU>
static int dispatch_cfg(GemmArgs a, int cfg, hipStream_t s) {
  switch (cfg) {
    case 0: return launch_tiled<T, 256, 256, 64, 2, 2, GLU>(a, s);
    case 1: return launch_tiled<T, 128, 128, 64, 2, 2, GLU>(a, s);
    case 2: return launch_tiled<T, 32, 256, 64, 1, 4, GLU>(a, s);
    default: return MI_MOE_EUNSUPPORTED;
  }
}

static bool tiled_ok(const GemmArgs& a, int in_rows_bound, bool glu) {
  if (a.K % 8 != 0 || a.N % 4 != 0) return false;
  if (!mi_aligned(a.in, 16) || !mi_aligned(a.w, 16) || !mi_aligned(a.out, 8)) return false;
  // 32-bit element offsets inside one operand
  if ((double)in_rows_bound * a.K >= 2147483648.0) return false;
  if ((double)(glu ? 2 : 1) * a.N * a.K >= 2147483648.0) return false;
  return true;
}

static int pick_cfg(const GemmArgs& a) {
  long avg = a.E > 0 ? (long)a.L / a.E : a.L;
  if (avg >= 512) return 0;
  if (avg >= 48) return 1;
  return 2;
}

static int run_gemm(GemmArgs a, int dtype, bool glu, int cfg, int in_rows_bound, hipStream_t s) {
  if (a.L == 0) return MI_MOE_OK;
  const bool fast = (dtype == MI_MOE_BF16 || dtype == MI_MOE_F16) && tiled_ok(a, in_rows_bound, glu);
  if (cfg == 3 || !fast) {
    if (cfg >= 0 && cfg != 3) return MI_MOE_EUNSUPPORTED;
    switch (dtype) {
      case MI_MOE_F32: return glu ? launch_naive<float, true>(a, s) : launch_naive<float, false>(a, s);
      case MI_MOE_F16: return glu ? launch_naive<f16_t, true>(a, s) : launch_naive<f16_t, false>(a, s);
      case MI_MOE_BF16: return glu ? launch_naive<bf16_t, true>(a, s) : launch_naive<bf16_t, false>(a, s);
      default: return MI_MOE_EDTYPE;
    }
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

extern "C" int mi_moe_scattered_gemm_cfg(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                                         const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                         int grouped_in, int grouped_out, int dtype, int cfg,
                                         mi_moe_stream_t stream) {
  int rc = check_common(in, w, out, sorted_scattered, expert_offsets, L, K, N, E, k, dtype,
                        !grouped_in || !grouped_out);
  if (rc != MI_MOE_OK) return rc;
  GemmArgs a;
  a.in = in; a.w = w; a.out = out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = K; a.N = N; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = !grouped_in; a.scatter = !grouped_out; a.remap = 1;
  return run_gemm(a, dtype, false, cfg, L, static_cast<hipStream_t>(stream));
}

extern "C" int mi_moe_scattered_gemm(const void* in, const void* w, void* out, const int32_t* sorted_scattered,
                                     const int32_t* expert_offsets, int L, int K, int N, int E, int k,
                                     int grouped_in, int grouped_out, int dtype, mi_moe_stream_t stream) {
  return mi_moe_scattered_gemm_cfg(in, w, out, sorted_scattered, expert_offsets, L, K, N, E, k, grouped_in,
                                   grouped_out, dtype, -1, stream);
}

extern "C" int mi_moe_up_swiglu_cfg(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                                    const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                                    int cfg, mi_moe_stream_t stream) {
  int rc = check_common(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, true);
  if (rc != MI_MOE_OK) return rc;
  GemmArgs a;
  a.in = x; a.w = w_fc; a.out = act_out;
  a.sorted_scattered = sorted_scattered; a.expert_offsets = expert_offsets;
  a.L = L; a.K = H; a.N = I; a.E = E; a.kdiv = k; a.n_tiles = 0;
  a.gather = 1; a.scatter = 0; a.remap = 1;
  return run_gemm(a, dtype, true, cfg, L, static_cast<hipStream_t>(stream));
}

extern "C" int mi_moe_up_swiglu(const void* x, const void* w_fc, void* act_out, const int32_t* sorted_scattered,
                                const int32_t* expert_offsets, int L, int H, int I, int E, int k, int dtype,
                                mi_moe_stream_t stream) {
  return mi_moe_up_swiglu_cfg(x, w_fc, act_out, sorted_scattered, expert_offsets, L, H, I, E, k, dtype, -1, stream);
}
