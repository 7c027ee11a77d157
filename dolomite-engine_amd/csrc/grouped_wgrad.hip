// Per-expert weight gradients of the scattered-MoE layer on gfx950 matrix cores:
//
//   dW[e][m][n] = sum over the rows r of expert e (expert-sorted order) of  A[ai(r)][m] * B[bi(r)][n]
//
// i.e. one "X^T dY" product per expert, contracted over that expert's rows.  The reference gets it from the
// backward of the external scattered_experts op (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:91-101);
// its two uses are d c_fc[e] = d_h[rows_e]^T x[token(rows_e)] and d c_proj[e] = dy[token(rows_e)]^T act[rows_e].
//
// Design
//   * Both operands are stored with the contraction index (the row) as the slow dimension, the opposite of what
//     the matrix instruction wants (8 consecutive contraction values per lane).  The tiles are staged in LDS as
//     they lie in HBM -- [row][256 columns] -- and the fragments are read with ds_read_b64_tr_b16, which transposes
//     4 rows x 16 columns across a group of 16 lanes: lane i of the group supplies the address of (row i / 4,
//     columns 4 * (i % 4) ..) and receives column i of the four rows.  Two such reads make one 16x16x32 operand.
//     The 32-byte column groups of a row are XOR-swizzled with the row number so that the 16 rows x 32 bytes of
//     one read spread over the banks.
//   * An expert's rows are cut into groups of `chunk` rows; a work item is one 256 x 256 output tile of one
//     group.  Items are dealt so that the 32 workgroups of an XCD work on the tiles of the same few groups at
//     the same time: the group's rows are then fetched from HBM once per XCD and shared through its L2.
//     Which XCD takes which groups is planned by a one-workgroup kernel in front: the groups are ranked by size,
//     longest first, and dealt to the eight XCDs back and forth (0..7, 7..0, ...), so that the XCDs get equal
//     work up to a small group and every XCD ends on its shortest items.  (Dealing the sorted rows into eight
//     equal ranges instead leaves the XCDs up to one group apart and costs 10 - 20 % under skewed loads.)
//     An item of an expert with several groups writes an fp32 partial tile and a second kernel sums the partials
//     of the expert in group order and rounds once (deterministic); an expert with one group is written directly,
//     one without rows gets zeros from the second kernel.
//   * HBM -> LDS by DMA (no registers), a ring of four 32-row slices with three in flight, and the forward
//     kernel's ping-pong schedule: the two waves of a SIMD alternate between a memory phase and a matrix phase.
//     A row's address is a scalar (index loads go through the scalar cache), the lanes add constant offsets.
#include "common.h"

#include <type_traits>

#define WGRAD_MAX_E 256

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
#define MI_LDS __attribute__((address_space(3)))

template <typename T> struct WgradMfma;
template <> struct WgradMfma<bf16_t> {
  static __device__ __forceinline__ f32x4 run(s16x8 a, s16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct WgradMfma<f16_t> {
  static __device__ __forceinline__ f32x4 run(s16x8 a, s16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

struct WgradArgs {
  const void* a;                  // (rows_a, M)
  const void* b;                  // (rows_b, N)
  const int32_t* a_idx;           // (L,) row of `a` for sorted row r, or null: r itself
  const int32_t* b_idx;           // same for `b`
  const int32_t* expert_offsets;  // (E,) inclusive ends of the experts' row ranges
  float* partial;                 // [group][M][N]
  void* dw;                       // (E, M, N): written directly for an expert with a single group
  int* next_item;                 // plan: [0..8) per-XCD work counters, zero on entry; [8..17) first slot of each XCD
                                  // in the list; [32..) the groups in the order the XCDs work through them
  int L, M, N, E, chunk, m_tiles, n_tiles;
};

__device__ __forceinline__ constexpr int wgrad_waitcnt(int vm, int lgkm) {
  // gfx9 encoding: vmcnt = {imm[15:14], imm[3:0]}, expcnt = imm[6:4] (7 = no wait), lgkmcnt = imm[11:8]
  return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}

// etab[2e] = groups of experts 0..e, etab[2e+1] = offsets[e]; returns nothing, all threads must call
__device__ __forceinline__ void wgrad_build_table(const int32_t* __restrict__ offsets, int E, int chunk, int* etab, int lane,
                                                  int wave) {
  if (wave == 0) {
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int end = e < E ? offsets[e] : 0;
      const int prev = (e < E && e > 0) ? offsets[e - 1] : 0;
      int incl = e < E ? (end - prev + chunk - 1) / chunk : 0;
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
  __syncthreads();
}

// Two rows of a tile (512 bytes each) into 1 KiB of LDS starting at `lds_addr`: lanes 0-31 fetch 16 bytes each
// from base + row_lo + off, lanes 32-63 from base + row_hi + off (32-bit byte offsets); lane l lands at
// lds_addr + 16 l.  The row offsets are scalars (a gathered operand has an unrelated address per row) and the
// lane offsets never change; their per-lane sum lives in a register that only this statement names.  Written as
// assembly for the same reason as in the forward kernel: the compiler would order every later LDS read behind the
// builtin form of this instruction with vmcnt(0).
__device__ __forceinline__ void wgrad_dma_row_pair(const void* base, uint32_t row_lo, uint32_t row_hi, uint32_t off,
                                                   uint64_t upper_half, uint32_t lds_addr) {
  uint32_t tmp;
  uint64_t saved;
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_mov_b64 %1, exec\n\t"
      "v_add_u32 %0, %4, %3\n\t"
      "s_mov_b64 exec, %7\n\t"
      "v_add_u32 %0, %5, %3\n\t"
      "s_mov_b64 exec, %1\n\t"
      "global_load_lds_dwordx4 %0, %6"
      : "=&v"(tmp), "=&s"(saved)
      : "s"(lds_addr), "v"(off), "s"(row_lo), "s"(row_hi), "s"(base), "s"(upper_half)
      : "memory", "m0");
}

template <typename T>
__global__ __launch_bounds__(512) void grouped_wgrad_kernel(WgradArgs a) {
  constexpr int BK = 32, TILE = 256;
  constexpr int OP_BYTES = BK * TILE * 2;  // one operand's 32 rows x 256 columns
  constexpr int STAGE_BYTES = 2 * OP_BYTES;
  constexpr int NSTAGE = 4, AHEAD = 3;
  constexpr int NLD = 4;                   // DMA instructions per wave and slice (4 row pairs)
  typedef const __attribute__((address_space(4))) int32_t* const_idx_t;
  typedef int32_t i32x8_a4 __attribute__((ext_vector_type(8), aligned(4)));
  typedef const __attribute__((address_space(4))) i32x8_a4* const_idx8_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int* etab = reinterpret_cast<int*>(smem_raw + NSTAGE * STAGE_BYTES);
  int* item_slot = etab + 2 * a.E;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 3, wn = wave >> 2;

  wgrad_build_table(a.expert_offsets, a.E, a.chunk, etab, lane, wave);
  const int tiles = a.m_tiles * a.n_tiles;
  const int xcd = blockIdx.x & 7;

  // An expert with n rows has ceil(n / chunk) groups of equal size (a multiple of 32 rows, the last one shorter).
  auto group_rows = [&](int n, int groups) { return ((n + groups - 1) / groups + 31) & ~31; };
  // this XCD's groups: slots [xfirst, xfirst + xgroups) of the planned list
  const int xfirst = a.next_item[8 + xcd];
  const int xgroups = a.next_item[8 + xcd + 1] - xfirst;
  const int* __restrict__ xlist = a.next_item + 32 + xfirst;
  const int items_x = xgroups * tiles;

  // ---- loader role: waves 0-3 stage operand A, waves 4-7 operand B; each wave rows 8 wq .. 8 wq + 7 of a slice --
  const bool load_b = wave >= 4;
  const int wq = wave & 3;
  const unsigned char* src = static_cast<const unsigned char*>(load_b ? a.b : a.a);
  const const_idx_t idx = reinterpret_cast<const_idx_t>(reinterpret_cast<uintptr_t>(load_b ? a.b_idx : a.a_idx));
  const int ld = load_b ? a.N : a.M;  // columns of the operand
  const uint32_t ldbytes32 = (uint32_t)ld * (uint32_t)sizeof(T);  // operands stay below 4 GiB (checked on the host)
  // LDS position lane % 32 of row `krow` holds the logical 16-byte piece whose 32-byte group is
  // (position / 2) ^ f(krow), f(krow) = (krow & 3) | (((krow >> 3) & 3) << 2); row pair p of the wave is
  // krow = 8 wq + 2 p + lane / 32, so f only depends on the parity of p
  int lcol[2];  // first column (element) of the lane's piece, for even / odd row pairs
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const int f = ((2 * par + (lane >> 5)) & 3) | (wq << 2);
    lcol[par] = (((((lane & 31) >> 1) ^ f) & 15) << 4) + (lane & 1) * 8;
  }
  const uint32_t lds0 = (uint32_t)(size_t)(MI_LDS void*)smem_raw;
  const uint32_t wave_lds = lds0 + (load_b ? OP_BYTES : 0) + 8 * wq * (TILE * 2);

  // ---- fragment read addresses (per lane): row 8q + 4h + i/4, column group F ^ f(row), piece i % 4 ----------
  const int fi = lane & 15, fq = lane >> 4;
  const int fl = (fi >> 2) | (fq << 2);
  const uint32_t frag_base = (8 * fq + (fi >> 2)) * (TILE * 2) + (fl << 5) + (fi & 3) * 8;

  // Items of an XCD are handed out in order through a counter: the workgroups of the XCD stay on neighbouring
  // items (same group of rows, shared through the L2) and none of them idles while another still has a queue.
  // (instantiated twice: for an operand gathered through an index array and for one read in place)
  auto run_items = [&](auto gather_tag) {
  constexpr bool GATHER = decltype(gather_tag)::value;
  for (;;) {
    if (tid == 0) *item_slot = atomicAdd(a.next_item + xcd, 1);
    __syncthreads();
    const int item = __builtin_amdgcn_readfirstlane(*item_slot);
    __syncthreads();
    if (item >= items_x) break;
    const int grp = __builtin_amdgcn_readfirstlane(xlist[item / tiles]);
    // A group's tiles are numbered in bands of 8 row tiles, column tile slowest inside a band: the 32 workgroups
    // of the XCD, which hold 32 consecutive items, then cover 8 x 4 tiles -- 12 operand slabs for 32 tiles.  (Row
    // tile fastest over all of them would re-read every A slab once per column tile: with 112 x 16 tiles that is
    // 16 passes over the whole A operand.)
    const int tile = item % tiles;
    const int band = tile / (8 * a.n_tiles);
    const int rem = tile - band * 8 * a.n_tiles;
    const int left = a.m_tiles - band * 8;
    const int width = left < 8 ? left : 8;
    const int nt = rem / width;
    const int mt = band * 8 + rem - nt * width;

    // group -> expert and its row range (wave-uniform)
    int r0 = 0, r1 = 1, expert = 0, expert_groups = 1;
    for (int e0 = 0; e0 < a.E; e0 += 64) {
      const int e = e0 + lane;
      const int incl = e < a.E ? etab[2 * e] : 0x7fffffff;
      const uint64_t hit = __ballot(incl > grp);
      if (hit) {
        const int ex = e0 + __ffsll((long long)hit) - 1;
        const int first = ex > 0 ? etab[2 * (ex - 1)] : 0;
        const int prev = ex > 0 ? etab[2 * (ex - 1) + 1] : 0;
        expert = ex;
        expert_groups = etab[2 * ex] - first;
        const int rows = group_rows(etab[2 * ex + 1] - prev, etab[2 * ex] - first);
        r0 = prev + (grp - first) * rows;
        r1 = etab[2 * ex + 1];
        if (r1 > r0 + rows) r1 = r0 + rows;
        break;
      }
    }
    r0 = __builtin_amdgcn_readfirstlane(r0);
    r1 = __builtin_amdgcn_readfirstlane(r1);
    expert = __builtin_amdgcn_readfirstlane(expert);
    expert_groups = __builtin_amdgcn_readfirstlane(expert_groups);
    const int nk = (r1 - r0 + BK - 1) / BK;

    // lane offsets of this tile; columns past the operand's width re-read the tile's first piece (their
    // products only reach output rows / columns that are never stored)
    const int col0 = (load_b ? nt : mt) * TILE;
    uint32_t loff[2];
#pragma unroll
    for (int par = 0; par < 2; ++par) loff[par] = (uint32_t)((col0 + lcol[par] < ld ? lcol[par] : 0) * sizeof(T));
    const unsigned char* tile_src = src + (size_t)col0 * sizeof(T);

    // rows of slice `slice` this wave fetches: sorted rows r0 + 32 slice + 8 wq + [0, 8), clamped into the group
    // (rows past its end are fetched again from its last row and masked out of the last slice's fragments)
    auto load_idx = [&](int slice, int (&rw)[8]) {
      const int first = r0 + slice * BK + 8 * wq;
      if (GATHER && first + 7 < r1) {
        // the usual case: eight consecutive indices in one scalar load
        const i32x8_a4 v = *reinterpret_cast<const_idx8_t>(idx + first);
#pragma unroll
        for (int i = 0; i < 8; ++i) rw[i] = v[i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          int r = first + i;
          if (r > r1 - 1) r = r1 - 1;
          rw[i] = GATHER ? idx[r] : r;
        }
      }
    };
    auto dma_slice = [&](const int (&rw)[8], int stage) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
        wgrad_dma_row_pair(tile_src, (uint32_t)rw[2 * p] * ldbytes32, (uint32_t)rw[2 * p + 1] * ldbytes32, loff[p & 1],
                           0xffffffff00000000ull, wave_lds + stage * STAGE_BYTES + 2 * p * (TILE * 2));
    };

    f32x4 acc[4][8];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int nb = 0; nb < 8; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    s16x8 af[4], bf[8];
    auto read_frag = [&](int stage, int opoff, int F) -> s16x8 {
      const uint32_t addr = lds0 + stage * STAGE_BYTES + opoff + (frag_base ^ ((uint32_t)F << 5));
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MI_LDS s16x4*)(size_t)addr);
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MI_LDS s16x4*)(size_t)(addr + 4 * TILE * 2));
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    auto read_frags = [&](int stage) {
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) af[mb] = read_frag(stage, 0, 4 * wm + mb);
#pragma unroll
      for (int nb = 0; nb < 8; ++nb) bf[nb] = read_frag(stage, OP_BYTES, 8 * wn + nb);
    };
    auto multiply = [&]() {
#pragma unroll
      for (int nb = 0; nb < 8; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb][nb] = WgradMfma<T>::run(af[mb], bf[nb], acc[mb][nb]);
    };
    // the last slice of a group may be short: element j of a fragment is row 8 (lane / 16) + j of the slice
    const int last_rows = r1 - r0 - (nk - 1) * BK;
    auto mask_frags = [&]() {
      uint32_t m[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int k = 8 * fq + 2 * t;
        m[t] = (k < last_rows ? 0x0000ffffu : 0u) | (k + 1 < last_rows ? 0xffff0000u : 0u);
      }
      auto apply = [&](s16x8& v) {
        u32x4 w = __builtin_bit_cast(u32x4, v);
#pragma unroll
        for (int t = 0; t < 4; ++t) w[t] &= m[t];
        v = __builtin_bit_cast(s16x8, w);
      };
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) apply(af[mb]);
#pragma unroll
      for (int nb = 0; nb < 8; ++nb) apply(bf[nb]);
    };

    // ---- K loop: the forward kernel's ping-pong schedule.  The waves wn == 0 and wn == 1 (one of each per SIMD)
    // run the same code one phase apart: while one group issues its 32 matrix instructions out of registers, the
    // other reads its fragments of the slice and issues its share of the DMA for the slice three ahead.
    int rw[8];
    load_idx(0, rw);
    dma_slice(rw, 0);
    load_idx(1, rw);
    dma_slice(rw, 1);
    load_idx(2, rw);
    dma_slice(rw, 2);
    load_idx(3, rw);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(wgrad_waitcnt((AHEAD - 1) * NLD, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (wn == 1) __builtin_amdgcn_s_barrier();
    for (int g = 0; g < nk; ++g) {
      const int cur = g & (NSTAGE - 1), fill = (g + AHEAD) & (NSTAGE - 1);
      // slices past the group's end are fetched like the others (clamped rows) and never multiplied.  The DMA goes
      // first: its row indices came in long ago, and a wait for them behind the fragment reads would also wait
      // for those (scalar loads and LDS reads share a counter)
      dma_slice(rw, fill);
      read_frags(cur);
      if (g == nk - 1 && last_rows < BK) mask_frags();
      asm volatile("" ::: "memory");
      // own DMA of slice g + 1 has landed (g + 2 and g + 3 stay in flight); fragments are in registers
      __builtin_amdgcn_s_waitcnt(wgrad_waitcnt((NSTAGE - 2) * NLD, 0));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      // the row indices of the next DMA come in through the scalar cache while the matrix pipe works
      load_idx(g + 4, rw);
      __builtin_amdgcn_sched_barrier(0);
      multiply();
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    if (wn == 0) __builtin_amdgcn_s_barrier();
    // surplus DMA (slices nk .. nk + 2) must land before the next item reuses the ring
    __builtin_amdgcn_s_waitcnt(wgrad_waitcnt(0, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // ---- output tile: register i of block (mb, nb) is row 16 mb + 4 (lane / 16) + i, column 16 nb + lane % 16.
    // An expert with one group is final: rounded and written straight into dw (whole 32-byte sectors per 16
    // lanes).  Otherwise an fp32 partial tile for the reduction kernel.
    if (expert_groups == 1) {
      T* __restrict__ out = static_cast<T*>(a.dw) + (size_t)expert * a.M * a.N;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int m = mt * TILE + wm * 64 + mb * 16 + 4 * fq + i;
          if (m < a.M) {
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
              const int n = nt * TILE + wn * 128 + nb * 16 + fi;
              if (n < a.N) Elt<T>::store(out + (size_t)m * a.N + n, acc[mb][nb][i]);
            }
          }
        }
    } else {
      float* __restrict__ out = a.partial + (size_t)grp * a.M * a.N;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int m = mt * TILE + wm * 64 + mb * 16 + 4 * fq + i;
          if (m < a.M) {
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
              const int n = nt * TILE + wn * 128 + nb * 16 + fi;
              if (n < a.N) out[(size_t)m * a.N + n] = acc[mb][nb][i];
            }
          }
        }
    }
  }
  };
  if (idx != nullptr) run_items(std::true_type{});
  else run_items(std::false_type{});
}

// Plan of one launch (one workgroup, in front of the main kernel): zero the eight work counters, rank the
// groups by their number of rows (longest first, ties in row order) and deal them to the XCDs back and forth.
//   plan[0..8)   work counters
//   plan[8..17)  first slot of XCD x in the list (slot 8 + 8 = one past the end)
//   plan[17]     number of experts the reduction has to write (those with no group or with several)
//   plan[32..)   group numbers (row order numbering, as the partial slabs and the reduction use) by slot
//   plan[red_at..)  (expert, first group, groups) of each of those experts, in expert order
// Up to WGRAD_PLAN_SORT groups are ranked; beyond that the groups are dealt in row order.
#define WGRAD_PLAN_SORT 8192
__global__ __launch_bounds__(1024) void wgrad_plan_kernel(const int32_t* __restrict__ offsets, int E, int chunk,
                                                          int* __restrict__ plan, int red_at) {
  __shared__ int first[WGRAD_MAX_E + 1];  // groups in front of expert e
  __shared__ int ends[WGRAD_MAX_E];       // the offsets (one round trip to memory for all of them)
  __shared__ int cnt[WGRAD_MAX_E];        // groups of expert e
  __shared__ int rows[WGRAD_PLAN_SORT];
  const int tid = threadIdx.x;
  if (tid < 8) plan[tid] = 0;
  for (int e = tid; e < E; e += blockDim.x) ends[e] = offsets[e];
  __syncthreads();
  // groups of expert e, then every expert adds up the ones in front of it by itself (E <= 256: no scan needed)
  for (int e = tid; e < E; e += blockDim.x) {
    const int n = ends[e] - (e > 0 ? ends[e - 1] : 0);
    cnt[e] = (n + chunk - 1) / chunk;
  }
  __syncthreads();
  for (int e = tid; e <= E; e += blockDim.x) {
    int g = 0, nred = 0;
    for (int i = 0; i < e; ++i) {
      const int c = cnt[i];
      g += c;
      nred += c != 1 ? 1 : 0;
    }
    first[e] = g;
    if (e == E) {
      plan[17] = nred;
    } else if (cnt[e] != 1) {  // not written by the main kernel
      plan[red_at + 3 * nred] = e;
      plan[red_at + 3 * nred + 1] = g;
      plan[red_at + 3 * nred + 2] = cnt[e];
    }
  }
  __syncthreads();
  const int G = first[E];
  const bool sorted = G <= WGRAD_PLAN_SORT;
  if (sorted) {
    // rows of every group: group i of an expert with n rows in `groups` groups of `per` rows each
    for (int e = tid; e < E; e += blockDim.x) {
      const int n = ends[e] - (e > 0 ? ends[e - 1] : 0);
      const int groups = first[e + 1] - first[e];
      if (groups == 0) continue;
      const int per = ((n + groups - 1) / groups + 31) & ~31;
      for (int i = 0; i < groups; ++i) {
        const int r1 = (i + 1) * per < n ? (i + 1) * per : n;
        rows[first[e] + i] = r1 - i * per;
      }
    }
  }
  __syncthreads();
  // XCD x gets the ranks 16 j + x and 16 j + 15 - x: G / 8 full rounds and part of one more
  const int full = G >> 3, rem = G & 7;
  if (tid < 9) {
    int start = 0;
    for (int x = 0; x < tid; ++x) start += full + (((full & 1) == 0 ? x < rem : x >= 8 - rem) ? 1 : 0);
    plan[8 + tid] = start;
  }
  for (int g = tid; g < G; g += blockDim.x) {
    int rank = g;
    if (sorted) {
      const int mine = rows[g];
      rank = 0;
      for (int o = 0; o < G; ++o) {
        const int r = rows[o];
        rank += (r > mine || (r == mine && o < g)) ? 1 : 0;
      }
    }
    const int round = rank >> 3, pos = rank & 7;
    const int x = (round & 1) == 0 ? pos : 7 - pos;
    int start = 0;
    for (int y = 0; y < x; ++y) start += full + (((full & 1) == 0 ? y < rem : y >= 8 - rem) ? 1 : 0);
    plan[32 + start + round] = g;
  }
}

// dW[e] = sum of expert e's partial slabs in group order, rounded once (experts with several groups); zeros for an
// expert without rows.  blockIdx.y walks the plan's list of such experts (without a plan -- a call with no rows at
// all -- every expert gets zeros); the blocks of an entry stride over the expert's 8-value chunks, four slabs'
// loads in flight per chunk.
template <typename T>
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ partial,
                                                           const int* __restrict__ plan, int red_at,
                                                           T* __restrict__ dw, long mn) {
  int e = blockIdx.y, first = 0, count = 0;
  if (plan != nullptr) {
    if ((int)blockIdx.y >= plan[17]) return;
    const int* entry = plan + red_at + 3 * blockIdx.y;
    e = entry[0];
    first = entry[1];
    count = entry[2];
  }
  const long n8 = mn / 8;
  const float* base = partial + (size_t)first * mn;
  T* out = dw + (size_t)e * mn;
  for (long id = (long)blockIdx.x * 256 + threadIdx.x; id < n8; id += (long)gridDim.x * 256) {
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    const float* p = base + id * 8;
    int g = 0;
    for (; g + 4 <= count; g += 4) {
      f32x4 v[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + (size_t)(g + j) * mn));
        v[2 * j + 1] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + (size_t)(g + j) * mn + 4));
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s0 += v[2 * j];
        s1 += v[2 * j + 1];
      }
    }
    for (; g < count; ++g) {
      s0 += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + (size_t)g * mn));
      s1 += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + (size_t)g * mn + 4));
    }
    u32x4 o;
    o[0] = pack2<T>(s0[0], s0[1]);
    o[1] = pack2<T>(s0[2], s0[3]);
    o[2] = pack2<T>(s1[0], s1[1]);
    o[3] = pack2<T>(s1[2], s1[3]);
    *reinterpret_cast<u32x4*>(out + id * 8) = o;
  }
}

// Rows per group: between 256 and 16384, a multiple of 32, and few enough groups that the fp32 partial tiles of
// the experts with several groups stay cheap: about 384 items (1.5 per CU) before the cap.  Measured on the
// Granite-3B-A800M shapes (262144 rows, 40 experts): every megabyte of partial tiles costs about as much as
// 0.07 % of the products, so long groups beat groups of 3040 - 6080 rows (about four items per CU) by 4 - 7 %
// under skewed loads and by 12 - 18 % under an even load (where no expert is split any more); the longest-first
// plan keeps the few long items balanced.
static int wgrad_chunk(int L, int E, int M, int N) {
  const long tiles = (long)mi_ceil_div(M, 256) * mi_ceil_div(N, 256);
  long groups = (384 + tiles - 1) / tiles;
  long chunk = L / (groups > 0 ? groups : 1);
  // With at least one item per CU from whole experts alone, an expert is only cut when it is half again as long as
  // the average one: under an even load nobody is (no partial tiles, no second pass over them); the long experts of
  // a skewed load still are.
  if ((long)E * tiles >= 256 && chunk < 3L * (L / E) / 2) chunk = 3L * (L / E) / 2;
  if (chunk > 16384) chunk = 16384;
  if (chunk < 256) chunk = 256;
  return (int)(chunk / 32 * 32);
}

static long wgrad_max_groups(int L, int E, int chunk) { return (long)L / chunk + (E < L ? E : L); }
static size_t wgrad_plan_bytes(long groups, int E) { return ((size_t)(32 + groups + 3 * (long)E) * sizeof(int) + 255) / 256 * 256; }

extern "C" size_t mi_moe_grouped_wgrad_workspace_bytes(int L, int E, int M, int N) {
  if (L < 1 || E < 1 || M < 1 || N < 1) return 0;
  // [partial slabs][plan: 32 ints (work counters, first slots) + one int per group + three per expert, padded to
  // 256 bytes]
  const long groups = wgrad_max_groups(L, E, wgrad_chunk(L, E, M, N));
  return (size_t)groups * (size_t)M * (size_t)N * sizeof(float) + wgrad_plan_bytes(groups, E);
}

extern "C" int mi_moe_grouped_wgrad(const void* a, const int32_t* a_idx, const void* b, const int32_t* b_idx,
                                    const int32_t* expert_offsets, void* dw, void* workspace, size_t workspace_bytes,
                                    int L, int a_rows, int b_rows, int M, int N, int E, int dtype, mi_moe_stream_t stream) {
  if (L < 0 || M < 1 || N < 1 || E < 1) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (M % 8 != 0 || N % 8 != 0 || E > WGRAD_MAX_E) return MI_MOE_EUNSUPPORTED;
  if (a_rows < 0 || b_rows < 0) return MI_MOE_ESHAPE;
  // rows are addressed with 32-bit byte offsets
  if ((uint64_t)a_rows * M * 2 >= (1ull << 32) || (uint64_t)b_rows * N * 2 >= (1ull << 32)) return MI_MOE_EUNSUPPORTED;
  if (!dw || !expert_offsets) return MI_MOE_ENULL;
  if (L > 0 && (!a || !b)) return MI_MOE_ENULL;
  if (!mi_aligned(a, 16) || !mi_aligned(b, 16) || !mi_aligned(dw, 16) || !mi_aligned(workspace, 16)) return MI_MOE_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long mn = (long)M * N;
  if (L > 0 && (!workspace || workspace_bytes < mi_moe_grouped_wgrad_workspace_bytes(L, E, M, N))) return MI_MOE_EWORKSPACE;

  WgradArgs g;
  g.a = a; g.b = b; g.a_idx = a_idx; g.b_idx = b_idx; g.expert_offsets = expert_offsets;
  g.partial = static_cast<float*>(workspace);
  g.dw = dw;
  g.next_item = nullptr;
  g.L = L; g.M = M; g.N = N; g.E = E;
  g.chunk = wgrad_chunk(L, E, M, N);
  const long max_groups = wgrad_max_groups(L, E, g.chunk);
  const int red_at = (int)(32 + max_groups);
  if (L > 0) {
    g.next_item = reinterpret_cast<int*>(static_cast<unsigned char*>(workspace) +
                                         (size_t)max_groups * (size_t)M * (size_t)N * sizeof(float));
    hipLaunchKernelGGL(wgrad_plan_kernel, dim3(1), dim3(1024), 0, s, expert_offsets, E, g.chunk, g.next_item, red_at);
  }
  g.m_tiles = mi_ceil_div(M, 256);
  g.n_tiles = mi_ceil_div(N, 256);
  const size_t lds = 4 * 2 * 32 * 256 * 2 + (size_t)E * 8 + 16;
  int cus = 0;
  int rc = mi_cu_count(&cus);
  if (rc != MI_MOE_OK) return rc;
  const long max_items = max_groups * g.m_tiles * g.n_tiles;
  long grid = cus < max_items ? cus : max_items;
  grid = (grid + 7) / 8 * 8;
  long rblocks = (mn / 8 + 255) / 256;
  if (rblocks > 256) rblocks = 256;
  if (dtype == MI_MOE_BF16) {
    auto kern = grouped_wgrad_kernel<bf16_t>;
    static std::atomic<uint64_t> lds_ok{0};
    if ((rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), MI_LDS_MAX_BYTES, lds_ok)) != MI_MOE_OK) return rc;
    if (L > 0) hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, s, g);
    hipLaunchKernelGGL((wgrad_reduce_kernel<bf16_t>), dim3((unsigned)rblocks, (unsigned)E), dim3(256), 0, s, g.partial,
                       g.next_item, red_at, static_cast<bf16_t*>(dw), mn);
  } else {
    auto kern = grouped_wgrad_kernel<f16_t>;
    static std::atomic<uint64_t> lds_ok{0};
    if ((rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), MI_LDS_MAX_BYTES, lds_ok)) != MI_MOE_OK) return rc;
    if (L > 0) hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, s, g);
    hipLaunchKernelGGL((wgrad_reduce_kernel<f16_t>), dim3((unsigned)rblocks, (unsigned)E), dim3(256), 0, s, g.partial,
                       g.next_item, red_at, static_cast<f16_t*>(dw), mn);
  }
  return mi_launch_status();
}

// ---- fp32 weight gradient on the matrix cores ----------------------------------------------------------------
// One workgroup per (expert, 128 x 128 tile of dW) walks the expert's rows 16 at a time: both operand slices go
// global -> registers -> LDS exactly as they lie in memory ([row][column], the loads of the next slice in flight
// while this one is multiplied), and the fragments of v_mfma_f32_32x32x2f32 are single floats -- lane l supplies
// a[row 2 j + l / 32][column l % 32] and the same element of b -- so no transposing read is needed: 32 lanes read
// 32 consecutive floats of one slice row.  The row pitch of 160 floats puts the two half waves (rows 2 j and
// 2 j + 1) on different halves of the 64 banks.  The rows are added in ascending order by one workgroup:
// deterministic, no workspace; experts without rows get zeros.  M % 4 == N % 4 == 0.
#define WGRAD_F32_TILE 128
#define WGRAD_F32_ROWS 16
#define WGRAD_F32_PITCH 160
__global__ __launch_bounds__(256) void grouped_wgrad_f32_kernel(const float* __restrict__ a,
                                                                const int32_t* __restrict__ a_idx,
                                                                const float* __restrict__ b,
                                                                const int32_t* __restrict__ b_idx,
                                                                const int32_t* __restrict__ offsets,
                                                                float* __restrict__ dw, int M, int N) {
  constexpr int TILE = WGRAD_F32_TILE, RS = WGRAD_F32_ROWS, PITCH = WGRAD_F32_PITCH;
  __shared__ __attribute__((aligned(16))) float sa[2][RS * PITCH];
  __shared__ __attribute__((aligned(16))) float sb[2][RS * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int e = blockIdx.z;
  const int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
  const int begin = e > 0 ? offsets[e - 1] : 0, end = offsets[e];
  const int nslices = (end - begin + RS - 1) / RS;

  // staging: thread t takes the float4 at column 4 (t % 32) of the slice rows t / 32 and t / 32 + 8, of both operands
  const int lrow = tid >> 5, lcol = (tid & 31) * 4;
  f32x4 ra[2], rb[2];
  auto load_slice = [&](int sl) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r = begin + sl * RS + lrow + 8 * j;
      ra[j] = rb[j] = (f32x4){0.f, 0.f, 0.f, 0.f};  // rows past the expert's end and columns past the edge add nothing
      if (r < end) {
        const size_t ar = a_idx ? (size_t)a_idx[r] : (size_t)r;
        const size_t br = b_idx ? (size_t)b_idx[r] : (size_t)r;
        if (m0 + lcol < M) ra[j] = *reinterpret_cast<const f32x4*>(a + ar * M + m0 + lcol);
        if (n0 + lcol < N) rb[j] = *reinterpret_cast<const f32x4*>(b + br * N + n0 + lcol);
      }
    }
  };
  auto store_slice = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      *reinterpret_cast<f32x4*>(&sa[buf][(lrow + 8 * j) * PITCH + lcol]) = ra[j];
      *reinterpret_cast<f32x4*>(&sb[buf][(lrow + 8 * j) * PITCH + lcol]) = rb[j];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;

  const int fcol = lane & 31, fk = lane >> 5;
  if (nslices > 0) {
    load_slice(0);
    store_slice(0);
  }
  __syncthreads();
  for (int sl = 0; sl < nslices; ++sl) {
    const int buf = sl & 1;
    if (sl + 1 < nslices) load_slice(sl + 1);
#pragma unroll
    for (int j = 0; j < RS / 2; ++j) {
      const float* pa = &sa[buf][(2 * j + fk) * PITCH + wm * 64 + fcol];
      const float* pb = &sb[buf][(2 * j + fk) * PITCH + wn * 64 + fcol];
      const float af[2] = {pa[0], pa[32]}, bf[2] = {pb[0], pb[32]};
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[mb], bf[nb], acc[mb][nb], 0, 0, 0);
    }
    if (sl + 1 < nslices) store_slice(buf ^ 1);
    __syncthreads();
  }
  // register i of lane l: row 8 (i / 4) + 4 (l / 32) + i % 4 of the block (the a operand's index), column l % 32
  float* __restrict__ out = dw + (size_t)e * M * N;
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int n = n0 + wn * 64 + nb * 32 + fcol;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wm * 64 + mb * 32 + 8 * (i / 4) + 4 * fk + (i % 4);
        if (m < M && n < N) out[(size_t)m * N + n] = acc[mb][nb][i];
      }
    }
}

extern "C" int mi_moe_grouped_wgrad_f32(const float* a, const int32_t* a_idx, const float* b, const int32_t* b_idx,
                                        const int32_t* expert_offsets, float* dw, int L, int M, int N, int E,
                                        mi_moe_stream_t stream) {
  if (L < 0 || M < 1 || N < 1 || E < 1 || E > 65535) return MI_MOE_ESHAPE;
  if (M % 4 != 0 || N % 4 != 0) return MI_MOE_EUNSUPPORTED;
  if (!dw || !expert_offsets) return MI_MOE_ENULL;
  if (L > 0 && (!a || !b)) return MI_MOE_ENULL;
  if (!mi_aligned(a, 16) || !mi_aligned(b, 16)) return MI_MOE_EALIGN;
  const dim3 grid(mi_ceil_div(N, WGRAD_F32_TILE), mi_ceil_div(M, WGRAD_F32_TILE), E);
  if (grid.y > 65535u) return MI_MOE_ESHAPE;
  hipLaunchKernelGGL(grouped_wgrad_f32_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a, a_idx, b, b_idx,
                     expert_offsets, dw, M, N);
  return mi_launch_status();
}

// ---- any-shape / any-dtype weight gradient (one thread per element of dW) ------------------------------------
// For fp32 and for shapes the matrix-core kernel above does not take.  Every element sums its expert's rows in
// ascending order in fp32 (deterministic) and is rounded once.  Correct, not fast; no workspace, no host round trip.
template <typename T>
__global__ __launch_bounds__(256) void grouped_wgrad_naive_kernel(const T* __restrict__ a, const int32_t* __restrict__ a_idx,
                                                                  const T* __restrict__ b, const int32_t* __restrict__ b_idx,
                                                                  const int32_t* __restrict__ offsets, T* __restrict__ dw,
                                                                  int M, int N) {
  const int e = blockIdx.z;
  const int n = blockIdx.x * 64 + (threadIdx.x & 63);
  const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (m >= M || n >= N) return;
  const int begin = e > 0 ? offsets[e - 1] : 0, end = offsets[e];
  float acc = 0.f;
  for (int r = begin; r < end; ++r) {
    const size_t ar = a_idx ? (size_t)a_idx[r] : (size_t)r;
    const size_t br = b_idx ? (size_t)b_idx[r] : (size_t)r;
    acc = fmaf(Elt<T>::load(a + ar * M + m), Elt<T>::load(b + br * N + n), acc);
  }
  Elt<T>::store(dw + ((size_t)e * M + m) * N + n, acc);
}

extern "C" int mi_moe_grouped_wgrad_naive(const void* a, const int32_t* a_idx, const void* b, const int32_t* b_idx,
                                          const int32_t* expert_offsets, void* dw, int L, int M, int N, int E, int dtype,
                                          mi_moe_stream_t stream) {
  if (L < 0 || M < 1 || N < 1 || E < 1 || E > 65535) return MI_MOE_ESHAPE;
  if (dtype != MI_MOE_F32 && dtype != MI_MOE_BF16 && dtype != MI_MOE_F16) return MI_MOE_EDTYPE;
  if (!dw || !expert_offsets) return MI_MOE_ENULL;
  if (L > 0 && (!a || !b)) return MI_MOE_ENULL;
  const dim3 grid(mi_ceil_div(N, 64), mi_ceil_div(M, 4), E);
  if (grid.y > 65535u) return MI_MOE_ESHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI_MOE_F32:
      hipLaunchKernelGGL((grouped_wgrad_naive_kernel<float>), grid, dim3(256), 0, s, static_cast<const float*>(a), a_idx,
                         static_cast<const float*>(b), b_idx, expert_offsets, static_cast<float*>(dw), M, N);
      break;
    case MI_MOE_F16:
      hipLaunchKernelGGL((grouped_wgrad_naive_kernel<f16_t>), grid, dim3(256), 0, s, static_cast<const f16_t*>(a), a_idx,
                         static_cast<const f16_t*>(b), b_idx, expert_offsets, static_cast<f16_t*>(dw), M, N);
      break;
    default:
      hipLaunchKernelGGL((grouped_wgrad_naive_kernel<bf16_t>), grid, dim3(256), 0, s, static_cast<const bf16_t*>(a), a_idx,
                         static_cast<const bf16_t*>(b), b_idx, expert_offsets, static_cast<bf16_t*>(dw), M, N);
  }
  return mi_launch_status();
}
