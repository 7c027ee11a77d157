// Diagnostic kernels: the pieces of the persistent grouped GEMM's inner loop (grouped_gemm.hip) run in isolation,
// so that a benchmark can put a measured ceiling next to the GEMM's own figure on the same GPU in the same process.
// Nothing in the layer calls these; they compute nothing useful.
//
// One workgroup of eight waves per compute unit works through `slices` K slices of a 256 x 256 bf16 tile exactly
// as the GEMM does (32-wide slices, wave tile 64 x 128, twelve 16-byte fragment reads and 32 v_mfma_f32_16x16x32 per
// wave and slice, four 1 KiB DMA instructions per wave and slice into a ring of four 32 KiB stages), with parts
// switched off:
//   mode 0   matrix instructions only (operands read once): what the matrix cores sustain on this data at the
//            clock the chip settles at
//   mode 1   + the LDS fragment reads of every slice (no DMA: the ring keeps its first contents)
//   mode 2   DMA only: L2 -> LDS fill rate of one workgroup per CU (addresses walk an L2-resident span)
//   mode 3   everything, in the GEMM's two-group ping-pong schedule
// `data` supplies the bytes (the caller chooses them: random bf16 values draw more power than zeros and lower the
// clock).  flops per slice and workgroup: 2 * 256 * 256 * 32; DMA bytes per slice and workgroup: 32 KiB.
#include "common.h"

typedef __attribute__((address_space(3))) void* probe_lds_ptr_t;

__device__ __forceinline__ constexpr int probe_waitcnt(int vm, int lgkm) {
  return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}

template <int MODE>
__global__ __launch_bounds__(512) void probe_kloop_kernel(const unsigned char* __restrict__ data, uint32_t span,
                                                          int slices, float* __restrict__ sink) {
  constexpr int STAGE = 32768, NSTAGE = 4, NLD = 4, MB = 4, NB = 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 3, wn = wave >> 2;
  const uint32_t lds0 = (uint32_t)(size_t)(probe_lds_ptr_t)smem;

  // DMA sources: instruction j of this wave fills stage rows (j * 8 + wave) * 16 .. + 16, lane -> row lane / 4,
  // 16-byte piece lane % 4 of a 64-byte row piece; rows 3072 bytes apart like the rows of a (tokens, 1536) matrix
  uint32_t goff[NLD];
  const uint32_t blk = (uint32_t)(((uint64_t)(blockIdx.x >> 3) * 7919u * 65536u) % span);
#pragma unroll
  for (int j = 0; j < NLD; ++j)
    goff[j] = ((blk + (uint32_t)((j * 8 + wave) * 16 + (lane >> 2)) * 3072u + (uint32_t)(lane & 3) * 16u) % span) & ~15u;
  auto dma_slice = [&](int kt, int stage) {
    const unsigned char* src = data + (size_t)(kt & 15) * 64;
#pragma unroll
    for (int j = 0; j < NLD; ++j)
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                   : : "s"(lds0 + stage * STAGE + (j * 8 + wave) * 1024), "v"(goff[j]), "s"(src) : "memory", "m0");
  };

  // fragment reads as in the GEMM: row lane % 16 of a 16-row block, k chunk lane / 16, slot chunk ^ ((row >> 1) & 3)
  const int frow = lane & 15, fq = lane >> 4;
  const uint32_t chunk = (uint32_t)((fq ^ ((frow >> 1) & 3)) * 16);
  bf16x8 xf[MB], wf[NB];
  auto read_frags = [&](int stage) {
    const unsigned char* s = smem + stage * STAGE + chunk;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[nb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(s + (256 + wn * 128 + nb * 16 + frow) * 64));
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      xf[mb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(s + (wm * 64 + mb * 16 + frow) * 64));
  };
  f32x4 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  auto mfma_step = [&]() {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nb], xf[mb], acc[nb][mb], 0, 0, 0);
  };

  // the ring's first contents
#pragma unroll
  for (int st = 0; st < NSTAGE; ++st) dma_slice(st, st);
  __builtin_amdgcn_s_waitcnt(probe_waitcnt(0, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_frags(0);

  if (MODE == 0) {
    for (int g = 0; g < slices; ++g) {
      mfma_step();
      __builtin_amdgcn_sched_barrier(0);
    }
  } else if (MODE == 1) {
    for (int g = 0; g < slices; ++g) {
      read_frags(g & (NSTAGE - 1));
      asm volatile("" ::: "memory");
      mfma_step();
      __builtin_amdgcn_sched_barrier(0);
    }
  } else if (MODE == 2) {
    for (int g = 0; g < slices; ++g) {
      dma_slice(g, g & (NSTAGE - 1));
      if ((g & 3) == 3) __builtin_amdgcn_s_waitcnt(probe_waitcnt(2 * NLD, 15));  // a few slices stay in flight
    }
  } else {
    // the GEMM's schedule: the wave groups wn = 0 / 1 (one wave of each per SIMD) run one phase apart; while one
    // issues its matrix instructions the other reads its fragments and issues its DMA for the slice three ahead
    if (wn == 1) __builtin_amdgcn_s_barrier();
    for (int g = 0; g < slices; ++g) {
      read_frags(g & (NSTAGE - 1));
      dma_slice(g + 3, (g + 3) & (NSTAGE - 1));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(probe_waitcnt(2 * NLD, 0));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      mfma_step();
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    if (wn == 0) __builtin_amdgcn_s_barrier();
  }
  __builtin_amdgcn_s_waitcnt(probe_waitcnt(0, 0));  // no DMA may outlive the workgroup's LDS
  float r = 0.f;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) r += acc[nb][mb][0] + acc[nb][mb][1] + acc[nb][mb][2] + acc[nb][mb][3];
  if (MODE == 2) r += (float)smem[tid];
  sink[(size_t)blockIdx.x * 512 + tid] = r;
}

extern "C" size_t mi_moe_probe_sink_bytes(void) {
  int cus = 0;
  if (mi_cu_count(&cus) != MI_MOE_OK) return 0;
  return (size_t)cus * 512 * sizeof(float);
}

extern "C" int mi_moe_probe_kloop(int mode, const void* data, size_t data_bytes, int slices, void* sink,
                                  size_t sink_bytes, mi_moe_stream_t stream) {
  if (mode < 0 || mode > 3 || slices < 1) return MI_MOE_ESHAPE;
  // the walk needs a span of at least the 512 rows x 3072 bytes one stage touches, plus the slice offsets
  if (data_bytes < (2u << 20) + 4096 || data_bytes >= (1ull << 32)) return MI_MOE_ESHAPE;
  if (!data || !sink) return MI_MOE_ENULL;
  if (!mi_aligned(data, 16)) return MI_MOE_EALIGN;
  int cus = 0;
  int rc = mi_cu_count(&cus);
  if (rc != MI_MOE_OK) return rc;
  if (sink_bytes < (size_t)cus * 512 * sizeof(float)) return MI_MOE_EWORKSPACE;
  const uint32_t span = (uint32_t)((data_bytes - 4096) & ~(size_t)0xffff);  // room for the slice offsets behind it
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = 4 * 32768;
  const unsigned char* d = static_cast<const unsigned char*>(data);
  float* out = static_cast<float*>(sink);
  static std::atomic<uint64_t> lds_ok[4];
#define PROBE_LAUNCH(M)                                                                                       \
  {                                                                                                           \
    auto kern = probe_kloop_kernel<M>;                                                                        \
    if ((rc = mi_allow_lds_once(reinterpret_cast<const void*>(kern), (int)lds, lds_ok[M])) != MI_MOE_OK) return rc; \
    hipLaunchKernelGGL(kern, dim3(cus), dim3(512), lds, s, d, span, slices, out);                             \
  }
  switch (mode) {
    case 0: PROBE_LAUNCH(0) break;
    case 1: PROBE_LAUNCH(1) break;
    case 2: PROBE_LAUNCH(2) break;
    default: PROBE_LAUNCH(3) break;
  }
#undef PROBE_LAUNCH
  return mi_launch_status();
}
