// Shared device/host helpers for the gfx950 scattered-MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi_moe.h"

#define MI_WAVE 64

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- element conversions (round-to-nearest-even, like torch's casts) -------------------------

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// fp32 -> bf16, round to nearest even, NaN stays NaN: one v_cvt_pk_bf16_f32 (two elements per instruction)
typedef __bf16 mi_bf16x2 __attribute__((ext_vector_type(2)));
typedef float mi_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}

template <typename T> struct Elt;
template <> struct Elt<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Elt<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) {
    return bf16_bits_to_float(*reinterpret_cast<const uint16_t*>(p));
  }
  static __device__ __forceinline__ void store(bf16_t* p, float v) {
    *reinterpret_cast<uint16_t*>(p) = float_to_bf16_bits(v);
  }
  static __device__ __forceinline__ float round(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }
};
template <> struct Elt<f16_t> {
  static __device__ __forceinline__ float load(const f16_t* p) { return (float)(*p); }
  static __device__ __forceinline__ void store(f16_t* p, float v) { *p = (f16_t)v; }
  static __device__ __forceinline__ float round(float v) { return (float)((f16_t)v); }
};

// pack two floats into two 16-bit elements of type T (low half = a)
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  const mi_f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, mi_bf16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  f16_t ha = (f16_t)a, hb = (f16_t)b;
  return (uint32_t)(*reinterpret_cast<uint16_t*>(&ha)) | ((uint32_t)(*reinterpret_cast<uint16_t*>(&hb)) << 16);
}

template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t v);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t v);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t v) { return __uint_as_float(v << 16); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t v) {
  uint16_t h = (uint16_t)(v & 0xffffu);
  return (float)(*reinterpret_cast<f16_t*>(&h));
}
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t v) {
  uint16_t h = (uint16_t)(v >> 16);
  return (float)(*reinterpret_cast<f16_t*>(&h));
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

// ---- host helpers ---------------------------------------------------------------------------

static inline int mi_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? MI_MOE_OK : (int)e;
}

// ---- per-device values that are read once and only read back afterwards ----------------------------------
// The launch paths need the number of compute units and, per kernel, a one-time opt-in to more than 64 KiB of
// dynamic LDS.  Both are properties of (device, kernel) that never change, so they are asked once per device and
// cached: a launch then costs hipGetDevice (thread-local) plus the launch itself.

#include <atomic>

#define MI_MAX_DEVICES 64

// number of compute units of the current device; *dev_out (optional) receives the device index
static inline int mi_cu_count(int* cus, int* dev_out = nullptr) {
  static std::atomic<int> cache[MI_MAX_DEVICES];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev_out) *dev_out = dev;
  int c = (dev >= 0 && dev < MI_MAX_DEVICES) ? cache[dev].load(std::memory_order_relaxed) : 0;
  if (c == 0) {
    e = hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0 && dev < MI_MAX_DEVICES) cache[dev].store(c, std::memory_order_relaxed);
  }
  *cus = c;
  return MI_MOE_OK;
}

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per (kernel, device).  `done` is a per-kernel bit mask of the
// devices already set up (callers keep one static mask per kernel instantiation).  The value asked for is the
// kernel's upper bound, so a later launch with less LDS needs no second call.
static inline int mi_allow_lds_once(const void* kern, int max_lds_bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  const uint64_t bit = (dev >= 0 && dev < 64) ? (1ull << dev) : 0ull;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return MI_MOE_OK;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, max_lds_bytes);
  if (e != hipSuccess) return (int)e;
  if (bit) done.fetch_or(bit, std::memory_order_release);
  return MI_MOE_OK;
}

#define MI_LDS_MAX_BYTES (160 * 1024)

static inline bool mi_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

static inline int mi_ceil_div(int a, int b) { return (a + b - 1) / b; }
__device__ __forceinline__ int mi_ceil_div_dev(int a, int b) { return (a + b - 1) / b; }
