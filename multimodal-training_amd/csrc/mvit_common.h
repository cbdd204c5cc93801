// Shared declarations for the MI355X (gfx950) vision-tower kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/mi355_vit.h"

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

#define MVIT_WAVE 64

// Records a formatted message for mvit_last_error() and returns `code`.
int mvit_set_error(int code, const char* fmt, ...);

#define MVIT_REQUIRE(cond, ...)                                   \
  do {                                                            \
    if (!(cond)) return mvit_set_error(MVIT_ERR_ARG, __VA_ARGS__); \
  } while (0)

// Checks the launch of the kernel just enqueued (configuration errors only; no sync).
#define MVIT_CHECK_LAUNCH(name)                                                        \
  do {                                                                                 \
    hipError_t e__ = hipGetLastError();                                                \
    if (e__ != hipSuccess)                                                             \
      return mvit_set_error(MVIT_ERR_LAUNCH, "%s launch: %s", name, hipGetErrorString(e__)); \
  } while (0)

static inline bool mvit_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Per-device host state (function attributes set, compute-unit counts, symbol addresses) is kept in arrays of this
// many slots indexed by the current device's ordinal.
#define MVIT_MAX_DEVICES 64
// Ordinal of the current device, or -1 (with the error recorded) when it cannot be told or has no slot.
static inline int mvit_current_device(const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MVIT_MAX_DEVICES) {
    mvit_set_error(MVIT_ERR_LAUNCH, "%s: hipGetDevice: %s (device %d, %d slots)", who, hipGetErrorString(e), dev, MVIT_MAX_DEVICES);
    return -1;
  }
  return dev;
}

template <typename T>
struct mvit_elem;
template <>
struct mvit_elem<float> {
  static constexpr int vec = 4;  // elements per 16-byte vector
};
template <>
struct mvit_elem<bf16_t> {
  static constexpr int vec = 8;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) {
  return (bf16_t)v;  // round-to-nearest-even
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
