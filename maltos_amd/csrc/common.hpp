// Shared device/host helpers for the gfx950 kernels: vector types, bf16 conversion, wavefront
// (64-lane) reductions and the thread-local error string behind mlts_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include <mutex>

#include "../../include/maltos_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define MLTS_WAVE 64

void mlts_set_error(const char* fmt, ...);
int mlts_check_launch(const char* what);

// Optional per-kernel timing (mlts_kernel_timing_enable): brackets a launch with HIP events on the
// launch stream.  Disabled by default; then the constructor and destructor are a single branch.
struct MltsKernelTimer {
  MltsKernelTimer(const char* name, hipStream_t stream);
  ~MltsKernelTimer();
  const char* name_;
  hipStream_t stream_;
  hipEvent_t start_;
  bool active_;
};

// One-time opt-in of a kernel to more than 48 KiB of dynamic LDS; safe when several host threads make their first launch
// of that kernel at once.  One instance per kernel instantiation (a function-local static).
struct MltsLdsOptIn {
  std::once_flag once;
  hipError_t err = hipSuccess;
  hipError_t reserve(const void* kernel, int bytes) {
    std::call_once(once, [&] { err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes); });
    return err;
  }
};

#define MLTS_REQUIRE(cond, ...)        \
  do {                                 \
    if (!(cond)) {                     \
      mlts_set_error(__VA_ARGS__);     \
      return MLTS_ERR_INVALID;         \
    }                                  \
  } while (0)

static inline bool mlts_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- element conversion -------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_f32(T x);
template <>
__device__ __forceinline__ float to_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ float to_f32<bf16_t>(bf16_t x) {
  return static_cast<float>(x);
}
template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
  return static_cast<bf16_t>(x);  // round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
}
// Round through T and come back to fp32: reproduces an eager op that materialises its result in T.
template <typename T>
__device__ __forceinline__ float round_to(float x) {
  return to_f32<T>(from_f32<T>(x));
}

// 16-byte vector of T
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  f32x4 v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, float x) { v[i] = x; }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  bf16x8 v;
  __device__ __forceinline__ float get(int i) const { return static_cast<float>(v[i]); }
  __device__ __forceinline__ void set(int i, float x) { v[i] = static_cast<bf16_t>(x); }
};

// ---- wavefront reductions (64 lanes) ------------------------------------------------------
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, MLTS_WAVE);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, MLTS_WAVE));
  return x;
}
__device__ __forceinline__ double wave_sum_f64(double x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, MLTS_WAVE);
  return x;
}
