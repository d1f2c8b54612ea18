// Shared device/host helpers for the gfx950 kernels of libomni_dit_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/omni_dit.h"

namespace odit {

// ---- error reporting (thread-local string behind odit_last_error) ----------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define ODIT_CHECK_ARG(cond, ...)   \
  do {                              \
    if (!(cond)) {                  \
      ::odit::set_error(__VA_ARGS__); \
      return ODIT_EINVAL;           \
    }                               \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return ODIT_ELAUNCH;
  }
  return ODIT_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- element types -----------------------------------------------------------------------------
// Storage structs are raw bit containers; all arithmetic goes through float.
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(bf16_t x) {
  return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}
__device__ __forceinline__ float to_float(f16_t x) { return static_cast<float>(x.v); }
__device__ __forceinline__ float to_float(float x) { return x; }

// round-to-nearest-even fp32 -> bf16, NaN kept quiet (same rule torch uses); gfx950 has the
// conversion in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  bf16_t r; r.bits = f32_to_bf16_bits(f); return r;
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) {
  f16_t r; r.v = static_cast<_Float16>(f); return r;
}
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }

// value of f after one rounding to T
template <typename T> __device__ __forceinline__ float round_to(float f) {
  return to_float(from_float<T>(f));
}

// ---- 16-byte vectors ---------------------------------------------------------------------------
template <typename T> struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  T e[N];
};
template <typename T> __device__ __forceinline__ Vec16<T> load16(const T* p) {
  static_assert(sizeof(Vec16<T>) == 16, "Vec16 must be 16 bytes");
  Vec16<T> v;
  *reinterpret_cast<uint4*>(&v) = *reinterpret_cast<const uint4*>(p);
  return v;
}
template <typename T> __device__ __forceinline__ void store16(T* p, const Vec16<T>& v) {
  *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(&v);
}

// ---- wavefront (64 lanes) reductions ------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
// sum over aligned groups of G consecutive lanes (G power of two <= 64)
template <int G> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// dispatch a callable templated on the element type
#define ODIT_DISPATCH_DTYPE(dtype, T, ...)                 \
  switch (dtype) {                                         \
    case ODIT_BF16: { using T = ::odit::bf16_t; __VA_ARGS__; } break; \
    case ODIT_F16:  { using T = ::odit::f16_t;  __VA_ARGS__; } break; \
    case ODIT_F32:  { using T = float;          __VA_ARGS__; } break; \
    default: ::odit::set_error("unknown dtype code %d", dtype); return ODIT_EINVAL; \
  }

}  // namespace odit
