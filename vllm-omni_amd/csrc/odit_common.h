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

// A number larger than any this function has returned before in this process (never 0, below 2^47): the
// epoch of the ticket words that rel_l1.hip and gemm_bf16.hip keep in caller scratch.
uint64_t next_ticket_epoch();

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
typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));
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
// the same for data that is read once: the load is marked non-temporal, so the lines do not push reusable
// data out of the caches
template <typename T> __device__ __forceinline__ Vec16<T> load16_stream(const T* p) {
  Vec16<T> v;
  *reinterpret_cast<u32x4_nt*>(&v) = __builtin_nontemporal_load(reinterpret_cast<const u32x4_nt*>(p));
  return v;
}
template <typename T> __device__ __forceinline__ void store16(T* p, const Vec16<T>& v) {
  *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(&v);
}

// ---- raw 16-byte register vectors --------------------------------------------------------------
// Rows kept in registers are held as the 16 bytes that were loaded (a native 4 x u32 vector) and
// unpacked element by element where they are used: a bf16 unpack is one shift or one and.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <typename T> __device__ __forceinline__ u32x4 load_raw(const T* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
template <typename T> __device__ __forceinline__ void store_raw(T* p, u32x4 v) {
  *reinterpret_cast<u32x4*>(p) = v;
}

template <typename T> struct Raw;
template <> struct Raw<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ float get(u32x4 v, int j) {
    const uint32_t w = v[j >> 1];
    return __uint_as_float((j & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  // writes elements 2*pair and 2*pair+1
  static __device__ __forceinline__ void set2(u32x4& v, int pair, float lo, float hi) {
    const f32x2 f = {lo, hi};
    v[pair] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
  }
};
template <> struct Raw<f16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ float get(u32x4 v, int j) {
    const uint32_t w = v[j >> 1];
    const uint16_t h = static_cast<uint16_t>((j & 1) ? (w >> 16) : (w & 0xffffu));
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
  }
  static __device__ __forceinline__ void set2(u32x4& v, int pair, float lo, float hi) {
    const f32x2 f = {lo, hi};
    v[pair] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  }
};
template <> struct Raw<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ float get(u32x4 v, int j) { return __uint_as_float(v[j]); }
  static __device__ __forceinline__ void set2(u32x4& v, int pair, float lo, float hi) {
    v[2 * pair] = __float_as_uint(lo);
    v[2 * pair + 1] = __float_as_uint(hi);
  }
};

// ---- wavefront (64 lanes) reductions ------------------------------------------------------------
// Cross-lane adds inside a 16-lane DPP row cost one VALU instruction each (no LDS crossbar trip):
// xor-1 and xor-2 quad permutes, then the half-row and full-row mirrors.
template <int CTRL> __device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
  return v + __int_as_float(moved);
}
// sum over aligned groups of G consecutive lanes, G in {2,4,8,16}; every lane of a group gets the sum
template <int G> __device__ __forceinline__ float row_group_sum(float v) {
  static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16, "group must fit a 16-lane row");
  if (G >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  if (G >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  if (G >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
  if (G >= 16) v = dpp_add<0x140>(v); // row_mirror
  return v;
}
// sum over the whole wavefront, returned in every lane (wave-uniform)
__device__ __forceinline__ float wave_sum(float v) {
  v = row_group_sum<16>(v);
  const int iv = __float_as_int(v);
  return __int_as_float(__builtin_amdgcn_readlane(iv, 0)) + __int_as_float(__builtin_amdgcn_readlane(iv, 16)) +
         __int_as_float(__builtin_amdgcn_readlane(iv, 32)) + __int_as_float(__builtin_amdgcn_readlane(iv, 48));
}
// sum over aligned groups of G consecutive lanes (G power of two <= 64)
template <int G> __device__ __forceinline__ float group_sum(float v) {
  if (G <= 16) return row_group_sum<(G <= 16 ? G : 16)>(v);
  v = row_group_sum<16>(v);
  if (G >= 32) v += __shfl_xor(v, 16, 64);
  if (G >= 64) v += __shfl_xor(v, 32, 64);
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
