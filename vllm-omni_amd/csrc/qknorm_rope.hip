// K2: fused QK-RMSNorm + rotary embedding + scatter of q/k/v into the joint [txt;img] buffers.
//
// The q, k and v rows of a token (H*D elements each, usually three adjacent slices of one fused-QKV
// GEMM output row) are each read once with 16-byte loads and written once into row
// (out_seq_offset + s) of the dense joint buffers, so the three torch.cat copies of the reference
// never happen. Algorithmic traffic: 2 * 3 * B*S*H*D * sizeof(T) (+ S*rot*4 bytes of cos/sin and the
// norm weights, cache-resident across heads and batch).
//
// Per-head statistics (and no statistics): one 16-byte vector per lane, a flat one-shot grid over
// all vectors of one part (grid.y = q | k | v). A head row is D/EPV consecutive lanes, so its mean
// square is a DPP reduction inside a 16-lane row (one shuffle more for 32 lanes); the kernel uses
// ~40 registers, so a CU keeps many loads in flight. Whole-row statistics (Wan): one wavefront per
// (token, part) holding the row in registers, reduced across the wavefront.
// Interleaved rotary pairs (2i, 2i+1) live inside one lane's vector; NeoX pairs are fetched from the
// lane rot/(2*EPV) away with a shuffle.
#include <type_traits>

#include "odit_common.h"

namespace odit {

template <int N> __device__ __forceinline__ void load_floats(const float* p, float (&dst)[N]) {
  if constexpr (N == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    dst[0] = t.x; dst[1] = t.y; dst[2] = t.z; dst[3] = t.w;
  } else if constexpr (N == 2) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    dst[0] = t.x; dst[1] = t.y;
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) dst[j] = p[j];
  }
}

// Weight multiply + rotation of ONE 16-byte vector x (already unpacked to float) that starts at
// offset d0 of its head. `wp` points at the weights of this vector (or is null), `rstd` is the
// reciprocal RMS that applies to it. GENERAL = false compiles the hot variant only (interleaved pairs,
// one final rounding); GENERAL = true takes NeoX pairing and reference rounding as wave-uniform
// run-time switches. Must be called by all lanes of the wavefront (the NeoX path shuffles).
template <typename T, typename TW, bool NORM, bool HEAD_ROUNDING, bool GENERAL>
__device__ __forceinline__ void transform_vec(float (&x)[Vec16<T>::N], float rstd, const TW* wp,
                                              const float* cos_row, const float* sin_row, int d0,
                                              int rot, bool valid, int lane, bool neox_rt,
                                              bool ref_round_rt) {
  constexpr int EPV = Vec16<T>::N;
  const bool NEOX = GENERAL && neox_rt;
  const bool REF_ROUND = GENERAL && ref_round_rt;
  if constexpr (NORM) {
    float wv[EPV];
    if (wp != nullptr && valid) {
      constexpr int EW = Vec16<TW>::N;
#pragma unroll
      for (int q = 0; q < EPV / EW; ++q) {
        const Vec16<TW> t = load16(wp + q * EW);
#pragma unroll
        for (int j = 0; j < EW; ++j) wv[q * EW + j] = to_float(t.e[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < EPV; ++j) wv[j] = 1.f;
    }
#pragma unroll
    for (int j = 0; j < EPV; ++j) {
      if (REF_ROUND && HEAD_ROUNDING) {
        x[j] = round_to<T>(round_to<T>(x[j] * rstd) * wv[j]);  // vLLM RMSNorm: cast, then weight
      } else {
        x[j] = x[j] * rstd * wv[j];
        if (REF_ROUND) x[j] = round_to<T>(x[j]);
      }
    }
  }
  if (cos_row == nullptr) return;
  if (!NEOX) {
    if (d0 < rot && valid) {
      float c[EPV / 2], s[EPV / 2];
      load_floats<EPV / 2>(cos_row + (d0 >> 1), c);
      load_floats<EPV / 2>(sin_row + (d0 >> 1), s);
#pragma unroll
      for (int j = 0; j < EPV / 2; ++j) {
        const float x0 = x[2 * j], x1 = x[2 * j + 1];
        if (REF_ROUND) {
          const float cc = round_to<T>(c[j]), ss = round_to<T>(s[j]);
          x[2 * j] = round_to<T>(x0 * cc) - round_to<T>(x1 * ss);
          x[2 * j + 1] = round_to<T>(x1 * cc) + round_to<T>(x0 * ss);
        } else {
          x[2 * j] = x0 * c[j] - x1 * s[j];
          x[2 * j + 1] = x1 * c[j] + x0 * s[j];
        }
      }
    }
  } else {
    // pair (d, d + rot/2): the partner vector sits rot/(2*EPV) lanes away inside the same head row
    const int half = rot >> 1;
    const int dist = half / EPV;
    const bool lower = d0 < half;
    const int src = lower ? lane + dist : lane - dist;
    float px[EPV];
#pragma unroll
    for (int j = 0; j < EPV; ++j) px[j] = __shfl(x[j], src & 63, 64);
    if (d0 < rot && valid) {
      const int t0 = lower ? d0 : d0 - half;
      const float sgn = lower ? -1.f : 1.f;
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        const float cj = cos_row[t0 + j], sj = sin_row[t0 + j];
        if (REF_ROUND) {
          x[j] = round_to<T>(x[j] * round_to<T>(cj)) + round_to<T>(sgn * px[j] * round_to<T>(sj));
        } else {
          x[j] = x[j] * cj + sgn * px[j] * sj;
        }
      }
    }
  }
}

template <typename T> __device__ __forceinline__ u32x4 pack_vec(const float (&x)[Vec16<T>::N]) {
  u32x4 o;
#pragma unroll
  for (int j = 0; j < Vec16<T>::N / 2; ++j) Raw<T>::set2(o, j, x[2 * j], x[2 * j + 1]);
  return o;
}

// Division of n < 2^31 by a launch constant d as one multiply-high and a shift: with l = ceil(log2 d) >= 1
// and mul = ceil(2^(31+l) / d) < 2^32, floor(n * mul / 2^(31+l)) = floor(n / d) exactly (the excess
// n * (mul - 2^(31+l)/d) / 2^(31+l) stays below 2^-l <= 1/d). d = 1 is the identity (mul = 0 marks it).
struct FastDiv {
  uint32_t mul, shift;
  static FastDiv make(uint32_t d) {
    if (d <= 1) return {0u, 0u};
    uint32_t l = 1;
    while ((1ull << l) < d) ++l;
    const uint64_t p2 = 1ull << (31 + l);
    return {static_cast<uint32_t>((p2 + d - 1) / d), l - 1};
  }
  __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return mul == 0u ? n : (__umulhi(n, mul) >> shift);
  }
};

// ---- per-head (or no) statistics: one vector per lane, grid (vectors / 256, parts) ---------------
// IDX32: vector numbers, token numbers and element offsets fit 31 bits: the two divisions per lane (by
// vectors per row, by tokens per batch row) become a multiply-high and a shift each and the addresses are a
// base pointer plus a 32-bit offset.
// One launch can carry TWO problems that write into the same joint buffers (the text rows and the image rows
// of a dual-stream block: different inputs, weights, tables, lengths and row offsets): workgroups
// [0, blocks0) belong to the first, the rest to the second. The choice is workgroup-uniform, so it costs a
// handful of scalar selects; a single problem is blocks0 = gridDim.x.
template <typename T, typename TW> struct QkFlatProblem {
  const T *q_in, *k_in, *v_in;
  const TW *wq, *wk;
  const float *cos_t, *sin_t;
  int S, out_seq_offset;
  int64_t is_b, is_s, total_vec;
  FastDiv by_s;
};

template <typename T, typename TW, int NORM_MODE, bool GENERAL, bool IDX32>
__global__ __launch_bounds__(256) void qknorm_flat_kernel(
    const QkFlatProblem<T, TW> p0, const QkFlatProblem<T, TW> p1, unsigned blocks0,
    T* __restrict__ q_out, T* __restrict__ k_out, T* __restrict__ v_out, int HD, int D, int rot,
    int S_total, float eps, int vec_per_row, bool neox, bool ref_round, FastDiv by_vpr, float inv_d) {
  constexpr int EPV = Vec16<T>::N;
  const int lane = threadIdx.x & 63;
  const bool second = blockIdx.x >= blocks0;  // workgroup-uniform
  const T* __restrict__ q_in = second ? p1.q_in : p0.q_in;
  const T* __restrict__ k_in = second ? p1.k_in : p0.k_in;
  const T* __restrict__ v_in = second ? p1.v_in : p0.v_in;
  const TW* __restrict__ wq = second ? p1.wq : p0.wq;
  const TW* __restrict__ wk = second ? p1.wk : p0.wk;
  const float* __restrict__ cos_t = second ? p1.cos_t : p0.cos_t;
  const float* __restrict__ sin_t = second ? p1.sin_t : p0.sin_t;
  const int S = second ? p1.S : p0.S;
  const int out_seq_offset = second ? p1.out_seq_offset : p0.out_seq_offset;
  const int64_t is_b = second ? p1.is_b : p0.is_b, is_s = second ? p1.is_s : p0.is_s;
  const int64_t total_vec = second ? p1.total_vec : p0.total_vec;
  const FastDiv by_s = {second ? p1.by_s.mul : p0.by_s.mul, second ? p1.by_s.shift : p0.by_s.shift};
  // grid.y: 0 = q together with k (when there is one), 1 = the copy of v. A lane takes the SAME vector
  // position of q and of k: one index computation, one pair of cos/sin loads, two loads in flight.
  const bool copy_v = blockIdx.y != 0;
  const int64_t i_raw = static_cast<int64_t>(blockIdx.x - (second ? blocks0 : 0u)) * 256 + threadIdx.x;
  const bool valid = i_raw < total_vec;
  const int64_t i = valid ? i_raw : total_vec - 1;  // clamped lanes compute, never store
  int e0, b, s;
  if constexpr (IDX32) {
    const unsigned iu = static_cast<unsigned>(i), vpr = static_cast<unsigned>(vec_per_row);
    const unsigned tok = by_vpr.div(iu);
    e0 = static_cast<int>(iu - tok * vpr) * EPV;
    b = static_cast<int>(by_s.div(tok));
    s = static_cast<int>(tok - static_cast<unsigned>(b) * static_cast<unsigned>(S));
  } else {
    const int64_t tok = i / vec_per_row;
    e0 = static_cast<int>(i - tok * vec_per_row) * EPV;
    b = static_cast<int>(tok / S);
    s = static_cast<int>(tok - static_cast<int64_t>(b) * S);
  }
  // IDX32 also means that every element offset below fits 31 bits (checked by the launcher)
  using off_t = typename std::conditional<IDX32, unsigned, int64_t>::type;
  const off_t in_off = static_cast<off_t>(b) * static_cast<off_t>(is_b) + static_cast<off_t>(s) * static_cast<off_t>(is_s) +
                       static_cast<off_t>(e0);
  const off_t out_off = (static_cast<off_t>(b) * static_cast<off_t>(S_total) + static_cast<off_t>(out_seq_offset + s)) *
                            static_cast<off_t>(HD) + static_cast<off_t>(e0);
  if (copy_v) {  // block-uniform
    const u32x4 r = load_raw(v_in + in_off);
    if (valid) __builtin_nontemporal_store(r, reinterpret_cast<u32x4*>(v_out + out_off));
    return;
  }
  const bool has_k = k_in != nullptr;  // launch-uniform
  const u32x4 rq = load_raw(q_in + in_off);
  const u32x4 rk = has_k ? load_raw(k_in + in_off) : u32x4{0u, 0u, 0u, 0u};
  float xq[EPV], xk[EPV];
#pragma unroll
  for (int j = 0; j < EPV; ++j) { xq[j] = Raw<T>::get(rq, j); xk[j] = Raw<T>::get(rk, j); }
  const int d0 = (D & (D - 1)) == 0 ? (e0 & (D - 1)) : e0 % D;  // head sizes are powers of two in practice
  float rstd_q = 1.f, rstd_k = 1.f;
  if constexpr (NORM_MODE == ODIT_NORM_HEAD) {
    float sq = 0.f, sk = 0.f;
#pragma unroll
    for (int j = 0; j < EPV; ++j) { sq = fmaf(xq[j], xq[j], sq); sk = fmaf(xk[j], xk[j], sk); }
    switch (D / EPV) {  // lanes per head row: wave-uniform
      case 64: sq = group_sum<64>(sq); sk = group_sum<64>(sk); break;
      case 32: sq = group_sum<32>(sq); sk = group_sum<32>(sk); break;
      case 16: sq = group_sum<16>(sq); sk = group_sum<16>(sk); break;
      case 8: sq = group_sum<8>(sq); sk = group_sum<8>(sk); break;
      case 4: sq = group_sum<4>(sq); sk = group_sum<4>(sk); break;
      case 2: sq = group_sum<2>(sq); sk = group_sum<2>(sk); break;
      default: break;
    }
    // a power-of-two head size divides exactly as a multiplication; any other keeps the division's rounding
    if ((D & (D - 1)) == 0) {  // launch-uniform
      rstd_q = rsqrtf(sq * inv_d + eps);
      rstd_k = rsqrtf(sk * inv_d + eps);
    } else {
      rstd_q = rsqrtf(sq / static_cast<float>(D) + eps);
      rstd_k = rsqrtf(sk / static_cast<float>(D) + eps);
    }
  }
  const float* cr = cos_t ? cos_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
  const float* sr = sin_t ? sin_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
  transform_vec<T, TW, NORM_MODE != ODIT_NORM_NONE, true, GENERAL>(xq, rstd_q, wq ? wq + d0 : nullptr, cr, sr, d0,
                                                                   rot, true, lane, neox, ref_round);
  if (has_k)
    transform_vec<T, TW, NORM_MODE != ODIT_NORM_NONE, true, GENERAL>(xk, rstd_k, wk ? wk + d0 : nullptr, cr, sr, d0,
                                                                     rot, true, lane, neox, ref_round);
  if (valid) {
    __builtin_nontemporal_store(pack_vec<T>(xq), reinterpret_cast<u32x4*>(q_out + out_off));
    if (has_k) __builtin_nontemporal_store(pack_vec<T>(xk), reinterpret_cast<u32x4*>(k_out + out_off));
  }
}

// ---- whole-row statistics: one wavefront per (token, part), row held in registers ---------------
template <typename T, typename TW, int NV, bool GENERAL>
__global__ __launch_bounds__(256) void qknorm_row_kernel(
    const T* __restrict__ q_in, const T* __restrict__ k_in, const T* __restrict__ v_in,
    T* __restrict__ q_out, T* __restrict__ k_out, T* __restrict__ v_out,
    const TW* __restrict__ wq, const TW* __restrict__ wk, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int B, int S, int HD, int D, int rot, int64_t is_b,
    int64_t is_s, int out_seq_offset, int S_total, float eps, bool neox, bool ref_round) {
  constexpr int EPV = Vec16<T>::N;
  const int lane = threadIdx.x & 63;
  const int kind = blockIdx.y == 0 ? 0 : (blockIdx.y == 1 && k_in != nullptr ? 1 : 2);
  const unsigned tok = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);  // B*S < 2^31 (checked by the caller)
  if (tok >= static_cast<unsigned>(B) * static_cast<unsigned>(S)) return;  // wave-uniform
  const int b = static_cast<int>(tok / static_cast<unsigned>(S));
  const int s = static_cast<int>(tok - static_cast<unsigned>(b) * static_cast<unsigned>(S));
  const T* in = (kind == 0 ? q_in : (kind == 1 ? k_in : v_in)) + b * is_b + s * is_s;
  T* out = (kind == 0 ? q_out : (kind == 1 ? k_out : v_out)) +
           (static_cast<int64_t>(b) * S_total + out_seq_offset + s) * HD;
  u32x4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e0 = (i * 64 + lane) * EPV;
    raw[i] = e0 < HD ? load_raw(in + e0) : u32x4{0u, 0u, 0u, 0u};
  }
  if (kind == 2) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e0 = (i * 64 + lane) * EPV;
      if (e0 < HD) store_raw(out + e0, raw[i]);
    }
    return;
  }
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int j = 0; j < EPV; ++j) { const float t = Raw<T>::get(raw[i], j); sq = fmaf(t, t, sq); }
  const float rstd = rsqrtf(wave_sum(sq) / static_cast<float>(HD) + eps);
  const TW* w = kind == 0 ? wq : wk;
  const float* cr = cos_t ? cos_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
  const float* sr = sin_t ? sin_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e0 = (i * 64 + lane) * EPV;
    const bool valid = e0 < HD;
    float x[EPV];
#pragma unroll
    for (int j = 0; j < EPV; ++j) x[j] = Raw<T>::get(raw[i], j);
    transform_vec<T, TW, true, false, GENERAL>(x, rstd, w ? w + e0 : nullptr, cr, sr, e0 % D, rot, valid, lane,
                                               neox, ref_round);
    if (valid) store_raw(out + e0, pack_vec<T>(x));
  }
}

}  // namespace odit

// The kernel family is compiled once per activation dtype (translation units selected with
// -DODIT_QK_TU=<odit_dtype code>) so the three can build in parallel; TU 0 also carries the
// argument checks and the exported entry point.
#ifndef ODIT_QK_TU
#error "compile with -DODIT_QK_TU=0|1|2"
#endif

namespace odit {

struct QkArgs {
  const void *q_in, *k_in, *v_in;
  void *q_out, *k_out, *v_out;
  const void *wq, *wk;
  const float *cos, *sin;
  int B, S, HD, D, rot;
  int64_t is_b, is_s;
  int out_seq_offset, S_total;
  float eps;
  int norm_mode;
  bool w_is_f32, neox, ref_round;
  int nv;
  hipStream_t stream;
  // optional second problem of the same launch (per-head or no statistics only): same outputs, head
  // layout, rotary width, weights' type and flags; its own inputs, weights, tables, length and row offset
  bool pair = false;
  const void *q_in2 = nullptr, *k_in2 = nullptr, *v_in2 = nullptr, *wq2 = nullptr, *wk2 = nullptr;
  const float *cos2 = nullptr, *sin2 = nullptr;
  int S2 = 0, out_seq_offset2 = 0;
  int64_t is_b2 = 0, is_s2 = 0;
};

int qknorm_rope_bf16(const QkArgs& a);
int qknorm_rope_f16(const QkArgs& a);
int qknorm_rope_f32(const QkArgs& a);

template <typename T, typename TW, int NORM_MODE, bool GENERAL> static int qk_flat(const QkArgs& a) {
  constexpr int EPV = Vec16<T>::N;
  const int vpr = a.HD / EPV;
  QkFlatProblem<T, TW> p0, p1;
  p0.q_in = static_cast<const T*>(a.q_in); p0.k_in = static_cast<const T*>(a.k_in); p0.v_in = static_cast<const T*>(a.v_in);
  p0.wq = static_cast<const TW*>(a.wq); p0.wk = static_cast<const TW*>(a.wk);
  p0.cos_t = a.cos; p0.sin_t = a.sin; p0.S = a.S; p0.out_seq_offset = a.out_seq_offset;
  p0.is_b = a.is_b; p0.is_s = a.is_s; p0.total_vec = static_cast<int64_t>(a.B) * a.S * vpr;
  p0.by_s = FastDiv::make(static_cast<uint32_t>(a.S));
  p1 = p0;
  if (a.pair) {
    p1.q_in = static_cast<const T*>(a.q_in2); p1.k_in = static_cast<const T*>(a.k_in2); p1.v_in = static_cast<const T*>(a.v_in2);
    p1.wq = static_cast<const TW*>(a.wq2); p1.wk = static_cast<const TW*>(a.wk2);
    p1.cos_t = a.cos2; p1.sin_t = a.sin2; p1.S = a.S2; p1.out_seq_offset = a.out_seq_offset2;
    p1.is_b = a.is_b2; p1.is_s = a.is_s2; p1.total_vec = static_cast<int64_t>(a.B) * a.S2 * vpr;
    p1.by_s = FastDiv::make(static_cast<uint32_t>(a.S2));
  }
  const int64_t blocks0 = (p0.total_vec + 255) / 256, blocks1 = a.pair ? (p1.total_vec + 255) / 256 : 0;
  const int nparts = 1 + (a.v_in != nullptr);  // q (with k) | v
  const dim3 grid(static_cast<unsigned>(blocks0 + blocks1), nparts);
#define ODIT_QK_FLAT(I32)                                                                          \
  hipLaunchKernelGGL((qknorm_flat_kernel<T, TW, NORM_MODE, GENERAL, I32>), grid, dim3(256), 0, a.stream, \
                     p0, p1, static_cast<unsigned>(blocks0), static_cast<T*>(a.q_out), static_cast<T*>(a.k_out), \
                     static_cast<T*>(a.v_out), a.HD, a.D, a.rot, a.S_total, a.eps, vpr, a.neox, a.ref_round, \
                     FastDiv::make(static_cast<uint32_t>(vpr)), 1.f / static_cast<float>(a.D))
  // 32-bit indexing: vector numbers and every element offset of the inputs and of the joint outputs below 2^31
  const int64_t in_span = (a.B - 1) * a.is_b + (a.S - 1) * a.is_s + a.HD;
  const int64_t in_span2 = a.pair ? (a.B - 1) * a.is_b2 + (a.S2 - 1) * a.is_s2 + a.HD : 0;
  const int64_t out_span = static_cast<int64_t>(a.B) * a.S_total * a.HD;
  const bool idx32 = p0.total_vec < (1ll << 31) && p1.total_vec < (1ll << 31) && blocks0 + blocks1 < (1ll << 31) &&
                     in_span < (1ll << 31) && in_span2 < (1ll << 31) && out_span < (1ll << 31) &&
                     a.is_b >= 0 && a.is_s >= 0 && a.is_b2 >= 0 && a.is_s2 >= 0;
  if (idx32) ODIT_QK_FLAT(true); else ODIT_QK_FLAT(false);
#undef ODIT_QK_FLAT
  return check_launch("odit_qknorm_rope");
}

template <typename T, typename TW, int NV, bool GENERAL> static int qk_row(const QkArgs& a) {
  const int64_t toks = static_cast<int64_t>(a.B) * a.S;
  const int nparts = 1 + (a.k_in != nullptr) + (a.v_in != nullptr);
  const dim3 grid(static_cast<unsigned>((toks + 3) / 4), nparts);
  hipLaunchKernelGGL((qknorm_row_kernel<T, TW, NV, GENERAL>), grid, dim3(256), 0, a.stream,
                     static_cast<const T*>(a.q_in), static_cast<const T*>(a.k_in),
                     static_cast<const T*>(a.v_in), static_cast<T*>(a.q_out), static_cast<T*>(a.k_out),
                     static_cast<T*>(a.v_out), static_cast<const TW*>(a.wq), static_cast<const TW*>(a.wk),
                     a.cos, a.sin, a.B, a.S, a.HD, a.D, a.rot, a.is_b, a.is_s, a.out_seq_offset,
                     a.S_total, a.eps, a.neox, a.ref_round);
  return check_launch("odit_qknorm_rope");
}

template <typename T, typename TW> static int qk_go(const QkArgs& a) {
  const bool general = a.neox || a.ref_round;
  switch (a.norm_mode) {
    case ODIT_NORM_NONE:
      return general ? qk_flat<T, TW, ODIT_NORM_NONE, true>(a) : qk_flat<T, TW, ODIT_NORM_NONE, false>(a);
    case ODIT_NORM_HEAD:
      return general ? qk_flat<T, TW, ODIT_NORM_HEAD, true>(a) : qk_flat<T, TW, ODIT_NORM_HEAD, false>(a);
    default:
      break;
  }
#define ODIT_QK_ROW(NVV) return general ? qk_row<T, TW, NVV, true>(a) : qk_row<T, TW, NVV, false>(a)
  if (a.nv <= 2) ODIT_QK_ROW(2);
  else if (a.nv <= 6) ODIT_QK_ROW(6);
  else if (a.nv <= 10) ODIT_QK_ROW(10);
  else ODIT_QK_ROW(16);
#undef ODIT_QK_ROW
}

#if ODIT_QK_TU == 0
int qknorm_rope_bf16(const QkArgs& a) {
  return a.w_is_f32 ? qk_go<bf16_t, float>(a) : qk_go<bf16_t, bf16_t>(a);
}
#elif ODIT_QK_TU == 1
int qknorm_rope_f16(const QkArgs& a) {
  return a.w_is_f32 ? qk_go<f16_t, float>(a) : qk_go<f16_t, f16_t>(a);
}
#else
int qknorm_rope_f32(const QkArgs& a) { return qk_go<float, float>(a); }
#endif

}  // namespace odit

#if ODIT_QK_TU == 0
namespace odit {

// argument checks of one problem and its launch arguments; *empty is set when there is nothing to do
static int qk_fill(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_out, void* v_out,
                   const void* wq, const void* wk, const float* cos, const float* sin, int B, int S, int H, int D,
                   int rot, const int64_t* in_strides, int out_seq_offset, int S_total, float eps, int norm_mode,
                   int w_dtype, int dtype, unsigned flags, void* stream, QkArgs& a, bool* empty) {
  ODIT_CHECK_ARG(dtype == ODIT_BF16 || dtype == ODIT_F16 || dtype == ODIT_F32,
                 "odit_qknorm_rope: unknown dtype code %d", dtype);
  ODIT_CHECK_ARG(q_in && q_out, "odit_qknorm_rope: q_in/q_out must not be null");
  ODIT_CHECK_ARG((k_in == nullptr) == (k_out == nullptr) && (v_in == nullptr) == (v_out == nullptr),
                 "odit_qknorm_rope: k/v input and output must be given together");
  ODIT_CHECK_ARG(in_strides != nullptr, "odit_qknorm_rope: in_strides must not be null");
  ODIT_CHECK_ARG(B >= 0 && S >= 0 && H > 0 && D > 0, "odit_qknorm_rope: bad shape");
  ODIT_CHECK_ARG(out_seq_offset >= 0 && out_seq_offset + S <= S_total,
                 "odit_qknorm_rope: rows [%d, %d) do not fit a joint sequence of %d", out_seq_offset,
                 out_seq_offset + S, S_total);
  ODIT_CHECK_ARG(norm_mode >= ODIT_NORM_NONE && norm_mode <= ODIT_NORM_ROW,
                 "odit_qknorm_rope: bad norm_mode %d", norm_mode);
  ODIT_CHECK_ARG((cos == nullptr) == (sin == nullptr), "odit_qknorm_rope: cos and sin go together");
  ODIT_CHECK_ARG(w_dtype == dtype || w_dtype == ODIT_F32,
                 "odit_qknorm_rope: w_dtype must equal dtype or be ODIT_F32");
  const int esz = dtype == ODIT_F32 ? 4 : 2;
  const int epv = 16 / esz;
  const int lanes_per_head = D / epv;
  ODIT_CHECK_ARG(D % epv == 0 && lanes_per_head <= 64 && (lanes_per_head & (lanes_per_head - 1)) == 0,
                 "odit_qknorm_rope: head size %d unsupported (needs D/%d a power of two <= 64)", D, epv);
  if (cos != nullptr) {
    ODIT_CHECK_ARG(rot > 0 && rot <= D && rot % 8 == 0,
                   "odit_qknorm_rope: rot=%d must be a multiple of 8 in (0, D]", rot);
    ODIT_CHECK_ARG(aligned16(cos) && aligned16(sin),
                   "odit_qknorm_rope: cos/sin must be 16-byte aligned");
    if (flags & ODIT_FLAG_NEOX)
      ODIT_CHECK_ARG((rot / 2) % epv == 0, "odit_qknorm_rope: NeoX rotary needs rot/2 %% %d == 0", epv);
  }
  ODIT_CHECK_ARG(in_strides[0] % epv == 0 && in_strides[1] % epv == 0,
                 "odit_qknorm_rope: input strides must be multiples of %d elements", epv);
  ODIT_CHECK_ARG(aligned16(q_in) && aligned16(k_in) && aligned16(v_in) && aligned16(q_out) &&
                     aligned16(k_out) && aligned16(v_out) && aligned16(wq) && aligned16(wk),
                 "odit_qknorm_rope: pointers must be 16-byte aligned");
  const int64_t HD = static_cast<int64_t>(H) * D;
  const int nv = static_cast<int>((HD + 64 * epv - 1) / (64 * epv));
  if (nv > 16 && norm_mode == ODIT_NORM_ROW) {
    set_error("odit_qknorm_rope: H*D=%lld exceeds the %d elements one wavefront keeps in registers",
              static_cast<long long>(HD), 16 * 64 * epv);
    return ODIT_ENOTSUP;
  }
  *empty = B == 0 || S == 0;
  ODIT_CHECK_ARG(static_cast<int64_t>(B) * S <= 0x7fffffffll, "odit_qknorm_rope: B*S exceeds 2^31 - 1 rows");
  a.q_in = q_in; a.k_in = k_in; a.v_in = v_in;
  a.q_out = q_out; a.k_out = k_out; a.v_out = v_out;
  a.wq = wq; a.wk = wk; a.cos = cos; a.sin = sin;
  a.B = B; a.S = S; a.HD = static_cast<int>(HD); a.D = D; a.rot = rot;
  a.is_b = in_strides[0]; a.is_s = in_strides[1];
  a.out_seq_offset = out_seq_offset; a.S_total = S_total; a.eps = eps;
  a.norm_mode = norm_mode;
  a.w_is_f32 = (w_dtype == ODIT_F32);
  a.neox = (flags & ODIT_FLAG_NEOX) != 0;
  a.ref_round = (flags & ODIT_FLAG_REF_ROUNDING) && dtype != ODIT_F32;
  a.nv = nv;
  a.stream = static_cast<hipStream_t>(stream);
  return ODIT_OK;
}

static int qk_dispatch(const QkArgs& a, int dtype) {
  switch (dtype) {
    case ODIT_BF16: return qknorm_rope_bf16(a);
    case ODIT_F16: return qknorm_rope_f16(a);
    default: return qknorm_rope_f32(a);
  }
}

}  // namespace odit

extern "C" int odit_qknorm_rope(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                                void* k_out, void* v_out, const void* wq, const void* wk,
                                const float* cos, const float* sin, int B, int S, int H, int D,
                                int rot, const int64_t in_strides[2], int out_seq_offset,
                                int S_total, float eps, int norm_mode, int w_dtype, int dtype,
                                unsigned flags, void* stream) {
  using namespace odit;
  QkArgs a;
  bool empty = false;
  const int rc = qk_fill(q_in, k_in, v_in, q_out, k_out, v_out, wq, wk, cos, sin, B, S, H, D, rot, in_strides,
                         out_seq_offset, S_total, eps, norm_mode, w_dtype, dtype, flags, stream, a, &empty);
  if (rc != ODIT_OK || empty) return rc;
  return qk_dispatch(a, dtype);
}

extern "C" int odit_qknorm_rope_pair(const void* const q_in[2], const void* const k_in[2],
                                     const void* const v_in[2], void* q_out, void* k_out, void* v_out,
                                     const void* const wq[2], const void* const wk[2],
                                     const float* const cos[2], const float* const sin[2], int B,
                                     const int S[2], int H, int D, int rot, const int64_t in_strides[4],
                                     const int out_seq_offset[2], int S_total, float eps, int norm_mode,
                                     int w_dtype, int dtype, unsigned flags, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(q_in && k_in && v_in && wq && wk && cos && sin && S && in_strides && out_seq_offset,
                 "odit_qknorm_rope_pair: null argument array");
  ODIT_CHECK_ARG((k_in[0] == nullptr) == (k_in[1] == nullptr) && (v_in[0] == nullptr) == (v_in[1] == nullptr) &&
                     (cos[0] == nullptr) == (cos[1] == nullptr),
                 "odit_qknorm_rope_pair: both problems take the same optional operands (k, v, rotary tables)");
  QkArgs a[2];
  bool empty[2] = {false, false};
  for (int i = 0; i < 2; ++i) {
    const int rc = qk_fill(q_in[i], k_in[i], v_in[i], q_out, k_in[i] ? k_out : nullptr, v_in[i] ? v_out : nullptr,
                           wq[i], wk[i], cos[i], sin[i], B, S[i], H, D, rot, in_strides + 2 * i, out_seq_offset[i],
                           S_total, eps, norm_mode, w_dtype, dtype, flags, stream, a[i], &empty[i]);
    if (rc != ODIT_OK) return rc;
  }
  // one launch when the flat kernel takes both; whole-row statistics, or an empty problem: one call each
  if (norm_mode == ODIT_NORM_ROW || empty[0] || empty[1]) {
    for (int i = 0; i < 2; ++i) {
      if (empty[i]) continue;
      const int rc = qk_dispatch(a[i], dtype);
      if (rc != ODIT_OK) return rc;
    }
    return ODIT_OK;
  }
  QkArgs m = a[0];
  m.pair = true;
  m.q_in2 = a[1].q_in; m.k_in2 = a[1].k_in; m.v_in2 = a[1].v_in; m.wq2 = a[1].wq; m.wk2 = a[1].wk;
  m.cos2 = a[1].cos; m.sin2 = a[1].sin; m.S2 = a[1].S; m.out_seq_offset2 = a[1].out_seq_offset;
  m.is_b2 = a[1].is_b; m.is_s2 = a[1].is_s;
  return qk_dispatch(m, dtype);
}
#endif
