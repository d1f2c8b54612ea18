// K3: fused LayerNorm + adaLN shift/scale modulation.
//
// The row is read from HBM exactly once (each lane keeps one or two 16-byte vectors of it in
// registers), both LayerNorm moments come from that single sweep, and the modulated row is written
// back once. Algorithmic traffic is therefore 2 * B*S*C * sizeof(T) (+ the [B,C] shift/scale rows,
// which stay L2-resident).
#include "odit_common.h"

namespace odit {

template <typename TM> struct ModLoader {
  // returns element c of a modulation row (or 0 when the pointer is null)
  static __device__ __forceinline__ float at(const TM* p, int c) { return p ? to_float(p[c]) : 0.f; }
};

// N consecutive parameters starting at p (16-byte aligned, N * sizeof(TP) a multiple of 16),
// fetched with 16-byte loads; `fill` when p is null.
template <typename TP, int N>
__device__ __forceinline__ void load_params(const TP* p, float fill, float (&dst)[N]) {
  constexpr int E = Vec16<TP>::N;
  static_assert(N % E == 0, "parameter run must be whole 16-byte vectors");
  if (p == nullptr) {
#pragma unroll
    for (int j = 0; j < N; ++j) dst[j] = fill;
    return;
  }
#pragma unroll
  for (int q = 0; q < N / E; ++q) {
    Vec16<TP> t = load16(p + q * E);
#pragma unroll
    for (int j = 0; j < E; ++j) dst[q * E + j] = to_float(t.e[j]);
  }
}

// One workgroup of W wavefronts per token row; every lane holds at most NVL 16-byte vectors of the
// row (as loaded, unpacked where used), so the kernel needs few registers and many rows are in flight
// per CU: while some waves wait for their loads others reduce or store, which is what keeps a
// read-once / write-once pass near the HBM rate. The two LayerNorm moments are taken in one sweep
// about the row's first element (a shift every wave can fetch by itself) and combined across the W
// waves through 2*W floats of LDS.
// PLAIN = the per-block call of the DiT step (shift and scale given, no per-token index, no LayerNorm
// affine): the optional operands cost registers and address arithmetic even when absent, and this
// pass lives on how many rows a CU keeps in flight. (A one-wavefront-per-row form with two rows per
// wavefront streams 5 % faster from cold buffers and 25 % slower on rows a GEMM has just written, which is
// what every call inside a block sees: 32.5 against 25.6 us per image + text pair launch in the step.)
//
// One launch can carry TWO problems of the same width (the image rows and the text rows of a dual-stream
// block): workgroups [0, rows0) belong to the first, the rest to the second; the choice is
// workgroup-uniform (scalar selects). A single problem is rows0 = gridDim.x.
template <typename T, typename TM> struct AdalnProblem {
  const T* x;
  T* out;
  const TM *shift, *scale;
  int S;
  int64_t xs_b, xs_s, os_b, os_s, mod_stride_b;
};

template <typename T, typename TM, int W, int NVL, bool REF_ROUND, bool PLAIN>
__global__ __launch_bounds__(W * 64) void adaln_rows_kernel(
    const AdalnProblem<T, TM> p0, const AdalnProblem<T, TM> p1, unsigned rows0,
    const int32_t* __restrict__ index,
    const float* __restrict__ ln_w, const float* __restrict__ ln_b,
    const float* __restrict__ shift_bias, const float* __restrict__ scale_bias, int B, int C,
    int64_t mod_stride_s, float eps) {
  constexpr int EPV = Vec16<T>::N;
  const int tid = threadIdx.x;
  const bool second = blockIdx.x >= rows0;  // workgroup-uniform
  const T* __restrict__ x = second ? p1.x : p0.x;
  T* __restrict__ out = second ? p1.out : p0.out;
  const TM* __restrict__ shift = second ? p1.shift : p0.shift;
  const TM* __restrict__ scale = second ? p1.scale : p0.scale;
  const int S = second ? p1.S : p0.S;
  const int64_t xs_b = second ? p1.xs_b : p0.xs_b, xs_s = second ? p1.xs_s : p0.xs_s;
  const int64_t os_b = second ? p1.os_b : p0.os_b, os_s = second ? p1.os_s : p0.os_s;
  const int64_t mod_stride_b = second ? p1.mod_stride_b : p0.mod_stride_b;
  const unsigned row = blockIdx.x - (second ? rows0 : 0u);  // the launcher keeps B*S below 2^31
  const int b = static_cast<int>(row / static_cast<unsigned>(S));
  const int s = static_cast<int>(row - static_cast<unsigned>(b) * static_cast<unsigned>(S));
  const T* xr = x + b * xs_b + s * xs_s;
  T* orow = out + b * os_b + s * os_s;

  u32x4 raw[NVL];
#pragma unroll
  for (int i = 0; i < NVL; ++i) {
    const int c0 = (i * (W * 64) + tid) * EPV;
    // the row is consumed once: keep it out of the way of the [B,C] modulation rows in L2
    raw[i] = c0 < C ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + c0)) : u32x4{0u, 0u, 0u, 0u};
  }
  const float k0 = to_float(xr[0]);  // same address for the whole workgroup: one broadcast load
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int i = 0; i < NVL; ++i) {
    const int c0 = (i * (W * 64) + tid) * EPV;
    if (c0 < C) {
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        const float d = Raw<T>::get(raw[i], j) - k0;
        s1 += d;
        s2 = fmaf(d, d, s2);
      }
    }
  }
  s1 = wave_sum(s1);
  s2 = wave_sum(s2);
  if (W > 1) {
    __shared__ float red[2][W];
    if ((tid & 63) == 0) { red[0][tid >> 6] = s1; red[1][tid >> 6] = s2; }
    __syncthreads();
    s1 = 0.f; s2 = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) { s1 += red[0][w]; s2 += red[1][w]; }
  }
  const float inv_c = 1.f / static_cast<float>(C);
  const float m1 = s1 * inv_c;
  const float mean = k0 + m1;
  const float rstd = rsqrtf(fmaxf(s2 * inv_c - m1 * m1, 0.f) + eps);

  int mrow = b;
  if (!PLAIN && index != nullptr && index[static_cast<int64_t>(b) * S + s] != 0) mrow = b + B;
  // per-token modulation rows (mod_stride_s != 0) and the float32 [C] tables added to them are
  // optional operands like the index: the PLAIN specialisation has neither
  const int64_t moff = mrow * mod_stride_b + (PLAIN ? 0 : s * mod_stride_s);
  const TM* sh = (PLAIN || shift) ? shift + moff : nullptr;
  const TM* sc = (PLAIN || scale) ? scale + moff : nullptr;

#pragma unroll
  for (int i = 0; i < NVL; ++i) {
    const int c0 = (i * (W * 64) + tid) * EPV;
    if (c0 < C) {
      float scl_v[EPV], shf_v[EPV], lw_v[EPV], lb_v[EPV];
      load_params<TM, EPV>(sc ? sc + c0 : nullptr, 0.f, scl_v);
      load_params<TM, EPV>(sh ? sh + c0 : nullptr, 0.f, shf_v);
      if (!PLAIN) {
        load_params<float, EPV>(ln_w ? ln_w + c0 : nullptr, 1.f, lw_v);
        load_params<float, EPV>(ln_b ? ln_b + c0 : nullptr, 0.f, lb_v);
        if (scale_bias || shift_bias) {
          float scb[EPV], shb[EPV];
          load_params<float, EPV>(scale_bias ? scale_bias + c0 : nullptr, 0.f, scb);
          load_params<float, EPV>(shift_bias ? shift_bias + c0 : nullptr, 0.f, shb);
#pragma unroll
          for (int j = 0; j < EPV; ++j) { scl_v[j] += scb[j]; shf_v[j] += shb[j]; }
        }
      }
      float r[EPV];
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        float y = (Raw<T>::get(raw[i], j) - mean) * rstd;
        if (!PLAIN && ln_w) y *= lw_v[j];
        if (!PLAIN && ln_b) y += lb_v[j];
        if (REF_ROUND) {
          // torch path: LN -> T, (1 + scale) -> T, product -> T, sum -> T
          r[j] = round_to<T>(round_to<T>(y) * round_to<T>(1.f + scl_v[j])) + shf_v[j];
        } else {
          r[j] = fmaf(y, 1.f + scl_v[j], shf_v[j]);
        }
      }
      u32x4 o;
#pragma unroll
      for (int j = 0; j < EPV / 2; ++j) Raw<T>::set2(o, j, r[2 * j], r[2 * j + 1]);
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(orow + c0));
    }
  }
}

// Any C (no vector-width or register-cache constraint): the row is read three times through L2.
template <typename T, typename TM, bool REF_ROUND>
__global__ __launch_bounds__(256) void adaln_rows_generic_kernel(
    const T* __restrict__ x, T* __restrict__ out, const TM* __restrict__ shift,
    const TM* __restrict__ scale, const int32_t* __restrict__ index,
    const float* __restrict__ ln_w, const float* __restrict__ ln_b,
    const float* __restrict__ shift_bias, const float* __restrict__ scale_bias, int B, int S, int C,
    int64_t xs_b, int64_t xs_s, int64_t os_b, int64_t os_s, int64_t mod_stride_b,
    int64_t mod_stride_s, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= static_cast<int64_t>(B) * S) return;
  const int b = static_cast<int>(row / S);
  const int s = static_cast<int>(row - static_cast<int64_t>(b) * S);
  const T* xr = x + b * xs_b + s * xs_s;
  T* orow = out + b * os_b + s * os_s;
  float sum = 0.f;
  for (int c = lane; c < C; c += 64) sum += to_float(xr[c]);
  const float inv_c = 1.f / static_cast<float>(C);
  const float mean = wave_sum(sum) * inv_c;
  float sq = 0.f;
  for (int c = lane; c < C; c += 64) { const float d = to_float(xr[c]) - mean; sq += d * d; }
  const float rstd = rsqrtf(wave_sum(sq) * inv_c + eps);
  int mrow = b;
  if (index != nullptr && index[static_cast<int64_t>(b) * S + s] != 0) mrow = b + B;
  const int64_t moff = mrow * mod_stride_b + s * mod_stride_s;
  const TM* sh = shift ? shift + moff : nullptr;
  const TM* sc = scale ? scale + moff : nullptr;
  for (int c = lane; c < C; c += 64) {
    float y = (to_float(xr[c]) - mean) * rstd;
    if (ln_w) y *= ln_w[c];
    if (ln_b) y += ln_b[c];
    const float scl = ModLoader<TM>::at(sc, c) + (scale_bias ? scale_bias[c] : 0.f);
    const float shf = ModLoader<TM>::at(sh, c) + (shift_bias ? shift_bias[c] : 0.f);
    float r;
    if (REF_ROUND) {
      r = round_to<T>(round_to<T>(y) * round_to<T>(1.f + scl)) + shf;
    } else {
      r = fmaf(y, 1.f + scl, shf);
    }
    orow[c] = from_float<T>(r);
  }
}

// One problem's row operands as the launcher takes them (second = nullptr: one problem).
struct AdalnRows {
  const void *x; void* out; const void *shift, *scale;
  int S;
  const int64_t *xs, *os;
  int64_t mod_stride_b;
};

template <typename T, typename TM, bool REF_ROUND>
static int launch_adaln(const AdalnRows& r0, const AdalnRows* r1,
                        const int32_t* index, const float* ln_w, const float* ln_b,
                        const float* shift_bias, const float* scale_bias, int B, int C,
                        int64_t mod_stride_s, float eps, hipStream_t stream) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int EPM = Vec16<TM>::N;
  auto fill = [](const AdalnRows& r) {
    AdalnProblem<T, TM> p;
    p.x = static_cast<const T*>(r.x); p.out = static_cast<T*>(r.out);
    p.shift = static_cast<const TM*>(r.shift); p.scale = static_cast<const TM*>(r.scale);
    p.S = r.S; p.xs_b = r.xs[0]; p.xs_s = r.xs[1]; p.os_b = r.os[0]; p.os_s = r.os[1];
    p.mod_stride_b = r.mod_stride_b;
    return p;
  };
  // EPV >= EPM always (TM is T or float), so C % EPV == 0 keeps parameter runs vector-aligned too.
  auto rows_vec_ok = [&](const AdalnRows& r) {
    return aligned16(r.x) && aligned16(r.out) && r.xs[0] % EPV == 0 && r.xs[1] % EPV == 0 && r.os[0] % EPV == 0 &&
           r.os[1] % EPV == 0 && aligned16(r.shift) && aligned16(r.scale) && r.mod_stride_b % EPM == 0;
  };
  const AdalnProblem<T, TM> p0 = fill(r0), p1 = r1 ? fill(*r1) : p0;
  const int64_t rows0 = static_cast<int64_t>(B) * r0.S, rows1 = r1 ? static_cast<int64_t>(B) * r1->S : 0;
  const int64_t rows = rows0 + rows1;
  const bool vec_ok = (C % EPV == 0) && rows_vec_ok(r0) && (!r1 || rows_vec_ok(*r1)) &&
                      mod_stride_s % EPM == 0 && aligned16(ln_w) && aligned16(ln_b) &&
                      aligned16(shift_bias) && aligned16(scale_bias);
  const int nvec = (C + EPV - 1) / EPV;  // 16-byte vectors per row
  const bool plain = r0.shift && r0.scale && (!r1 || (r1->shift && r1->scale)) && !index && !ln_w && !ln_b &&
                     !shift_bias && !scale_bias && mod_stride_s == 0;
#define ODIT_ADALN_LAUNCH(WW, NVLL, PL)                                                            \
  hipLaunchKernelGGL((adaln_rows_kernel<T, TM, WW, NVLL, REF_ROUND, PL>),                          \
                     dim3(static_cast<unsigned>(rows)), dim3(WW * 64), 0, stream, p0, p1,          \
                     static_cast<unsigned>(rows0), index, ln_w, ln_b, shift_bias, scale_bias, B,   \
                     C, mod_stride_s, eps)
#define ODIT_ADALN_CASE(WW, NVLL)                                                                  \
  do { if (plain) ODIT_ADALN_LAUNCH(WW, NVLL, true); else ODIT_ADALN_LAUNCH(WW, NVLL, false); } while (0)
  if (vec_ok && nvec <= 8 * 64 * 2 && rows <= 0x7fffffffll) {
    if (nvec <= 64) ODIT_ADALN_CASE(1, 1);
    else if (nvec <= 128) ODIT_ADALN_CASE(2, 1);
    else if (nvec <= 256) ODIT_ADALN_CASE(4, 1);
    else if (nvec <= 384) ODIT_ADALN_CASE(3, 2);
    else if (nvec <= 512) ODIT_ADALN_CASE(4, 2);
    else if (nvec <= 768) ODIT_ADALN_CASE(6, 2);
    else ODIT_ADALN_CASE(8, 2);
  } else {
    // any width: one launch per problem
    for (const AdalnRows* r : {&r0, r1}) {
      if (r == nullptr) continue;
      const int64_t n = static_cast<int64_t>(B) * r->S;
      const dim3 grid(static_cast<unsigned>((n + 3) / 4));
      hipLaunchKernelGGL((adaln_rows_generic_kernel<T, TM, REF_ROUND>), grid, dim3(256), 0, stream,
                         static_cast<const T*>(r->x), static_cast<T*>(r->out),
                         static_cast<const TM*>(r->shift), static_cast<const TM*>(r->scale), index, ln_w,
                         ln_b, shift_bias, scale_bias, B, r->S, C, r->xs[0], r->xs[1], r->os[0], r->os[1],
                         r->mod_stride_b, mod_stride_s, eps);
    }
  }
#undef ODIT_ADALN_CASE
#undef ODIT_ADALN_LAUNCH
  return check_launch("odit_adaln_modulate");
}

}  // namespace odit

extern "C" int odit_adaln_modulate(const void* x, void* out, const void* shift, const void* scale,
                                   const int32_t* index, const float* ln_weight,
                                   const float* ln_bias, const float* shift_bias,
                                   const float* scale_bias, int B, int S, int C,
                                   const int64_t x_strides[2], const int64_t out_strides[2],
                                   int64_t mod_stride_b, int64_t mod_stride_s, float eps,
                                   int mod_dtype, int dtype, unsigned flags, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(x && out, "odit_adaln_modulate: x/out must not be null");
  ODIT_CHECK_ARG(x_strides && out_strides, "odit_adaln_modulate: strides must not be null");
  ODIT_CHECK_ARG(B >= 0 && S >= 0 && C > 0, "odit_adaln_modulate: bad shape B=%d S=%d C=%d", B, S, C);
  ODIT_CHECK_ARG(mod_dtype == dtype || mod_dtype == ODIT_F32,
                 "odit_adaln_modulate: mod_dtype must equal dtype or be ODIT_F32 (got %d vs %d)",
                 mod_dtype, dtype);
  ODIT_CHECK_ARG(static_cast<int64_t>(B) * S < (1ll << 33), "odit_adaln_modulate: too many rows");
  ODIT_CHECK_ARG(mod_stride_b >= 0 && mod_stride_s >= 0, "odit_adaln_modulate: negative modulation stride");
  ODIT_CHECK_ARG(!(index && mod_stride_s != 0),
                 "odit_adaln_modulate: per-token modulation rows and a row index exclude each other");
  if (B == 0 || S == 0) return ODIT_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool rr = (flags & ODIT_FLAG_REF_ROUNDING) && mod_dtype == dtype && dtype != ODIT_F32;
  const AdalnRows r0{x, out, shift, scale, S, x_strides, out_strides, mod_stride_b};
#define ODIT_ADALN_GO(T, TM)                                                                     \
  return rr ? launch_adaln<T, TM, true>(r0, nullptr, index, ln_weight, ln_bias, shift_bias,       \
                                        scale_bias, B, C, mod_stride_s, eps, st)                  \
            : launch_adaln<T, TM, false>(r0, nullptr, index, ln_weight, ln_bias, shift_bias,      \
                                         scale_bias, B, C, mod_stride_s, eps, st)
  if (mod_dtype == dtype) {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_ADALN_GO(T, T));
  } else {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_ADALN_GO(T, float));
  }
#undef ODIT_ADALN_GO
  return ODIT_OK;
}

extern "C" int odit_adaln_modulate_pair(const void* const x[2], void* const out[2], const void* const shift[2],
                                        const void* const scale[2], int B, const int S[2], int C,
                                        const int64_t x_strides[4], const int64_t out_strides[4],
                                        const int64_t mod_stride_b[2], float eps, int mod_dtype, int dtype,
                                        unsigned flags, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(x && out && shift && scale && S && x_strides && out_strides && mod_stride_b,
                 "odit_adaln_modulate_pair: null argument array");
  for (int i = 0; i < 2; ++i) {
    ODIT_CHECK_ARG(S[i] <= 0 || (x[i] && out[i]), "odit_adaln_modulate_pair: x/out must not be null");
    ODIT_CHECK_ARG(S[i] >= 0 && mod_stride_b[i] >= 0, "odit_adaln_modulate_pair: bad S or modulation stride");
  }
  ODIT_CHECK_ARG(B >= 0 && C > 0, "odit_adaln_modulate_pair: bad shape B=%d C=%d", B, C);
  ODIT_CHECK_ARG(mod_dtype == dtype || mod_dtype == ODIT_F32,
                 "odit_adaln_modulate_pair: mod_dtype must equal dtype or be ODIT_F32 (got %d vs %d)", mod_dtype, dtype);
  ODIT_CHECK_ARG(static_cast<int64_t>(B) * (static_cast<int64_t>(S[0]) + S[1]) < (1ll << 31),
                 "odit_adaln_modulate_pair: too many rows");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool rr = (flags & ODIT_FLAG_REF_ROUNDING) && mod_dtype == dtype && dtype != ODIT_F32;
  const AdalnRows r0{x[0], out[0], shift[0], scale[0], S[0], x_strides, out_strides, mod_stride_b[0]};
  const AdalnRows r1{x[1], out[1], shift[1], scale[1], S[1], x_strides + 2, out_strides + 2, mod_stride_b[1]};
  if (B == 0 || (S[0] == 0 && S[1] == 0)) return ODIT_OK;
  // an empty problem leaves a single one
  const AdalnRows& first = S[0] > 0 ? r0 : r1;
  const AdalnRows* second = (S[0] > 0 && S[1] > 0) ? &r1 : nullptr;
#define ODIT_ADALN_GO2(T, TM)                                                                        \
  return rr ? launch_adaln<T, TM, true>(first, second, nullptr, nullptr, nullptr, nullptr, nullptr, B, C, 0, eps, st) \
            : launch_adaln<T, TM, false>(first, second, nullptr, nullptr, nullptr, nullptr, nullptr, B, C, 0, eps, st)
  if (mod_dtype == dtype) {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_ADALN_GO2(T, T));
  } else {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_ADALN_GO2(T, float));
  }
#undef ODIT_ADALN_GO2
  return ODIT_OK;
}
