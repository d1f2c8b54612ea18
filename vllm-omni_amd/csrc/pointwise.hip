// K4 gated residual and the two activation helpers: pure streaming passes, 16 bytes per lane per
// access. Algorithmic traffic of the gated residual is 3 * B*S*C * sizeof(T) (read h, read y, write out);
// the [B,C] gate row stays cache-resident.
#include "odit_common.h"

namespace odit {

constexpr int kStreamUnroll = 1;  // 16-byte vectors per thread; measured: more per thread streams slower here

// GBIAS: a float32 [C] table is added to the gate (the gate is then table + per-token row, formed in
// registers); a template parameter so the plain pass carries no trace of it.
template <typename T, typename TG, bool REF_ROUND, bool GBIAS>
__global__ __launch_bounds__(256) void gated_residual_kernel(
    const T* __restrict__ h, const T* __restrict__ y, const TG* __restrict__ gate,
    const float* __restrict__ gate_bias, T* __restrict__ out, int S, int vec_per_row,
    int64_t total_vecs, int64_t hs_b, int64_t hs_s, int64_t ys_b, int64_t ys_s, int64_t os_b,
    int64_t os_s, int64_t gs_b, int64_t gs_s) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int EPG = Vec16<TG>::N;
  constexpr int U = kStreamUnroll;
  // a block owns 256*U consecutive vectors; vector u of a thread sits 256 vectors after vector u-1,
  // so every load/store instruction of the block touches one contiguous 4 KB run
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (256 * U) + threadIdx.x;
  Vec16<T> hv[U], yv[U];
  float g[U][EPV];
  int64_t ooff[U];
  bool ok[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * 256;
    ok[u] = i < total_vecs;
    if (ok[u]) {
      const int64_t row = i / vec_per_row;
      const int c0 = static_cast<int>(i - row * vec_per_row) * EPV;
      const int b = static_cast<int>(row / S);
      const int s = static_cast<int>(row - static_cast<int64_t>(b) * S);
      hv[u] = load16(h + b * hs_b + s * hs_s + c0);
      yv[u] = load16(y + b * ys_b + s * ys_s + c0);
      ooff[u] = b * os_b + s * os_s + c0;
      if (gate != nullptr) {
        const TG* gp = gate + b * gs_b + s * gs_s + c0;
#pragma unroll
        for (int q = 0; q < EPV / EPG; ++q) {
          const Vec16<TG> gv = load16(gp + q * EPG);
#pragma unroll
          for (int j = 0; j < EPG; ++j) g[u][q * EPG + j] = to_float(gv.e[j]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < EPV; ++j) g[u][j] = GBIAS ? 0.f : 1.f;
      }
      if (GBIAS) {
#pragma unroll
        for (int q = 0; q < EPV / 4; ++q) {
          const Vec16<float> bv = load16(gate_bias + c0 + q * 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) g[u][q * 4 + j] += bv.e[j];
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (ok[u]) {
      Vec16<T> ov;
#pragma unroll
      for (int j = 0; j < EPV; ++j) {
        const float hf = to_float(hv[u].e[j]);
        const float yf = to_float(yv[u].e[j]);
        const float r = REF_ROUND ? hf + round_to<T>(g[u][j] * yf) : fmaf(g[u][j], yf, hf);
        ov.e[j] = from_float<T>(r);
      }
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&ov), reinterpret_cast<u32x4*>(out + ooff[u]));
    }
  }
}

// scalar tail version for shapes / alignments the vector kernel cannot take
template <typename T, typename TG, bool REF_ROUND>
__global__ __launch_bounds__(256) void gated_residual_scalar_kernel(
    const T* __restrict__ h, const T* __restrict__ y, const TG* __restrict__ gate,
    const float* __restrict__ gate_bias, T* __restrict__ out, int S, int C, int64_t total,
    int64_t hs_b, int64_t hs_s, int64_t ys_b, int64_t ys_s, int64_t os_b, int64_t os_s,
    int64_t gs_b, int64_t gs_s) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t row = i / C;
    const int c = static_cast<int>(i - row * C);
    const int b = static_cast<int>(row / S);
    const int s = static_cast<int>(row - static_cast<int64_t>(b) * S);
    const float hf = to_float(h[b * hs_b + s * hs_s + c]);
    const float yf = to_float(y[b * ys_b + s * ys_s + c]);
    const float g = (gate ? to_float(gate[b * gs_b + s * gs_s + c]) : (gate_bias ? 0.f : 1.f)) +
                    (gate_bias ? gate_bias[c] : 0.f);
    const float r = REF_ROUND ? hf + round_to<T>(g * yf) : fmaf(g, yf, hf);
    out[b * os_b + s * os_s + c] = from_float<T>(r);
  }
}

static inline unsigned stream_grid(int64_t work_items) {
  // enough 256-thread blocks to cover the work once, capped at 16 blocks per CU of a 256-CU part
  const int64_t blocks = (work_items + 255) / 256;
  return static_cast<unsigned>(blocks < 1 ? 1 : (blocks > 256 * 16 ? 256 * 16 : blocks));
}

template <typename T, typename TG, bool REF_ROUND>
static int launch_gated(const void* h, const void* y, const void* gate, const float* gate_bias,
                        void* out, int B, int S, int C, const int64_t* hs, const int64_t* ys,
                        const int64_t* os, const int64_t* gs, hipStream_t stream) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int EPG = Vec16<TG>::N;
  const int64_t gs0 = gs ? gs[0] : 0, gs1 = gs ? gs[1] : 0;
  const bool vec_ok = C % EPV == 0 && aligned16(h) && aligned16(y) && aligned16(out) &&
                      aligned16(gate) && aligned16(gate_bias) && hs[0] % EPV == 0 && hs[1] % EPV == 0 && ys[0] % EPV == 0 &&
                      ys[1] % EPV == 0 && os[0] % EPV == 0 && os[1] % EPV == 0 && gs0 % EPG == 0 &&
                      gs1 % EPG == 0;
  if (vec_ok) {
    const int vpr = C / EPV;
    const int64_t total = static_cast<int64_t>(B) * S * vpr;
    const int64_t nblk = (total + 256 * kStreamUnroll - 1) / (256 * kStreamUnroll);
#define ODIT_GATED_LAUNCH(GB)                                                                      \
  hipLaunchKernelGGL((gated_residual_kernel<T, TG, REF_ROUND, GB>),                                \
                     dim3(static_cast<unsigned>(nblk)), dim3(256), 0, stream,                      \
                     static_cast<const T*>(h), static_cast<const T*>(y),                           \
                     static_cast<const TG*>(gate), gate_bias, static_cast<T*>(out), S, vpr, total, \
                     hs[0], hs[1], ys[0], ys[1], os[0], os[1], gs0, gs1)
    if (gate_bias) ODIT_GATED_LAUNCH(true); else ODIT_GATED_LAUNCH(false);
#undef ODIT_GATED_LAUNCH
  } else {
    const int64_t total = static_cast<int64_t>(B) * S * C;
    hipLaunchKernelGGL((gated_residual_scalar_kernel<T, TG, REF_ROUND>), dim3(stream_grid(total)),
                       dim3(256), 0, stream, static_cast<const T*>(h), static_cast<const T*>(y),
                       static_cast<const TG*>(gate), gate_bias, static_cast<T*>(out), S, C, total,
                       hs[0], hs[1], ys[0], ys[1], os[0], os[1], gs0, gs1);
  }
  return check_launch("odit_gated_residual");
}

// ---- activations -------------------------------------------------------------------------------
struct GeluTanh {
  static __device__ __forceinline__ float apply(float x) {
    // 0.5 x (1 + tanh(u)) == x * sigmoid(2u),  u = sqrt(2/pi) (x + 0.044715 x^3)
    const float u = 0.7978845608028654f * x * fmaf(0.044715f * x, x, 1.f);
    return x / (1.f + __expf(-2.f * u));
  }
};
struct Silu {
  static __device__ __forceinline__ float apply(float x) { return x / (1.f + __expf(-x)); }
};

template <typename T, typename F>
__global__ __launch_bounds__(256) void unary_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                    int64_t n_vec, int64_t n) {
  constexpr int EPV = Vec16<T>::N;
  constexpr int U = kStreamUnroll;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (256 * U) + threadIdx.x;
  Vec16<T> v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * 256;
    if (i < n_vec) v[u] = load16(x + i * EPV);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * 256;
    if (i < n_vec) {
#pragma unroll
      for (int j = 0; j < EPV; ++j) v[u].e[j] = from_float<T>(F::apply(to_float(v[u].e[j])));
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&v[u]), reinterpret_cast<u32x4*>(out + i * EPV));
    }
  }
  // scalar tail (and the whole array when 16-byte access is not possible): first block only
  if (blockIdx.x == 0)
    for (int64_t i = n_vec * EPV + threadIdx.x; i < n; i += 256)
      out[i] = from_float<T>(F::apply(to_float(x[i])));
}

template <typename T, typename F>
static int launch_unary(const void* x, void* out, int64_t n, hipStream_t stream, const char* what) {
  constexpr int EPV = Vec16<T>::N;
  const int64_t n_vec = (aligned16(x) && aligned16(out)) ? n / EPV : 0;
  int64_t nblk = (n_vec + 256 * kStreamUnroll - 1) / (256 * kStreamUnroll);
  if (nblk < 1) nblk = 1;
  hipLaunchKernelGGL((unary_kernel<T, F>), dim3(static_cast<unsigned>(nblk)), dim3(256), 0, stream,
                     static_cast<const T*>(x), static_cast<T*>(out), n_vec, n);
  return check_launch(what);
}

}  // namespace odit

extern "C" int odit_gated_residual(const void* h, const void* y, const void* gate,
                                   const float* gate_bias, void* out, int B, int S, int C,
                                   const int64_t h_strides[2],
                                   const int64_t y_strides[2], const int64_t out_strides[2],
                                   const int64_t gate_strides[2], int gate_dtype, int dtype,
                                   unsigned flags, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(h && y && out, "odit_gated_residual: h/y/out must not be null");
  ODIT_CHECK_ARG(h_strides && y_strides && out_strides, "odit_gated_residual: null strides");
  ODIT_CHECK_ARG(gate == nullptr || gate_strides != nullptr,
                 "odit_gated_residual: gate given without gate_strides");
  ODIT_CHECK_ARG(B >= 0 && S >= 0 && C > 0, "odit_gated_residual: bad shape B=%d S=%d C=%d", B, S, C);
  ODIT_CHECK_ARG(gate_dtype == dtype || gate_dtype == ODIT_F32,
                 "odit_gated_residual: gate_dtype must equal dtype or be ODIT_F32");
  if (B == 0 || S == 0) return ODIT_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool rr = (flags & ODIT_FLAG_REF_ROUNDING) && gate_dtype == dtype && dtype != ODIT_F32;
#define ODIT_GR_GO(T, TG)                                                                       \
  return rr ? launch_gated<T, TG, true>(h, y, gate, gate_bias, out, B, S, C, h_strides,         \
                                        y_strides, out_strides, gate_strides, st)               \
            : launch_gated<T, TG, false>(h, y, gate, gate_bias, out, B, S, C, h_strides,        \
                                         y_strides, out_strides, gate_strides, st)
  if (gate_dtype == dtype) {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_GR_GO(T, T));
  } else {
    ODIT_DISPATCH_DTYPE(dtype, T, ODIT_GR_GO(T, float));
  }
#undef ODIT_GR_GO
  return ODIT_OK;
}

extern "C" int odit_gelu_tanh(const void* x, void* out, int64_t n, int dtype, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(n >= 0 && (n == 0 || (x && out)), "odit_gelu_tanh: bad arguments");
  if (n == 0) return ODIT_OK;
  ODIT_DISPATCH_DTYPE(dtype, T, return (launch_unary<T, GeluTanh>(
                                    x, out, n, static_cast<hipStream_t>(stream), "odit_gelu_tanh")));
  return ODIT_OK;
}

extern "C" int odit_silu(const void* x, void* out, int64_t n, int dtype, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(n >= 0 && (n == 0 || (x && out)), "odit_silu: bad arguments");
  if (n == 0) return ODIT_OK;
  ODIT_DISPATCH_DTYPE(dtype, T, return (launch_unary<T, Silu>(
                                    x, out, n, static_cast<hipStream_t>(stream), "odit_silu")));
  return ODIT_OK;
}
