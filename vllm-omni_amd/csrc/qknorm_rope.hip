// K2: fused QK-RMSNorm + rotary embedding + scatter of q/k/v into the joint [txt;img] buffers.
//
// One 64-lane wavefront per token. The token's q, k and v rows (H*D elements each, usually three
// adjacent slices of one fused-QKV GEMM output row) are each read once with 16-byte loads and
// written once into row (out_seq_offset + s) of the dense joint buffers, so the three torch.cat
// copies of the reference never happen. Algorithmic traffic: 2 * 3 * B*S*H*D * sizeof(T)
// (+ S*rot*4 bytes of cos/sin, L2-resident across heads and batch).
//
// Lane layout: vector i*64+lane of the row covers elements e0..e0+EPV-1, e0 = (i*64+lane)*EPV, i.e.
// head e0/D, offset e0%D. A head row occupies D/EPV consecutive lanes, so the per-head mean square
// is a shuffle reduction over an aligned lane group; the whole-row variant reduces over the wave.
// Interleaved rotary pairs (2i, 2i+1) live inside one lane's vector; NeoX pairs are fetched from the
// lane rot/(2*EPV) away with a shuffle.
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

// GENERAL = false compiles the hot variant only (interleaved pairs, one final rounding); GENERAL =
// true takes NeoX pairing and reference rounding as wave-uniform run-time switches.
template <typename T, typename TW, int NV, int NORM_MODE, bool GENERAL>
__device__ __forceinline__ void norm_rope_row(const T* __restrict__ in, T* __restrict__ out,
                                              const TW* __restrict__ w,
                                              const float* __restrict__ cos_row,
                                              const float* __restrict__ sin_row, int HD, int D,
                                              int rot, float eps, int lane, bool neox_rt,
                                              bool ref_round_rt) {
  constexpr int EPV = Vec16<T>::N;
  const bool NEOX = GENERAL && neox_rt;
  const bool REF_ROUND = GENERAL && ref_round_rt;
  float v[NV][EPV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e0 = (i * 64 + lane) * EPV;
    if (e0 < HD) {
      const Vec16<T> t = load16(in + e0);
#pragma unroll
      for (int j = 0; j < EPV; ++j) v[i][j] = to_float(t.e[j]);
    } else {
#pragma unroll
      for (int j = 0; j < EPV; ++j) v[i][j] = 0.f;
    }
  }

  // ---- RMS statistics ----
  float rstd[NV];
  if constexpr (NORM_MODE == ODIT_NORM_ROW) {
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
      for (int j = 0; j < EPV; ++j) sq += v[i][j] * v[i][j];
    const float r = rsqrtf(wave_sum(sq) / static_cast<float>(HD) + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) rstd[i] = r;
  } else if constexpr (NORM_MODE == ODIT_NORM_HEAD) {
    const int lanes_per_head = D / EPV;  // power of two, <= 64 (checked on the host)
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float sq = 0.f;
#pragma unroll
      for (int j = 0; j < EPV; ++j) sq += v[i][j] * v[i][j];
      for (int off = lanes_per_head >> 1; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
      rstd[i] = rsqrtf(sq / static_cast<float>(D) + eps);
    }
  }

#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e0 = (i * 64 + lane) * EPV;
    const int d0 = e0 % D;
    float x[EPV];
#pragma unroll
    for (int j = 0; j < EPV; ++j) x[j] = v[i][j];

    if constexpr (NORM_MODE != ODIT_NORM_NONE) {
      float wv[EPV];
      if (w != nullptr && e0 < HD) {
        const TW* wp = w + (NORM_MODE == ODIT_NORM_ROW ? e0 : d0);
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
        if (REF_ROUND && NORM_MODE == ODIT_NORM_HEAD) {
          x[j] = round_to<T>(round_to<T>(x[j] * rstd[i]) * wv[j]);
        } else {
          x[j] = x[j] * rstd[i] * wv[j];
          if (REF_ROUND) x[j] = round_to<T>(x[j]);
        }
      }
    }

    // ---- rotary ----
    if (cos_row != nullptr) {
      if (!NEOX) {
        if (d0 < rot && e0 < HD) {
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
        // pair (d, d + rot/2): partner vector sits rot/(2*EPV) lanes away (same i: a head row never
        // straddles two register vectors of one lane because D/EPV lanes hold it contiguously)
        const int half = rot >> 1;
        const int dist = half / EPV;
        const bool lower = d0 < half;
        const int src = lower ? lane + dist : lane - dist;
        float px[EPV];
#pragma unroll
        for (int j = 0; j < EPV; ++j) px[j] = __shfl(x[j], src & 63, 64);
        if (d0 < rot && e0 < HD) {
          float c[EPV], s[EPV];
          const int t0 = lower ? d0 : d0 - half;
#pragma unroll
          for (int j = 0; j < EPV; ++j) { c[j] = cos_row[t0 + j]; s[j] = sin_row[t0 + j]; }
#pragma unroll
          for (int j = 0; j < EPV; ++j) {
            const float sgn = lower ? -1.f : 1.f;
            if (REF_ROUND) {
              const float cc = round_to<T>(c[j]), ss = round_to<T>(s[j]);
              x[j] = round_to<T>(x[j] * cc) + round_to<T>(sgn * px[j] * ss);
            } else {
              x[j] = x[j] * c[j] + sgn * px[j] * s[j];
            }
          }
        }
      }
    }

    if (e0 < HD) {
      Vec16<T> o;
#pragma unroll
      for (int j = 0; j < EPV; ++j) o.e[j] = from_float<T>(x[j]);
      store16(out + e0, o);
    }
  }
}

template <typename T, int NV>
__device__ __forceinline__ void copy_row(const T* __restrict__ in, T* __restrict__ out, int HD,
                                         int lane) {
  constexpr int EPV = Vec16<T>::N;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e0 = (i * 64 + lane) * EPV;
    if (e0 < HD) store16(out + e0, load16(in + e0));
  }
}

template <typename T, typename TW, int NV, int NORM_MODE, bool GENERAL>
__global__ __launch_bounds__(256) void qknorm_rope_kernel(
    const T* __restrict__ q_in, const T* __restrict__ k_in, const T* __restrict__ v_in,
    T* __restrict__ q_out, T* __restrict__ k_out, T* __restrict__ v_out,
    const TW* __restrict__ wq, const TW* __restrict__ wk, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int B, int S, int HD, int D, int rot, int64_t is_b,
    int64_t is_s, int out_seq_offset, int S_total, float eps, bool neox, bool ref_round) {
  const int lane = threadIdx.x & 63;
  const int64_t tok = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (tok >= static_cast<int64_t>(B) * S) return;
  const int b = static_cast<int>(tok / S);
  const int s = static_cast<int>(tok - static_cast<int64_t>(b) * S);
  const int64_t in_off = b * is_b + s * is_s;
  const int64_t out_off = (static_cast<int64_t>(b) * S_total + out_seq_offset + s) * HD;
  const float* cr = cos_t ? cos_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
  const float* sr = sin_t ? sin_t + static_cast<int64_t>(s) * (rot >> 1) : nullptr;
  norm_rope_row<T, TW, NV, NORM_MODE, GENERAL>(q_in + in_off, q_out + out_off, wq, cr, sr, HD, D,
                                                rot, eps, lane, neox, ref_round);
  if (k_in != nullptr)
    norm_rope_row<T, TW, NV, NORM_MODE, GENERAL>(k_in + in_off, k_out + out_off, wk, cr, sr, HD, D,
                                                  rot, eps, lane, neox, ref_round);
  if (v_in != nullptr) copy_row<T, NV>(v_in + in_off, v_out + out_off, HD, lane);
}

template <typename T, typename TW, int NORM_MODE, bool GENERAL>
static int launch_qknorm_nv(bool neox, bool ref_round, int nv, dim3 grid, hipStream_t stream, const void* q_in,
                            const void* k_in, const void* v_in, void* q_out, void* k_out,
                            void* v_out, const void* wq, const void* wk, const float* cos_t,
                            const float* sin_t, int B, int S, int HD, int D, int rot, int64_t is_b,
                            int64_t is_s, int out_seq_offset, int S_total, float eps) {
#define ODIT_QK_CASE(NVV)                                                                         \
  hipLaunchKernelGGL((qknorm_rope_kernel<T, TW, NVV, NORM_MODE, GENERAL>), grid, dim3(256),        \
                     0, stream, static_cast<const T*>(q_in), static_cast<const T*>(k_in),         \
                     static_cast<const T*>(v_in), static_cast<T*>(q_out), static_cast<T*>(k_out), \
                     static_cast<T*>(v_out), static_cast<const TW*>(wq),                          \
                     static_cast<const TW*>(wk), cos_t, sin_t, B, S, HD, D, rot, is_b, is_s,      \
                     out_seq_offset, S_total, eps, neox, ref_round)
  if (nv <= 2) ODIT_QK_CASE(2);
  else if (nv <= 6) ODIT_QK_CASE(6);
  else if (nv <= 10) ODIT_QK_CASE(10);
  else ODIT_QK_CASE(16);
#undef ODIT_QK_CASE
  return check_launch("odit_qknorm_rope");
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
};

int qknorm_rope_bf16(const QkArgs& a);
int qknorm_rope_f16(const QkArgs& a);
int qknorm_rope_f32(const QkArgs& a);

template <typename T, typename TW> static int qk_go(const QkArgs& a) {
  const int64_t toks = static_cast<int64_t>(a.B) * a.S;
  const dim3 grid(static_cast<unsigned>((toks + 3) / 4));
#define ODIT_QK_ARGS                                                                             \
  a.neox, a.ref_round, a.nv, grid, a.stream, a.q_in, a.k_in, a.v_in, a.q_out, a.k_out, a.v_out,  \
      a.wq, a.wk, a.cos, a.sin, a.B, a.S, a.HD, a.D, a.rot, a.is_b, a.is_s, a.out_seq_offset,    \
      a.S_total, a.eps
#define ODIT_QK_MODE(MODE)                                                             \
  return (a.neox || a.ref_round) ? launch_qknorm_nv<T, TW, MODE, true>(ODIT_QK_ARGS)   \
                                 : launch_qknorm_nv<T, TW, MODE, false>(ODIT_QK_ARGS);
  switch (a.norm_mode) {
    case ODIT_NORM_NONE: ODIT_QK_MODE(ODIT_NORM_NONE)
    case ODIT_NORM_HEAD: ODIT_QK_MODE(ODIT_NORM_HEAD)
    default: ODIT_QK_MODE(ODIT_NORM_ROW)
  }
#undef ODIT_QK_MODE
#undef ODIT_QK_ARGS
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
extern "C" int odit_qknorm_rope(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                                void* k_out, void* v_out, const void* wq, const void* wk,
                                const float* cos, const float* sin, int B, int S, int H, int D,
                                int rot, const int64_t in_strides[2], int out_seq_offset,
                                int S_total, float eps, int norm_mode, int w_dtype, int dtype,
                                unsigned flags, void* stream) {
  using namespace odit;
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
  if (nv > 16) {
    set_error("odit_qknorm_rope: H*D=%lld exceeds the %d elements one wavefront keeps in registers",
              static_cast<long long>(HD), 16 * 64 * epv);
    return ODIT_ENOTSUP;
  }
  if (B == 0 || S == 0) return ODIT_OK;
  QkArgs a;
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
  switch (dtype) {
    case ODIT_BF16: return qknorm_rope_bf16(a);
    case ODIT_F16: return qknorm_rope_f16(a);
    default: return qknorm_rope_f32(a);
  }
}
#endif
