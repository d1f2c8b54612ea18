// The elementwise tail of the hand-written GEMM kernels: what happens to 8 consecutive output features of
// one row on their way from the fp32 accumulators to memory (bias, GELU(tanh), gate, residual, rounding).
// Shared by the stream-K kernel for few rows (gemm_bf16.hip) and the tile kernel for many (gemm_bf16_tile.hip).
#pragma once

#include "attn_common.h"
#include "gemm_bf16.h"

namespace odit {

struct GemmEpilogue {
  const void *bias, *residual, *gate;
  void* out;
  int M, N;
  int64_t ldo, ldr, ldg;
  int epilogue, gate_f32, rows_per_gate;
};

__device__ __forceinline__ float gemm_gelu_tanh(float x) {
  const float u = 0.7978845608028654f * x * fmaf(0.044715f * x, x, 1.f);
  return x / (1.f + __expf(-2.f * u));
}

// y[0..8) = accumulators of row m, features n .. n + 7 (n a multiple of 8, m < M, n < N): applies the
// epilogue and stores 16 bytes
__device__ __forceinline__ void gemm_epilogue_store8(const GemmEpilogue& p, int m, int n, float (&y)[8]) {
  const bf16_t* bias_h = static_cast<const bf16_t*>(p.bias);
  const float* bias_f = static_cast<const float*>(p.bias);
  const bool gelu = p.epilogue == ODIT_EPI_GELU_TANH || p.epilogue == ODIT_EPI_BIAS_GELU_TANH;
  const bool gated = p.epilogue == ODIT_EPI_GATED_RESIDUAL || p.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE;
  const bool pre = p.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE;
  if (gated) {
    const int64_t grow = p.rows_per_gate > 0 ? static_cast<int64_t>(m / p.rows_per_gate) * p.ldg : 0;
    float gt[8], bs[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { gt[u] = 1.f; bs[u] = 0.f; }
    if (p.gate != nullptr) {
      if (p.gate_f32) {
        const float* gp = static_cast<const float*>(p.gate) + grow + n;
        const f32x4_v g0 = *reinterpret_cast<const f32x4_v*>(gp), g1 = *reinterpret_cast<const f32x4_v*>(gp + 4);
#pragma unroll
        for (int u = 0; u < 4; ++u) { gt[u] = g0[u]; gt[4 + u] = g1[u]; }
      } else {
        const u32x4 gv = load_raw(static_cast<const bf16_t*>(p.gate) + grow + n);
#pragma unroll
        for (int u = 0; u < 8; ++u) gt[u] = Raw<bf16_t>::get(gv, u);
      }
    }
    if (p.bias != nullptr) {
      if (pre) {  // float32, already multiplied by the gate, one vector per gate vector
        const float* bp = bias_f + grow + n;
        const f32x4_v b0 = *reinterpret_cast<const f32x4_v*>(bp), b1 = *reinterpret_cast<const f32x4_v*>(bp + 4);
#pragma unroll
        for (int u = 0; u < 4; ++u) { bs[u] = b0[u]; bs[4 + u] = b1[u]; }
      } else {
        const u32x4 bv = load_raw(bias_h + n);
#pragma unroll
        for (int u = 0; u < 8; ++u) bs[u] = gt[u] * Raw<bf16_t>::get(bv, u);
      }
    }
    const u32x4 rv = load_raw(static_cast<const bf16_t*>(p.residual) + m * p.ldr + n);
#pragma unroll
    for (int u = 0; u < 8; ++u) y[u] = fmaf(gt[u], y[u], bs[u]) + Raw<bf16_t>::get(rv, u);
  } else {
    if (p.bias != nullptr) {
      const u32x4 bv = load_raw(bias_h + n);
#pragma unroll
      for (int u = 0; u < 8; ++u) y[u] += Raw<bf16_t>::get(bv, u);
    }
    if (gelu) {
#pragma unroll
      for (int u = 0; u < 8; ++u) y[u] = gemm_gelu_tanh(y[u]);
    }
  }
  u32x4 o;
#pragma unroll
  for (int u = 0; u < 4; ++u) Raw<bf16_t>::set2(o, u, y[2 * u], y[2 * u + 1]);
  store_raw(static_cast<bf16_t*>(p.out) + m * p.ldo + n, o);
}

inline GemmEpilogue gemm_epilogue_of(const GemmCall& c) {
  GemmEpilogue e;
  e.bias = c.bias; e.residual = c.residual; e.gate = c.gate; e.out = c.out;
  e.M = c.M; e.N = c.N; e.ldo = c.ldo; e.ldr = c.ldr; e.ldg = c.ldg;
  e.epilogue = c.epilogue; e.gate_f32 = c.gate_f32; e.rows_per_gate = c.rows_per_gate;
  return e;
}

}  // namespace odit
