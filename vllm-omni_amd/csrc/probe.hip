// Calibration probe for the roofline: the sustained rate of v_mfma_f32_32x32x16_bf16 with nothing else
// in the loop (operands and accumulators in registers, two wavefronts per SIMD), for two kinds of
// operand data. The matrix pipe of this part is power-limited: with constant operands it sustains about
// 2.2 PFLOP/s, with random operands (what activations look like) about 1.6 PFLOP/s, against the
// 2.5 PFLOP/s that 256 CUs x 4 SIMDs x one 32-cycle MFMA at 2.4 GHz would give. A kernel's fraction
// of the nominal peak has to be read against these.
//
// Built into a library of its own (libomni_dit_probe.so): a measurement aid for bench.py, not part of the
// product's C ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace odit {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float probe_f32x16;

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

template <bool RANDOM>
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
  probe_bf16x8 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (RANDOM) {  // random sign and mantissa, exponent within +-2 of 1.0
        uint32_t h = probe_hash(threadIdx.x * 131u + blockIdx.x * 7919u + j * 17u + i);
        a[j][i] = (__bf16)__uint_as_float(((h & 1u) << 31) | ((124u + (h >> 1) % 5u) << 23) | ((h >> 9) & 0x7f0000u));
        h = probe_hash(h);
        b[j][i] = (__bf16)__uint_as_float(((h & 1u) << 31) | ((124u + (h >> 1) % 5u) << 23) | ((h >> 9) & 0x7f0000u));
      } else {
        a[j][i] = (__bf16)1.0f;
        b[j][i] = (__bf16)0.5f;
      }
    }
  probe_f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 8; ++m)
      acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m & 3], b[(m + 1) & 3], acc[m & 3], 0, 0, 0);
    if ((it & 255) == 255) {  // keep the accumulators finite
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] *= 1e-3f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[j][e];
  sink[static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x] = s;
}

}  // namespace odit

// Launches `workgroups` workgroups of 8 wavefronts that issue nothing but v_mfma_f32_32x32x16_bf16
// (iters x 8 per wavefront) on register operands holding constant (random_operands = 0) or pseudo-random
// data, writes one float per thread to `sink` (workgroups * 512 floats) and returns the flop count of the
// launch in *flop. Timed by the caller with events on `stream`. Returns 0, -1 (bad argument) or -3 (launch).
extern "C" int odit_probe_mfma(int random_operands, int iters, int workgroups, float* sink, double* flop, void* stream) {
  using namespace odit;
  if (iters <= 0 || workgroups <= 0 || sink == nullptr) return -1;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (random_operands) {
    hipLaunchKernelGGL(probe_mfma_kernel<true>, dim3(workgroups), dim3(512), 0, st, sink, iters);
  } else {
    hipLaunchKernelGGL(probe_mfma_kernel<false>, dim3(workgroups), dim3(512), 0, st, sink, iters);
  }
  if (flop) *flop = static_cast<double>(workgroups) * 8 /*waves*/ * iters * 8 /*MFMAs*/ * 32768.0;
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
