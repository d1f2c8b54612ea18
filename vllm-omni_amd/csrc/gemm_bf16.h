// Hand-written bf16 GEMM for projections with few rows (the text stream of a dual-stream block):
// interface between linear.hip (problem checks, dispatch) and gemm_bf16.hip (the kernel).
#pragma once

#include "odit_common.h"

namespace odit {

// y[M,N] = epilogue(x[M,K] W[N,K]^T); the epilogue codes are those of odit_linear.
struct GemmCall {
  const void *x, *w, *bias, *residual, *gate;
  void* out;
  int M, N, K;
  int64_t ldx, ldw, ldo, ldr;
  int epilogue;       // enum odit_epilogue
  int gate_f32;       // gate (and, in the pre-scaled form, bias) are float32
  int rows_per_gate;  // consecutive rows that share one gate vector (0 = all rows)
  int64_t ldg;        // elements between consecutive gate vectors (and pre-scaled bias vectors)
};

constexpr int kGemmBM = 128;  // rows of x per output tile
constexpr int kGemmBN = 192;  // rows of W (output features) per output tile
constexpr int kGemmBK = 64;   // reduction elements per pipeline step

// scratch of the kernel: one 64-bit ticket word per output tile, then two partial-tile slots per workgroup
constexpr size_t kGemmCounterBytes = 32768;
constexpr size_t kGemmSlotBytes = static_cast<size_t>(kGemmBM) * kGemmBN * sizeof(float);
constexpr int kGemmMaxWorkers = 256;
constexpr size_t kGemmScratchBytes = kGemmCounterBytes + 2 * kGemmMaxWorkers * kGemmSlotBytes;

// whether the kernel takes this problem (bf16, K a multiple of 64, N of 8, 64 <= M <= 1024, 16-byte
// aligned rows, operands addressable with 32-bit byte offsets)
bool gemm_streamk_takes(const GemmCall& c, int dtype);

// `scratch` (kGemmScratchBytes, 256-byte aligned): its first kGemmCounterBytes must have been zero-filled
// once; they are zero again when the kernel has finished, and what an unfinished launch left there is
// overridden by the next launch (its ticket words carry a larger epoch).
int launch_gemm_streamk(const GemmCall& c, void* scratch, hipStream_t stream);

// workgroups the launch would use and the reduction steps each of them runs
void gemm_streamk_shape(int M, int N, int K, int device_cus, int* workers, int* steps_per_worker, int* tiles);

// compute units of the current device (0 when it cannot be read)
int device_cus();

// ---- gemm_bf16_tile.hip: one 256 x 256 (or 256 x 192) output tile per workgroup, for many rows -------
// whether the kernel takes this problem (bf16, K a multiple of 64, N of 8, 16-byte aligned rows,
// operands addressable with 32-bit byte offsets); it needs no scratch
bool gemm_tile_takes(const GemmCall& c, int dtype);
int launch_gemm_tile(const GemmCall& c, int device_cus, hipStream_t stream);
// features per tile (256 or 192: whichever fills the last round of workgroups better) and tiles of a launch
int gemm_tile_plan(int M, int N, int device_cus, int* tile_n, int* tiles);

}  // namespace odit
