// Types shared by the attention kernels: MFMA wrappers, launch parameters, workgroup-id remap.
#pragma once

#include "odit_common.h"

namespace odit {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_v;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_v;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_v;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_v;
typedef uint32_t u32x4_v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_v __attribute__((ext_vector_type(2)));
typedef float f32x4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_v;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_v;

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  using frag = bf16x8_v;
  static __device__ __forceinline__ f32x16_v run(frag a, frag b, f32x16_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const f32x2_v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_v));  // v_cvt_pk_bf16_f32
  }
};
template <> struct Mma<f16_t> {
  using frag = f16x8_v;
  static __device__ __forceinline__ f32x16_v run(frag a, frag b, f32x16_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const f32x2_v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2_v));
  }
};

struct AttnParams {
  const void* q; const void* k; const void* v; void* o;
  const uint8_t* mask; float* lse;
  int B, Sq, Sk, H, Hkv;
  int64_t qs_b, qs_s, qs_h, ks_b, ks_s, ks_h, vs_b, vs_s, vs_h, os_b, os_s, os_h;
  float scale, scale_log2;
  int n_qblocks, total_blocks;
  // optional second output: query rows >= q_split are written to o_tail[row - q_split]
  void* o_tail; int q_split;
  int64_t ts_b, ts_s, ts_h;
  // optional second value tensor: key rows >= k_split take their values from v_tail[row - k_split]
  // (same row stride as v; only the software-pipelined kernel of attn_fwd_dma.hip reads it)
  const void* v_tail; int k_split;
  int64_t vt_b, vt_h;
  // key-split tail (attn_fwd_dma.hip): workgroup ids < n_full own a whole (q-block, head, batch) unit;
  // the remaining units are cut into key_chunks ranges of tiles_per_chunk key tiles each, one
  // workgroup per range, which leave unnormalised partial results in `ws` for the merge kernel
  int n_full, key_chunks, tiles_per_chunk;
  float* ws;
  // persistent form (attn_fwd_dma.hip): one ticket word per XCD, 64 bytes apart, from which its workgroups draw
  // their next unit: (epoch << 24 | tickets drawn), zero between launches; epoch = number of this launch,
  // larger than that of any earlier launch of the process
  unsigned long long* queue;
  unsigned long long epoch;
};

constexpr size_t kAttnQueueBytes = 1024;  // head of the workspace: the ticket words of the persistent form

// address of output row `row` of (batch b, head h): head of the joint sequence in `o`, tail in `o_tail`
template <typename T>
__device__ __forceinline__ T* out_row_ptr(const AttnParams& p, int b, int h, int row) {
  if (p.o_tail != nullptr && row >= p.q_split)
    return static_cast<T*>(p.o_tail) + b * p.ts_b + h * p.ts_h + static_cast<int64_t>(row - p.q_split) * p.ts_s;
  return static_cast<T*>(p.o) + b * p.os_b + h * p.os_h + static_cast<int64_t>(row) * p.os_s;
}

constexpr int kNumXcd = 8;

// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; give every XCD a contiguous
// range of logical ids instead, so neighbours in (q-block, head) order share an L2.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  const int xcd = bid % kNumXcd, local = bid / kNumXcd;
  const int per = total / kNumXcd, rem = total % kNumXcd;
  return xcd * per + (xcd < rem ? xcd : rem) + local;
}


// software-pipelined kernel with direct global->LDS tile loads (attn_fwd_dma.hip); returns
// ODIT_ENOTSUP when the tensors cannot be addressed with 32-bit buffer offsets
// `ws` (may be null) is scratch for the key-split tail; see attn_dma_workspace_bytes.
int launch_attn_dma(AttnParams& p, int dtype, int D, hipStream_t stream, void* ws, size_t ws_bytes);

// bytes of scratch with which launch_attn_dma can split the last, partly filled round of workgroups
// along the keys (0 when this shape gains nothing from it)
size_t attn_dma_workspace_bytes(int B, int Sq, int Sk, int H, int D);


// whether launch_attn_dma takes a problem of head size D with these key/value row strides (elements)
bool attn_dma_addressable(int Sk, int D, int64_t k_seq_stride, int64_t v_seq_stride);

// text description of the launches launch_attn_dma makes for a shape; returns their number
int attn_dma_plan(int B, int Sq, int Sk, int H, int D, bool with_workspace, char* text, size_t text_bytes);

}  // namespace odit
