// Key-split tail shared by the attention kernels: how the last, partly filled round of workgroups is cut
// along the keys, and the kernel that merges the partial results.
#pragma once

#include "attn_common.h"

namespace odit {

// Merge of the key-split tail: one wavefront per query row adds the row's key_chunks partial results,
//   O = sum_c 2^((m_c - m) c) O_c / sum_c 2^((m_c - m) c) l_c,   m = max_c m_c,
// and writes the row (and its log-sum-exp) where the unsplit kernel would have.
constexpr int kMergeMaxChunks = 16;  // = kMaxKeyChunks below

template <typename T, int D, int BM>
__global__ __launch_bounds__(256) void attn_merge_kernel(const AttnParams p, int n_parts) {
  using M = Mma<T>;
  const int lane = threadIdx.x & 63;
  const int64_t gr = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);  // (tail unit, row in unit)
  const int unit = static_cast<int>(gr / BM), r = static_cast<int>(gr % BM);
  if (unit >= n_parts / p.key_chunks) return;
  const int pid = p.n_full + unit;
  const int qb = pid % p.n_qblocks, bh = pid / p.n_qblocks;
  const int h = bh % p.H, b = bh / p.H;
  const int row = qb * BM + r;
  if (row >= p.Sq) return;
  const float* ml = p.ws + static_cast<int64_t>(n_parts) * BM * D;
  // every load of the row is issued before the first use: the loop bounds are compile-time (kMergeMaxChunks
  // is the most ranges plan_tail hands out) and the ranges beyond key_chunks are predicated off, so the
  // kernel pays one memory latency, not one per range
  constexpr int EPL = D / 64;  // consecutive elements per lane
  float mc[kMergeMaxChunks], lc[kMergeMaxChunks], part[kMergeMaxChunks][EPL];
#pragma unroll
  for (int cidx = 0; cidx < kMergeMaxChunks; ++cidx) {
    const bool on = cidx < p.key_chunks;
    const int64_t pr = static_cast<int64_t>(unit * p.key_chunks + (on ? cidx : 0)) * BM + r;
    mc[cidx] = on ? ml[pr * 2] : -INFINITY;
    lc[cidx] = on ? ml[pr * 2 + 1] : 0.f;
    const float* src = p.ws + pr * D + lane * EPL;
#pragma unroll
    for (int e = 0; e < EPL; ++e) part[cidx][e] = on ? src[e] : 0.f;
  }
  float m = -INFINITY;
#pragma unroll
  for (int cidx = 0; cidx < kMergeMaxChunks; ++cidx) m = fmaxf(m, mc[cidx]);
  const float m_safe = m == -INFINITY ? 0.f : m;
  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  float l = 0.f;
#pragma unroll
  for (int cidx = 0; cidx < kMergeMaxChunks; ++cidx) {
    // same order of accumulation as a loop over the ranges; weight 0 for an empty or absent range
    const float wgt = cidx < p.key_chunks ? __builtin_amdgcn_exp2f((mc[cidx] - m_safe) * p.scale_log2) : 0.f;
    l = fmaf(wgt, lc[cidx], l);
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = fmaf(wgt, part[cidx][e], acc[e]);
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  T* op = out_row_ptr<T>(p, b, h, row) + lane * EPL;
  if constexpr (EPL == 2) {
    *reinterpret_cast<uint32_t*>(op) = M::pack2(acc[0] * inv, acc[1] * inv);
  } else {
    op[0] = from_float<T>(acc[0] * inv);
  }
  if (p.lse != nullptr && lane == 0)
    p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Sq + row] = l > 0.f ? m * p.scale + __logf(l) : -INFINITY;
}

// How the last round of workgroups is cut along the keys. `slots` workgroups run at once; after
// `units / slots` full rounds, `rem` units are left: when they would occupy at most a quarter of the
// slots, each is cut into as many key ranges as fit the slots (ranges of an even number of tiles, at
// least kMinTilesPerChunk), so the tail takes 1/key_chunks of a round instead of most of one. Measured
// side by side in one process at rem = 96 of 512 slots (the 4352-token, 48-head shape): the unsplit tail
// costs 0.5 of a round (its workgroups have their CUs to themselves), the split one 0.2 of a round plus
// two more launches and the partial results: 471 -> 454 us. At rem = 256 (half the slots, two ranges)
// the split loses, 227 -> 242 us; twice as many, shorter ranges lose as well. Running the key ranges on
// a side stream, concurrently with the full units, gave nothing over the same-stream order.
struct TailPlan { int rem, key_chunks, tiles_per_chunk; };
constexpr int kMinTilesPerChunk = 8;
constexpr int kMaxKeyChunks = kMergeMaxChunks;

// workgroups resident at once: compute units x workgroups per unit (8 / nw for the nw-wave kernels that run
// two wavefronts per SIMD; pass nw = 8 for one workgroup per unit)
inline int device_slots(int nw) {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256 * (8 / nw);
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev] * (8 / nw);
}

#ifndef ODIT_ATTN_TAIL_DIV
#define ODIT_ATTN_TAIL_DIV 4   // split the last round's units by keys when they fill at most 1/4 of the GPU
#endif

inline TailPlan plan_tail(int64_t units, int n_tiles, int slots) {
  TailPlan t{0, 1, n_tiles};
  const int rem = static_cast<int>(units % slots);
  if (rem == 0 || ODIT_ATTN_TAIL_DIV * rem > slots) return t;
  int kc = slots / rem;
  if (kc > kMaxKeyChunks) kc = kMaxKeyChunks;
  if (kc > n_tiles / kMinTilesPerChunk) kc = n_tiles / kMinTilesPerChunk;
  if (kc < 2) return t;
  int tpc = (n_tiles + kc - 1) / kc;
  tpc += tpc & 1;                      // even, so a tile's LDS buffer is still (tile index & 1)
  kc = (n_tiles + tpc - 1) / tpc;      // drop ranges that the rounding emptied
  if (kc < 2) return t;
  t.rem = rem; t.key_chunks = kc; t.tiles_per_chunk = tpc;
  return t;
}

inline size_t tail_ws_bytes(const TailPlan& t, int bm, int D) {
  return t.rem == 0 ? 0 : static_cast<size_t>(t.rem) * t.key_chunks * bm * (D + 2) * sizeof(float);
}


}  // namespace odit
