// bf16 GEMM y = x W^T for projections with many rows (the image stream: M of several thousand), one
// 256 x 256 (or 256 x 192) output tile per workgroup.
//
// Workgroup: 8 wavefronts, two per SIMD, laid out 4 (rows) x 2 (features); a wave owns 64 rows x 128 (96)
// features = 2 x 4 (2 x 3) accumulators of v_mfma_f32_32x32x16_bf16 with W rows as the A operand, so a lane
// ends up with one output row and 4 x 4 consecutive features per accumulator. Per reduction step of 64 a
// wave reads 6 (5) fragments of 1 KB from LDS for every 8 (6) matrix instructions. (The kernel is a template
// over the wave layout; a 2 x 2 layout of four waves with 128 x 128 corners would read a third less, but its
// 256 accumulator registers fill the accumulation file exactly and the compiler's register allocation then
// falls apart, so only the eight-wave layout is instantiated.)
//
// Tile movement: a step is a 256 x 64 piece of x and a 256 (192) x 64 piece of W, 128-byte rows, moved from
// global memory straight into LDS by `buffer_load_dwordx4 ... lds` (one wave instruction fills 1 KB = 8
// rows; the lane chooses WHAT it fetches: 16-byte chunk (l % 8) ^ ((row >> 1) & 7) of its row, which makes
// the 16-byte fragment reads of 16 consecutive rows cover all 64 banks). Rows past the end of x or W read
// as zeros through the buffer descriptor. Two LDS stages of 64 (56) KB.
//
// Pipeline: ONE barrier per step, placed so that no wave ever waits for LDS behind it. Fragments are read
// one k16 slice ahead of the matrix instructions that consume them, spread over those instructions. When a
// wave has issued the reads of step i's last slice it waits for them (and for its own tile loads of step
// i + 1), then meets the others at the barrier: behind it stage i is free and stage i + 1 is complete, so
// the wave issues the first half of its loads of step i + 2 into stage i, the reads of step i + 1's first
// slice, and only then the matrix instructions of step i's last slice, which cover the latency of both; the
// second half of the loads goes out during the next slice.
//
// Workgroup order: ids are remapped so that the 32 workgroups resident on one XCD at a time form a block of
// 8 row tiles x 4 feature tiles, i.e. fetch 8 pieces of x and 4 of W per step into that XCD's L2 instead of
// 32 of each.
//
// Epilogue: accumulators go through LDS (fp32, 64 features at a time, 68 floats per row: the 16-byte writes
// of 16 rows cover all banks) and leave as 16-byte pieces of 8 features, whole 128-byte lines per row; bias,
// activation, gate and residual are applied on the way out (gemm_epilogue.h).
//
// What bounds it: LDS. A step of a 256 x 256 tile reads 192 KB of fragments and takes 64 KB of tile loads,
// 256 KB through an LDS that moves 128 bytes per cycle, against 2048 cycles of matrix work per SIMD at the
// nominal rate: 125 bytes per cycle, nothing left. Measured at M = 8192, cold weights (us, this kernel /
// hipBLASLt's best): N = 12288, K = 3072 with GELU 574 / 449; N = 9216, K = 3072 431 / 434; N = 3072,
// K = 3072 gated 142 / 118; N = 3072, K = 12288 gated 637 / 427. Timing-only builds on the first problem
// (ODIT_TILE_ABLATE): matrix instructions alone 390, plus fragment reads 483, plus tile loads instead 517,
// tile loads and barrier without any matrix instruction 495 - the two kinds of LDS traffic add up instead of
// hiding behind the matrix pipe. The library's kernel for the same tile runs four waves with 128 x 128 corners
// (128 KB of fragment reads per step) at 76 % matrix-pipe busy against 56 % here. That layout was also built with
// the 256 accumulators at fixed accumulation registers named in one-instruction inline assembly (no register
// allocation problem left: 102 vector registers, no scratch, same results): 560 us with the tile loads going
// through registers, 610 direct to LDS, and 405 us = 1.53 PFLOP/s with no tile traffic at all - the fetches from
// L2, not LDS and not the matrix pipe, are what separates both layouts from the library.
#include <type_traits>

#include "gemm_epilogue.h"

// Timing-only builds (wrong results): bit 0 = no tile loads in the main loop, 1 = no matrix instructions,
// 2 = no barrier, 3 = tile loads never waited for, 4 = no fragment reads in the main loop.
#ifndef ODIT_TILE_ABLATE
#define ODIT_TILE_ABLATE 0
#endif


namespace odit {

namespace {

constexpr int kTileM = 256;                       // rows of x per tile
constexpr int kTileK = 64;                        // reduction elements per step
constexpr int kTileXBytes = kTileM * kTileK * 2;  // 32 KB per stage
constexpr int kEpiPitch = 68;                     // floats per staged row of 64 features
constexpr int kEpiBytes = kTileM * 2 * kEpiPitch * 4;  // 256 rows x two halves of the features, 64 at a time

struct TileParams {
  const void *x, *w;
  int M, N, K;
  int64_t ldx, ldw;
  GemmEpilogue ep;
  uint32_t x_bytes, w_bytes;
  int m_tiles, n_tiles, k_steps, group_m;
};

typedef __attribute__((address_space(3))) void* lds_void_p;

// NT: 32-feature accumulators per wave along the features (the tile is 64 NT features wide: two waves side by
// side); WM: waves along the rows (4: eight waves of 64 rows, two per SIMD; 2: four waves of 128 rows, one per
// SIMD with twice the accumulators, which reads a third less from LDS per matrix instruction).
template <int NT, int WM>
__global__ __launch_bounds__(WM * 2 * 64) __attribute__((amdgpu_waves_per_eu(WM / 2, WM / 2))) void gemm_bf16_tile_kernel(const TileParams p) {
  using M = Mma<bf16_t>;
  using frag = typename M::frag;
  constexpr int kTileWaves = WM * 2;
  constexpr int TM = 8 / WM;                  // 32-row accumulators per wave along the rows
  constexpr int BN = 64 * NT;                 // features per tile
  constexpr int WBytes = BN * kTileK * 2;
  constexpr int Stage = kTileXBytes + WBytes;
  constexpr int NInst = Stage / 1024;         // wave instructions per step (64 or 56)
  constexpr int IPW = NInst / kTileWaves;     // per wavefront (8 or 7)
  constexpr int XInst = kTileXBytes / 1024;   // the first 32 fill the x piece
  constexpr int LdsBytes = 2 * Stage > kEpiBytes ? 2 * Stage : kEpiBytes;
  static_assert(NInst % kTileWaves == 0, "tile loads must divide evenly over the wavefronts");
  __shared__ __attribute__((aligned(1024))) char lds[LdsBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const int wm = wave % WM, wn = wave / WM;
  const int lrow = lane >> 3, lpc = lane & 7;

  // tile of this workgroup: groups of group_m row tiles, feature tiles outer inside a group
  int mt, nt;
  {
    const int L = xcd_remap(blockIdx.x, gridDim.x);
    const int per_group = p.group_m * p.n_tiles;
    const int g = L / per_group;
    const int first_m = g * p.group_m;
    const int gm = p.m_tiles - first_m < p.group_m ? p.m_tiles - first_m : p.group_m;
    const int r = L - g * per_group;
    nt = r / gm;
    mt = first_m + (r - nt * gm);
  }
  const int m0 = mt * kTileM, n0 = nt * BN;

  auto make_rsrc = [](const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4_v r;
    r.x = static_cast<uint32_t>(a); r.y = static_cast<uint32_t>(a >> 32) & 0xffffu; r.z = bytes; r.w = 0x00020000u;
    return r;
  };
  const u32x4_v xrsrc = make_rsrc(p.x, p.x_bytes);
  const u32x4_v wrsrc = make_rsrc(p.w, p.w_bytes);

  // Instruction q = wave * IPW + i of a step fills LDS bytes [q KB, q KB + 1 KB) of the stage: rows
  // 8 q' .. 8 q' + 7 of the x piece (q' = q < 32) or of the W piece (q' = q - 32). Lane l lands in row
  // 8 q' + l / 8, physical chunk l % 8, and fetches logical chunk (l % 8) ^ ((row >> 1) & 7) with
  // (row >> 1) & 7 = 4 (q' & 1) | (l / 8 >> 1): a per-lane row offset per operand plus a chunk offset whose
  // bit 6 follows the parity of q'; the rest of the address (first row of the instruction, reduction step)
  // is scalar.
  const uint32_t ldx2 = static_cast<uint32_t>(p.ldx * 2), ldw2 = static_cast<uint32_t>(p.ldw * 2);
  const uint32_t rowx = static_cast<uint32_t>(lrow) * ldx2, roww = static_cast<uint32_t>(lrow) * ldw2;
  const uint32_t chunk0 = static_cast<uint32_t>((lpc ^ (lrow >> 1)) << 4);  // q' even; odd flips bit 6 (chunk ^ 4)
  uint32_t srow[IPW];  // byte offset of each instruction's first row
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int q = wave * IPW + i;
    const bool isx = q < XInst;
    const int qq = isx ? q : q - XInst;
    srow[i] = isx ? static_cast<uint32_t>(m0 + 8 * qq) * ldx2 : static_cast<uint32_t>(n0 + 8 * qq) * ldw2;
  }
  const int q0 = wave * IPW;

  // instructions [i0, i1) of this wave's share of step kk's tile loads, into stage `stage`
  auto issue = [&](int kk, int stage, int i0, int i1) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t kb = static_cast<uint32_t>(kk) * (kTileK * 2);
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_p)(lds + stage * Stage + q0 * 1024)));
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      if (i < i0 || i >= i1) continue;
      const int q = q0 + i;
      const bool isx = q < XInst;  // wave-uniform
      const int par = (isx ? q : q - XInst) & 1;
      const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds0 + i * 1024);
      const uint32_t soff = __builtin_amdgcn_readfirstlane(srow[i] + kb);
      const u32x4_v rs = isx ? xrsrc : wrsrc;
      const uint32_t vo = (isx ? rowx : roww) + (chunk0 ^ static_cast<uint32_t>(par << 6));
      // m0 (the LDS destination of the load) is a reserved register: naming it as clobbered draws a
      // warning per expansion, and leaving it out would hide the write from the compiler
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   :
                   : "s"(m0v), "v"(vo), "s"(rs), "s"(soff)
                   : "memory", "m0");
#pragma clang diagnostic pop
    }
#endif
  };

  f32x16_v acc[NT][TM];
#pragma unroll
  for (int tn = 0; tn < NT; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[tn][tm][e] = 0.f;

  // fragment (sub-tile t, k16 slice ks) of a piece: row 32 t + l32, logical chunk 2 ks + hh
  const int frag_lane = l32 * 128 + ((hh ^ ((l32 >> 1) & 7)) << 4);
  const int x_off = wm * (32 * TM * 128) + frag_lane;
  const int w_off = kTileXBytes + wn * (32 * NT * 128) + frag_lane;

  frag xf[2][TM], wf[2][NT];
  auto fetch = [&](int stage, int ks, int set) {
    if ((ODIT_TILE_ABLATE & 16) && (ks != 0 || stage != 0)) return;
    const char* xb = lds + stage * Stage;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
      xf[set][tm] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(xb + tm * (32 * 128) + (x_off ^ (ks * 32))));
#pragma unroll
    for (int tn = 0; tn < NT; ++tn)
      wf[set][tn] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(xb + tn * (32 * 128) + (w_off ^ (ks * 32))));
  };
  auto multiply = [&](int set) {
    if (ODIT_TILE_ABLATE & 2) return;
#pragma unroll
    for (int tn = 0; tn < NT; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = M::run(wf[set][tn], xf[set][tm], acc[tn][tm]);
  };

  const int nk = p.k_steps;
  // The reduction starts at a different step in every row tile and wraps around: the rows of x and W are a
  // multiple of 4 KB apart for the usual reduction lengths, so at one reduction offset every row of a tile sits in
  // the same memory channel, and workgroups that all stand at the same offset queue up in front of it. Row tiles
  // 256 bytes (two steps) apart spread over the channels; the feature tiles of one row tile keep the same offset,
  // so they still find each other's x pieces in L2. Worth 0 to 5 % (M = 8192, us without / with: N=9216 K=3072
  // 430 / 406, N=3072 K=12288 630 / 613, N=12288 K=3072 567 / 568); what such strides really cost shows when the
  // rows are padded by 128 bytes instead: 628 -> 509 us at K=12288, 536 -> 506 at K=3072 (hipBLASLt's kernels are
  // indifferent to it). Sums are formed in the rotated order.
  constexpr int kStagger = 32;
  const int stagger = ((mt % kStagger) * 2) % nk;
  auto wrapk = [&](int j) {   // reduction step of the j-th step this workgroup runs (j < nk + 3)
    int t = j + stagger;
    t = t >= nk ? t - nk : t;
    return t >= nk ? t - nk : t;
  };
  // A step's tile loads go out in two halves, each spread over the matrix instructions of one k16 slice (the
  // texture addresser takes a wave instruction every 16 cycles: issued faster, the loads fill its queue and the
  // wave, which issues in order, stalls in front of its next matrix instruction): the first half of step i + 2
  // right after the barrier that frees its stage (slice 3 of step i), the second half in slice 0 of step i + 1.
  constexpr int H0 = (IPW + 1) / 2;  // instructions of the first half
  auto issue_spread = [&](int kk, int stage, int i0, int i1, int part, int parts) {
    const int n = i1 - i0, a = i0 + n * part / parts, b = i0 + n * (part + 1) / parts;
    issue(kk, stage, a, b);
  };
  issue(wrapk(0), 0, 0, IPW);
  if (nk > 1) {
    issue(wrapk(1), 1, 0, H0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(H0) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  fetch(0, 0, 0);

  // one reduction step on stage `stage` (compile-time): slices 0..2, the barrier, then slice 3 in the shadow of
  // which the first fragment reads of step i + 1 are issued.
  auto step = [&](int i, auto stage_c) {
    constexpr int stage = decltype(stage_c)::value;
    const bool next = i + 1 < nk, more = i + 2 < nk;
#pragma unroll
    for (int ks = 0; ks < 3; ++ks) {
      fetch(stage, ks + 1, (ks + 1) & 1);
      if (ks == 0 && !(ODIT_TILE_ABLATE & 1)) {
        // slice 0 carries the second half of step i + 1's tile loads, a few per group of matrix instructions
#pragma unroll
        for (int tn = 0; tn < NT; ++tn) {
          if (next) issue_spread(wrapk(i + 1), stage ^ 1, H0, IPW, tn, NT);
          if (!(ODIT_TILE_ABLATE & 2))
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = M::run(wf[0][tn], xf[0][tm], acc[tn][tm]);
          __builtin_amdgcn_sched_barrier(0);
        }
        continue;
      }
      multiply(ks & 1);
      // the reads of the next slice are spread over the matrix instructions of this one: every wave of the
      // workgroup is at the same point of its step, and a burst of reads from all of them queues up in LDS
      constexpr int R = TM + NT, Q = TM * NT, per_read = Q / R;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, per_read, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, Q - R * per_read, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // the fragments of slice 3 are in registers, and this wave's loads of step i + 1 have landed ...
    if (ODIT_TILE_ABLATE & 8) __builtin_amdgcn_s_waitcnt(0xc07f); else  // lgkmcnt(0) only
    __builtin_amdgcn_s_waitcnt(0);
    // ... in every wave: stage `stage` is free, stage `stage ^ 1` is complete
    if (!(ODIT_TILE_ABLATE & 4)) __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // (after the last step this reads a stage nobody has filled: the values are never used)
    fetch(stage ^ 1, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tn = 0; tn < NT; ++tn) {
      if (more && !(ODIT_TILE_ABLATE & 1)) issue_spread(wrapk(i + 2), stage, 0, H0, tn, NT);
      if (!(ODIT_TILE_ABLATE & 2))
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = M::run(wf[1][tn], xf[1][tm], acc[tn][tm]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  {
    const std::integral_constant<int, 0> s0;
    const std::integral_constant<int, 1> s1;
    for (int i = 0; i < nk; i += 2) {
      step(i, s0);
      if (i + 1 < nk) step(i + 1, s1);
    }
  }

  // ---- epilogue: 64 features of the wave's 64 x (32 NT) corner at a time through its own LDS region ----
  // (every wave is past the last barrier, so no wave reads a stage any more)
  constexpr int WR = 32 * TM;  // rows of the wave's corner
  float* stg = reinterpret_cast<float*>(lds) + wave * (WR * kEpiPitch);
  const int mw = m0 + wm * WR, nw = n0 + wn * (32 * NT);
#pragma unroll
  for (int pass = 0; pass < (NT + 1) / 2; ++pass) {
    constexpr int kFull = 2;
    const int tn0 = pass * kFull;
    const int ntn = NT - tn0 < kFull ? NT - tn0 : kFull;  // 32-feature accumulators in this pass
#pragma unroll
    for (int tn = 0; tn < NT; ++tn) {
      if (tn / kFull != pass) continue;  // resolved at compile time: both loops are unrolled
      const int t = tn % kFull;
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4_v q;
#pragma unroll
          for (int u = 0; u < 4; ++u) q[u] = acc[tn][tm][g * 4 + u];
          *reinterpret_cast<f32x4_v*>(stg + (tm * 32 + l32) * kEpiPitch + t * 32 + g * 8 + hh * 4) = q;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int cpr = 4 * ntn;  // 16-byte output pieces per row
#pragma unroll 4
    for (int it = 0; it < cpr * (WR / 64); ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / cpr, ch = idx - row * cpr;
      const int m = mw + row;
      const int n = nw + tn0 * 32 + ch * 8;
      const f32x4_v lo = *reinterpret_cast<const f32x4_v*>(stg + row * kEpiPitch + ch * 8);
      const f32x4_v hi = *reinterpret_cast<const f32x4_v*>(stg + row * kEpiPitch + ch * 8 + 4);
      if (m >= p.M || n >= p.N) continue;
      float y[8];
#pragma unroll
      for (int u = 0; u < 4; ++u) { y[u] = lo[u]; y[4 + u] = hi[u]; }
      gemm_epilogue_store8(p.ep, m, n, y);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

#ifndef ODIT_TILE_WM
#define ODIT_TILE_WM 4
#endif
#ifndef ODIT_TILE_NT
#define ODIT_TILE_NT (ODIT_TILE_WM == 2 ? 3 : 0)
#endif

// 192-wide tiles when they fill the last round of workgroups better (N = 9216 or 3072 on 256 CUs)
int tile_nt_for(int M, int N, int cus) {
  if (ODIT_TILE_NT != 0) return ODIT_TILE_NT;
  const int64_t mt = (M + kTileM - 1) / kTileM;
  int best = 4;
  int64_t best_cost = -1;
  for (int nt : {4, 3}) {
    const int64_t tiles = mt * ((N + 64 * nt - 1) / (64 * nt));
    const int64_t cost = ((tiles + cus - 1) / cus) * nt;  // rounds x time of one tile
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = nt; }
  }
  return best;
}

}  // namespace

bool gemm_tile_takes(const GemmCall& c, int dtype) {
  if (dtype != ODIT_BF16) return false;
  if (c.M < 1 || c.K % kTileK != 0 || c.N % 8 != 0) return false;
  if (c.ldx % 8 != 0 || c.ldw % 8 != 0 || c.ldo % 8 != 0) return false;
  if (!aligned16(c.x) || !aligned16(c.w) || !aligned16(c.out)) return false;
  if (c.bias != nullptr && (reinterpret_cast<uintptr_t>(c.bias) & 15u) != 0) return false;
  const bool gated = c.epilogue == ODIT_EPI_GATED_RESIDUAL || c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE;
  if (gated) {
    if (c.residual == nullptr || c.ldr % 8 != 0 || !aligned16(c.residual)) return false;
    if (c.gate != nullptr && (!aligned16(c.gate) || c.ldg % 8 != 0)) return false;
    if (c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE && !c.gate_f32) return false;
  }
  // 32-bit byte offsets, with room for the rows of a last, partly filled tile
  const uint64_t xb = (static_cast<uint64_t>(c.M) + kTileM) * c.ldx * 2, wb = (static_cast<uint64_t>(c.N) + 256) * c.ldw * 2;
  if (xb >= (1ull << 32) || wb >= (1ull << 32)) return false;
  const int64_t tiles = static_cast<int64_t>((c.M + kTileM - 1) / kTileM) * ((c.N + 191) / 192);
  return tiles < (1ll << 30);
}

int gemm_tile_plan(int M, int N, int cus, int* tile_n, int* tiles) {
  const int nt = tile_nt_for(M, N, cus > 0 ? cus : 256);
  *tile_n = 64 * nt;
  *tiles = ((M + kTileM - 1) / kTileM) * ((N + 64 * nt - 1) / (64 * nt));
  return nt;
}

int launch_gemm_tile(const GemmCall& c, int cus, hipStream_t stream) {
  TileParams p;
  p.x = c.x; p.w = c.w;
  p.M = c.M; p.N = c.N; p.K = c.K;
  p.ldx = c.ldx; p.ldw = c.ldw;
  p.ep = gemm_epilogue_of(c);
  p.x_bytes = static_cast<uint32_t>((static_cast<uint64_t>(c.M - 1) * c.ldx + c.K) * 2);
  p.w_bytes = static_cast<uint32_t>((static_cast<uint64_t>(c.N - 1) * c.ldw + c.K) * 2);
  int tile_n = 0, tiles = 0;
  const int nt = gemm_tile_plan(c.M, c.N, cus, &tile_n, &tiles);
  p.m_tiles = (c.M + kTileM - 1) / kTileM;
  p.n_tiles = (c.N + tile_n - 1) / tile_n;
  p.k_steps = c.K / kTileK;
  p.group_m = 8;
  constexpr int WM = ODIT_TILE_WM;
  if (nt == 4) {
    hipLaunchKernelGGL((gemm_bf16_tile_kernel<4, WM>), dim3(tiles), dim3(WM * 2 * 64), 0, stream, p);
  } else {
    hipLaunchKernelGGL((gemm_bf16_tile_kernel<3, WM>), dim3(tiles), dim3(WM * 2 * 64), 0, stream, p);
  }
  return check_launch("odit_linear (tile kernel)");
}

}  // namespace odit
