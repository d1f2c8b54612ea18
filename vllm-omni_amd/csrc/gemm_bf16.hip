// bf16 GEMM y = x W^T for projections with few rows (M of a few hundred: the text stream), where a
// tile-per-workgroup launch leaves most of the 256 CUs idle or badly balanced.
//
// Work split ("stream-K"): the output is cut into 128 x 192 tiles and every tile's reduction into steps
// of 64 elements. The workgroups come in groups of m_tiles (one per row tile); the steps of all feature
// tiles, laid end to end, are dealt out in equal contiguous ranges to the groups, so that every CU has
// the same number of steps whatever the shape. The workgroups of a group sit on one XCD and walk the
// same (feature tile, step) pairs side by side: a piece of W comes from memory once and is found in that
// XCD's L2 by the others. A range covers the tail of one feature tile, maybe whole tiles, and the head
// of another. A tile finished by one workgroup alone goes straight through the epilogue. Otherwise a
// contributor that finds the tile's counter short of full leaves its fp32 partial tile in a scratch slot
// (write-through stores) and takes a ticket; the last arriver adds the partial tiles in workgroup order
// (its own, still in registers, in its place: the sum does not depend on who arrives last), runs the
// epilogue and resets the counter. Nobody waits for anybody. A ticket word is (epoch << 16 | tickets): a
// contributor first raises the word to this launch's epoch with an atomic maximum, so what an earlier
// launch left there (one that never finished, say) cannot be mistaken for this launch's tickets.
//
// Workgroup: 8 wavefronts = 2 halves of each step's reduction x 4 corners (64 x 96) of the tile; a wave
// holds 3 x 2 accumulators of v_mfma_f32_32x32x16_bf16 (W rows as the A operand, x rows as B: a lane
// ends up with one row m of the output and 4 x 4 consecutive features n). Two waves per SIMD cover each
// other's LDS latency and tile-load issue. When the range ends the two halves meet through LDS, each
// wave keeping three of the six accumulators.
//
// Tile movement: a pipeline step is a 128 x 64 piece of x and a 192 x 64 piece of W, 128-byte rows,
// moved from global memory straight into LDS by `buffer_load_dwordx4 ... lds` (one wave instruction
// fills 1 KB = 8 rows; lane l's 16 bytes land at base + 16 l, so the lane chooses WHAT to fetch:
// the 16-byte chunk (l % 8) ^ ((row >> 1) & 7) of its row, which makes the 16-byte fragment reads of
// 16 consecutive rows cover all 64 banks). Four LDS stages of 40 KB: the loads of step i + 3 are issued
// while step i is multiplied. One barrier per step.
//
// What bounds it. Per step a CU moves 40 KB into LDS and reads 80 KB of fragments back for 768 cycles
// of matrix work per SIMD: 156 bytes per cycle against an LDS that moves 128, so the step cannot take
// less than 940 cycles, and every piece of W is fetched by m_tiles workgroups and every piece of x by
// all feature tiles (378 MB through the L2s for M=512, N=9216, K=3072). Larger tiles would ease both
// but leave a 512-row problem with too few tiles to balance without far more partial-tile traffic.
// Measured at M=512 (cold weights): 0.84 us per step; N=3072, K=12288 in 58 us against 72 us for the
// library's best kernel, N=9216, K=3072 in 52 us against 43 us.
#include "gemm_epilogue.h"

namespace odit {

namespace {

constexpr int kStages = 4;  // LDS stages; kStages - 1 steps of loads are in flight
constexpr int kXTileBytes = kGemmBM * kGemmBK * 2;   // 16 KB
constexpr int kWTileBytes = kGemmBN * kGemmBK * 2;   // 24 KB
constexpr int kStageBytes = kXTileBytes + kWTileBytes;
constexpr int kInstPerStage = kStageBytes / 1024;     // 40 wave instructions per step
constexpr int kWaves = 8;
constexpr int kIPW = kInstPerStage / kWaves;          // 5 per wavefront
constexpr int kXInst = kXTileBytes / 1024;            // the first 16 fill the x piece
constexpr int kSlotFloats = kGemmBM * kGemmBN;
static_assert(kInstPerStage % kWaves == 0, "tile loads must divide evenly over the wavefronts");

struct GemmParams {
  const void *x, *w;
  int M, N, K;
  int64_t ldx, ldw;
  GemmEpilogue ep;
  uint32_t x_bytes, w_bytes;
  int m_tiles, k_steps, workers, groups;
  int64_t total_steps;  // per group: feature tiles x reduction steps
  unsigned long long* counters;  // one ticket word per output tile: (epoch << 16 | tickets drawn), zero between launches
  unsigned long long epoch;      // larger than that of any earlier launch of the process
  float* slots;
};

typedef __attribute__((address_space(3))) void* lds_void_p;

// worker whose range [v S / W, (v + 1) S / W) holds `step`
__device__ __forceinline__ int worker_of(int64_t step, int64_t S, int W) {
  return static_cast<int>(((step + 1) * W - 1) / S);
}

__global__ __launch_bounds__(kWaves * 64, 1) void gemm_bf16_streamk_kernel(const GemmParams p) {
  using M = Mma<bf16_t>;
  using frag = typename M::frag;
  __shared__ __attribute__((aligned(1024))) char lds[kStages * kStageBytes];
  int* const flag = reinterpret_cast<int*>(lds + kStages * kStageBytes - 16);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in a scalar register
  const int l32 = lane & 31, hh = lane >> 5;
  const int kh = wave >> 2, w4 = wave & 3;  // half of each step's reduction, corner of the tile
  const int wm = w4 & 1, wn = w4 >> 1;
  const int lrow = lane >> 3, lpc = lane & 7;

  // the m_tiles workgroups of a group walk the same range of (feature tile, reduction step) pairs, one
  // row tile each, side by side on one XCD: a piece of W is fetched from memory once and found in that
  // XCD's L2 by the others
  const int v = xcd_remap(blockIdx.x, p.workers);
  const int group = v / p.m_tiles, mt = v - group * p.m_tiles;
  const int64_t S = p.total_steps;
  int64_t s = group * S / p.groups;
  const int64_t s_end = (group + 1) * S / p.groups;

  auto make_rsrc = [](const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4_v r;
    r.x = static_cast<uint32_t>(a); r.y = static_cast<uint32_t>(a >> 32) & 0xffffu; r.z = bytes; r.w = 0x00020000u;
    return r;
  };
  const u32x4_v xrsrc = make_rsrc(p.x, p.x_bytes);
  const u32x4_v wrsrc = make_rsrc(p.w, p.w_bytes);
  // instruction q = wave * kIPW + i of a step fills LDS bytes [q KB, q KB + 1 KB) of the stage: q < 16 is x
  const int q0 = wave * kIPW;

  // fragment (sub-tile t, k16 step ks) of a piece: row 32 t + l32, logical chunk 2 ks + hh
  const int frag_lane = l32 * 128 + ((hh ^ ((l32 >> 1) & 7)) << 4);

  while (s < s_end) {
    const int t = static_cast<int>(s / p.k_steps);  // feature tile
    const int kk0 = static_cast<int>(s - static_cast<int64_t>(t) * p.k_steps);
    const int nk = static_cast<int>((p.k_steps - kk0) < (s_end - s) ? (p.k_steps - kk0) : (s_end - s));
    const int m0 = mt * kGemmBM, n0 = t * kGemmBN;

    // per-lane byte offsets of the chunks this lane moves (rows past the end re-read the last row:
    // their products land in output rows / features that are never stored)
    uint32_t voff[kIPW];
#pragma unroll
    for (int i = 0; i < kIPW; ++i) {
      const int q = q0 + i;
      const bool isx = q < kXInst;
      const int r = (isx ? q : q - kXInst) * 8 + lrow;
      int rg = isx ? m0 + r : n0 + r;
      const int last = isx ? p.M - 1 : p.N - 1;
      rg = rg < last ? rg : last;
      const uint32_t ldb = static_cast<uint32_t>((isx ? p.ldx : p.ldw) * 2);
      voff[i] = static_cast<uint32_t>(rg) * ldb + static_cast<uint32_t>((lpc ^ ((r >> 1) & 7)) << 4);
    }

    // instructions [i0, i1) of this wave's share of step kk's tile loads
    auto issue = [&](int kk, int stage, int i0, int i1) {
#if defined(__HIP_DEVICE_COMPILE__)
      const uint32_t soff = static_cast<uint32_t>(kk) * (kGemmBK * 2);
      const uint32_t lds0 =
          static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_p)(lds + stage * kStageBytes + q0 * 1024)));
#pragma unroll
      for (int i = 0; i < kIPW; ++i) {
        if (i < i0 || i >= i1) continue;
        const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds0 + i * 1024);
        const bool isx = q0 + i < kXInst;  // wave-uniform
        const u32x4_v rs = isx ? xrsrc : wrsrc;
        // m0 (the LDS destination of the load) is a reserved register: naming it as clobbered draws a
        // warning per expansion, and leaving it out would hide the write from the compiler
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(m0v), "v"(voff[i]), "s"(rs), "s"(soff)
                     : "memory", "m0");
#pragma clang diagnostic pop
      }
#endif
    };

    f32x16_v acc[3][2];
#pragma unroll
    for (int tn = 0; tn < 3; ++tn)
#pragma unroll
      for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[tn][tm][e] = 0.f;

    __syncthreads();  // every wave has left the LDS uses of the previous segment
#pragma unroll
    for (int d = 0; d < kStages - 1; ++d)
      if (d < nk) issue(kk0 + d, d, 0, kIPW);
    int stage = 0;
    for (int i = 0; i < nk; ++i) {
      // the loads of step i have landed (those of later steps may still be in flight) ...
      const int ahead = nk - 1 - i < kStages - 2 ? nk - 1 - i : kStages - 2;  // later steps already issued
      if (ahead >= 2) {
        asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
      } else if (ahead == 1) {
        asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      // ... in every wave, and every wave is done with the stage that the next loads overwrite
      __builtin_amdgcn_s_barrier();
      const int st_new = stage == 0 ? kStages - 1 : stage - 1;  // (stage + kStages - 1) % kStages
      const bool more = i + kStages - 1 < nk;
      const char* xb = lds + stage * kStageBytes + wm * (64 * 128);
      const char* wb = lds + stage * kStageBytes + kXTileBytes + wn * (96 * 128);
      // This wave multiplies k16 steps 2 kh and 2 kh + 1 of the piece; the fragments of the second are
      // read while the six MFMAs of the first run, and the wave's five tile-load instructions for step
      // i + kStages - 1 go out in between (issued in one burst they hold the wave up for longer than
      // the matrix pipe has work queued).
      frag xf[2][2], wf[2][3];
      auto fetch = [&](int kq) {
        const int kx = (2 * kh + kq) * 32;
#pragma unroll
        for (int tm = 0; tm < 2; ++tm)
          xf[kq][tm] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(xb + tm * (32 * 128) + (frag_lane ^ kx)));
#pragma unroll
        for (int tn = 0; tn < 3; ++tn)
          wf[kq][tn] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(wb + tn * (32 * 128) + (frag_lane ^ kx)));
      };
      fetch(0);
#pragma unroll
      for (int kq = 0; kq < 2; ++kq) {
        if (kq == 0) fetch(1);
#pragma unroll
        for (int tn = 0; tn < 3; ++tn)
#pragma unroll
          for (int tm = 0; tm < 2; ++tm) acc[tn][tm] = M::run(wf[kq][tn], xf[kq][tm], acc[tn][tm]);
        if (more) issue(kk0 + i + kStages - 1, st_new, kq == 0 ? 0 : 3, kq == 0 ? 3 : kIPW);
        __builtin_amdgcn_sched_barrier(0);
      }
      stage = stage == kStages - 1 ? 0 : stage + 1;
    }
    s += nk;

    // ---- the two halves of the reduction meet: each wave keeps three of the six accumulators ----
    // wave (kh, w4) owns accumulators 3 kh .. 3 kh + 2 (index 2 tn + tm), gives the other three to its
    // partner through LDS and adds the partner's three to its own
    f32x16_v own[3];
    {
      __syncthreads();  // the stages are idle from here
      f32x4_v* xch = reinterpret_cast<f32x4_v*>(lds);  // [w4][giver kh][3][4 g][64 lanes] x 16 bytes
      auto give = [&](int sl, const f32x16_v& a) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4_v q;
#pragma unroll
          for (int u = 0; u < 4; ++u) q[u] = a[g * 4 + u];
          xch[(((w4 * 2 + kh) * 3 + sl) * 4 + g) * 64 + lane] = q;
        }
      };
      if (kh == 0) { give(0, acc[1][1]); give(1, acc[2][0]); give(2, acc[2][1]); }
      else         { give(0, acc[0][0]); give(1, acc[0][1]); give(2, acc[1][0]); }
      __syncthreads();
      auto take = [&](int sl, const f32x16_v& a) {
        f32x16_v r;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4_v q = xch[(((w4 * 2 + (kh ^ 1)) * 3 + sl) * 4 + g) * 64 + lane];
#pragma unroll
          for (int u = 0; u < 4; ++u) r[g * 4 + u] = a[g * 4 + u] + q[u];
        }
        return r;
      };
      if (kh == 0) { own[0] = take(0, acc[0][0]); own[1] = take(1, acc[0][1]); own[2] = take(2, acc[1][0]); }
      else         { own[0] = take(0, acc[1][1]); own[1] = take(1, acc[2][0]); own[2] = take(2, acc[2][1]); }
    }

    // ---- who else works on this tile ----
    const int64_t tile_s0 = static_cast<int64_t>(t) * p.k_steps;
    const int v_first = worker_of(tile_s0, S, p.groups);  // first and last group on this feature tile
    const int v_last = worker_of(tile_s0 + p.k_steps - 1, S, p.groups);
    if (v_first != v_last) {
      // slot 0 of a workgroup is for the tile its range starts in, slot 1 for any later one;
      // layout of a slot: [w4][accumulator 0..5][16][64 lanes]
      auto slot_of = [&](int j) {
        const int first_tile = static_cast<int>((j * S / p.groups) / p.k_steps);
        return p.slots + (static_cast<size_t>(2 * (j * p.m_tiles + mt) + (first_tile == t ? 0 : 1))) * kSlotFloats;
      };
      const int lane_off = (w4 * 6 + kh * 3) * (16 * 64) + lane;
      unsigned long long* ctr = p.counters + t * p.m_tiles + mt;
      const unsigned long long full = (p.epoch << 16) + static_cast<unsigned>(v_last - v_first);
      // When every other contributor has already taken its ticket this workgroup is the last arriver
      // and keeps its partial tile in registers; otherwise the tile goes to the slot first and the
      // ticket is taken after it (whoever then holds the last ticket reduces).
      if (tid == 0)
        *reinterpret_cast<volatile int*>(flag) =
            __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == full ? 1 : 0;
      __syncthreads();
      const bool known_last = *reinterpret_cast<volatile int*>(flag) != 0;
      __syncthreads();  // the flag is read before it is written again
      if (known_last) {
        if (tid == 0) __hip_atomic_store(ctr, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        float* mine = slot_of(group) + lane_off;
#pragma unroll
        for (int sl = 0; sl < 3; ++sl)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            __hip_atomic_store(mine + (sl * 16 + e) * 64, own[sl][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0);  // the partial tile has reached memory before the ticket is taken
        __syncthreads();
        if (tid == 0) {
          // two atomics of one thread on one address: applied in program order
          __hip_atomic_fetch_max(ctr, p.epoch << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const unsigned long long ticket = __hip_atomic_fetch_add(ctr, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const int last = ticket == full;
          if (last) __hip_atomic_store(ctr, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          *reinterpret_cast<volatile int*>(flag) = last;
        }
        __syncthreads();
        if (*reinterpret_cast<volatile int*>(flag) == 0) continue;
      }
      // last arriver: partial tiles in workgroup order (its own, still in registers, in its place), one
      // contributor per round trip
      f32x16_v sum[3];
      bool started = false;
      for (int j = v_first; j <= v_last; ++j) {
        if (j == group) {
#pragma unroll
          for (int sl = 0; sl < 3; ++sl)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum[sl][e] = started ? sum[sl][e] + own[sl][e] : own[sl][e];
        } else {
          const float* theirs = slot_of(j) + lane_off;
          float part[48];
#pragma unroll
          for (int e = 0; e < 48; ++e)
            part[e] = __hip_atomic_load(theirs + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int sl = 0; sl < 3; ++sl)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum[sl][e] = started ? sum[sl][e] + part[sl * 16 + e] : part[sl * 16 + e];
        }
        started = true;
      }
#pragma unroll
      for (int sl = 0; sl < 3; ++sl) own[sl] = sum[sl];
    } else {
      __syncthreads();  // the exchange area is read out before the epilogue reuses it
    }

    // ---- epilogue ----
    // A lane holds one output row and 4 x 4 features per accumulator: stored from there, every wave
    // instruction would touch 32 output rows with 16 bytes each. Each 64 x 96 corner goes through LDS
    // instead (fp32, 100 floats per row: the 16-byte writes of 16 rows cover all banks) and leaves as
    // 16-byte pieces of 8 features, 12 consecutive lanes per output row; bias, activation, gate and
    // residual are applied on the way out, where their loads are row-contiguous too.
    {
      constexpr int kPitch = 100;
      float* stg = reinterpret_cast<float*>(lds) + w4 * (64 * kPitch);
#pragma unroll
      for (int sl = 0; sl < 3; ++sl) {
        const int si = kh * 3 + sl, tn = si >> 1, tm = si & 1;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4_v q;
#pragma unroll
          for (int u = 0; u < 4; ++u) q[u] = own[sl][g * 4 + u];
          *reinterpret_cast<f32x4_v*>(stg + (tm * 32 + l32) * kPitch + tn * 32 + g * 8 + hh * 4) = q;
        }
      }
      __syncthreads();  // a corner is written by two waves and read by the same two
#pragma unroll 3
      for (int it = 0; it < 6; ++it) {
        const int idx = (kh * 6 + it) * 64 + lane;
        const int row = idx / 12, ch = idx - row * 12;
        const int m = m0 + wm * 64 + row;
        const int n = n0 + wn * 96 + ch * 8;
        const f32x4_v lo = *reinterpret_cast<const f32x4_v*>(stg + row * kPitch + ch * 8);
        const f32x4_v hi = *reinterpret_cast<const f32x4_v*>(stg + row * kPitch + ch * 8 + 4);
        if (m >= p.M || n >= p.N) continue;
        float y[8];
#pragma unroll
        for (int u = 0; u < 4; ++u) { y[u] = lo[u]; y[4 + u] = hi[u]; }
        gemm_epilogue_store8(p.ep, m, n, y);
      }
    }
  }
}

}  // namespace

int device_cus() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cus[dev] = n;
  }
  return cus[dev];
}

void gemm_streamk_shape(int M, int N, int K, int cus, int* workers, int* steps_per_worker, int* tiles) {
  const int m_tiles = (M + kGemmBM - 1) / kGemmBM, n_tiles = (N + kGemmBN - 1) / kGemmBN;
  const int64_t total = static_cast<int64_t>(n_tiles) * (K / kGemmBK);  // steps of one row tile
  int64_t groups = (cus < kGemmMaxWorkers ? cus : kGemmMaxWorkers) / m_tiles;
  if (groups < 1) groups = 1;
  if (total < groups) groups = total;
  *workers = static_cast<int>(groups) * m_tiles;
  *steps_per_worker = static_cast<int>((total + groups - 1) / groups);
  *tiles = m_tiles * n_tiles;
}

bool gemm_streamk_takes(const GemmCall& c, int dtype) {
  if (dtype != ODIT_BF16) return false;
  if (c.M < 64 || c.M > 1024 || c.K % kGemmBK != 0 || c.N % 8 != 0) return false;
  if (c.ldx % 8 != 0 || c.ldw % 8 != 0 || c.ldo % 8 != 0) return false;
  if (!aligned16(c.x) || !aligned16(c.w) || !aligned16(c.out)) return false;
  if (c.bias != nullptr && (reinterpret_cast<uintptr_t>(c.bias) & 15u) != 0) return false;
  const bool gated = c.epilogue == ODIT_EPI_GATED_RESIDUAL || c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE;
  if (gated) {
    if (c.residual == nullptr || c.ldr % 8 != 0 || !aligned16(c.residual)) return false;
    if (c.gate != nullptr && (!aligned16(c.gate) || c.ldg % 8 != 0)) return false;
    if (c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE && !c.gate_f32) return false;
  }
  const uint64_t xb = (static_cast<uint64_t>(c.M - 1) * c.ldx + c.K) * 2, wb = (static_cast<uint64_t>(c.N - 1) * c.ldw + c.K) * 2;
  if (xb >= (1ull << 32) || wb >= (1ull << 32)) return false;
  const int64_t tiles = static_cast<int64_t>((c.M + kGemmBM - 1) / kGemmBM) * ((c.N + kGemmBN - 1) / kGemmBN);
  return tiles * sizeof(unsigned long long) <= kGemmCounterBytes;
}

int launch_gemm_streamk(const GemmCall& c, void* scratch, hipStream_t stream) {
  const int cus = device_cus();
  if (cus <= 0) { set_error("odit_linear: cannot read the device's compute-unit count"); return ODIT_ELAUNCH; }
  GemmParams p;
  p.x = c.x; p.w = c.w;
  p.M = c.M; p.N = c.N; p.K = c.K;
  p.ldx = c.ldx; p.ldw = c.ldw;
  p.ep = gemm_epilogue_of(c);
  p.x_bytes = static_cast<uint32_t>((static_cast<uint64_t>(c.M - 1) * c.ldx + c.K) * 2);
  p.w_bytes = static_cast<uint32_t>((static_cast<uint64_t>(c.N - 1) * c.ldw + c.K) * 2);
  p.m_tiles = (c.M + kGemmBM - 1) / kGemmBM;
  p.k_steps = c.K / kGemmBK;
  int spw = 0, tiles = 0;
  gemm_streamk_shape(c.M, c.N, c.K, cus, &p.workers, &spw, &tiles);
  p.groups = p.workers / p.m_tiles;
  p.total_steps = static_cast<int64_t>(tiles / p.m_tiles) * p.k_steps;
  p.counters = static_cast<unsigned long long*>(scratch);
  p.epoch = next_ticket_epoch();
  p.slots = reinterpret_cast<float*>(static_cast<char*>(scratch) + kGemmCounterBytes);
  hipLaunchKernelGGL(gemm_bf16_streamk_kernel, dim3(p.workers), dim3(kWaves * 64), 0, stream, p);
  return check_launch("odit_linear (stream-K kernel)");
}

}  // namespace odit
