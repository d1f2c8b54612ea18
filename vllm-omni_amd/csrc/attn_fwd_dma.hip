// K1, production variant: software-pipelined flash attention whose K/V tiles go from global memory
// straight into LDS (buffer_load ... lds), with no staging registers, no LDS store instructions and
// no per-tile address arithmetic.
//
// Tile movement. A tile is 64 keys x D elements, row-major, unpadded (256 B rows for D = 128). One
// `buffer_load_dwordx4 ... lds` of a wavefront fills 1 KB of LDS: lane l's 16 bytes land at
// base + 16*l (measured), so the PLACE is fixed and the lane picks WHAT it fetches. Lane l therefore
// fetches, for tile row r = 4*i + l/16 and physical 16-byte chunk pc = l%16, the logical chunk
// pc ^ f(r): the swizzle lives in the global address. Per-lane byte offsets are computed once; the
// tile index only moves a scalar offset. The buffer descriptor's size is the end of the last valid
// key row, so rows past Sk read as zeros without any clamping.
//   K:  f(r) = r % 16       a quarter-wave (16 key rows, one chunk column) of a ds_read_b128 covers
//                           all 64 banks
//   V:  f(r) = 4 * (r % 4)  the 4 keys x 4 eight-byte words of two ds_read_b64_tr_b16 groups cover
//                           all 64 banks
// Fragment addresses then are (per-lane base) XOR (a compile-time constant) plus an immediate.
//
// Everything else (transposed S^T = K Q^T / O^T = V^T P^T formulation, one query per lane, lazy
// rescale, stage A = next-tile QK^T MFMAs interleaved with this tile's exp2 work, stage B = PV, one
// barrier per tile - two in the anti-phase form of 8 wavefronts, see NW below -, XCD-aware workgroup order)
// is as in attn_fwd_pipe_kernel.
//
// Persistent form (MODE 2), a measurement aid that no default launch uses (ODIT_ATTN_PERSISTENT=1 in the
// environment turns it on for launches of 4-wavefront workgroups, i.e. with ODIT_ATTN_WAVES=4 at head size 128). With more units than workgroup slots the launch has as many workgroups as run at
// once, and each runs unit after unit as ONE stream of key tiles: the tile pipeline runs across the unit
// boundary. Units are handed out dynamically: every XCD owns a contiguous eighth of the units (neighbours in
// (q block, head) order share keys and values in its L2), its workgroups start on the first ones and draw the
// next from the XCD's ticket word in scratch whenever they begin a unit, one unit ahead of need, so the draw's
// latency hides behind that unit's first tile. While a unit's last tiles are multiplied, the K and V tiles of
// the next unit's first keys are already on their way into LDS; the last tile's stage A computes the next
// unit's first scores from that unit's queries (fetched a tile earlier into the fragment registers the finished
// unit no longer needs); after the last tile's stage B the finished unit is normalised and stored and the
// running maximum, sum and accumulators start again. A unit then costs its key tiles and one fetch of its
// queries, not a workgroup dispatch, a cold prologue and a drained pipeline at its end.
// What it measured (bf16, D = 128, us, one workgroup per unit / persistent, same process, same box):
//   B=2 S=4352 H=24 (3.19 rounds)  506 / 532      B=2 S=4096 H=24 (3.00 rounds)  433 / 447
//   B=1 S=4608 H=24 (1.69 rounds)  306 / 316      B=2 S=32760 H=40 (40 rounds)   39709 / 41187
// i.e. 3 to 5 % slower everywhere, also at 40 units per workgroup where the boundaries no longer matter: the
// steady-state tile loop itself is slower. It carries the next unit's state and the boundary's branches in 97 of
// 102 scalar registers, so the tile loads' LDS destinations and the fragment addresses are formed again in every
// tile instead of being held: the hardware counters show 5.77 vector instructions per MFMA against 4.82 and the
// matrix pipe busy 50.8 % of the cycles against 57.0 %. And what it saves is little: at 8 key tiles per unit, where
// a unit's fixed cost (8 us: dispatch, cold first tiles, first scores, store) is a third of the unit, it runs in
// the time of one workgroup per unit (899 / 901 us at 32760 queries x 512 keys x 40 heads), so its boundary costs
// what a dispatch and a cold start cost. With a fixed assignment of units (w, w + W, ...) instead of the ticket
// words it was 6 % slower: compute units do not all run at one speed, and the dispatcher (or the tickets) gives
// the faster ones more work. Neither form removes the cost of a last round that is partly filled: that needs
// units cut along the keys (MODE 1).
#include <stddef.h>

#include <cstdlib>

#include "attn_common.h"
#include "attn_tail.h"

// LDS fragment reads issued ahead of the MFMA that consumes them (K: 16-byte reads, V: pairs of
// transpose reads); overridable for tuning builds.
#ifndef ODIT_ATTN_KPF
#define ODIT_ATTN_KPF 3
#endif
#ifndef ODIT_ATTN_VPF
#define ODIT_ATTN_VPF 3
#endif

namespace odit {

// A kernel argument fetched again from the argument segment at the point of use (a scalar load the compiler can
// neither hoist nor merge with others). The persistent form reads what it needs at a unit boundary this way:
// taken from the by-value argument struct, those fields would be held in scalar registers across the whole tile
// loop, which has none to spare.
template <typename V> __device__ __forceinline__ V kernel_arg(size_t offset) {
  typedef __attribute__((address_space(4))) const char* arg_ptr;
  arg_ptr base = (arg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
  return *(const volatile __attribute__((address_space(4))) V*)(base + offset);
}
#define ODIT_ARG(field) (PERSIST ? kernel_arg<decltype(AttnParams::field)>(offsetof(AttnParams, field)) : p.field)

typedef short s16x4_d __attribute__((ext_vector_type(4)));
typedef short s16x8_d __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_d* lds_s16x4_p;
typedef __attribute__((address_space(3))) void* lds_void_p;

// MODE 0: workgroup i owns unit i (a q block of one head of one batch row), all keys.
// MODE 1: launched after the full rounds for the units that are left over: workgroup i owns key
//         tiles [jt0, n_tiles) of unit n_full + i / key_chunks and leaves an unnormalised partial
//         result in scratch for attn_merge_kernel.
// MODE 2: persistent, see above.
// Separate instantiations, so the extra bookkeeping of one cannot disturb the register allocation of another.
template <typename T, int D, int NW, int MODE>
__global__ __launch_bounds__(NW * 64, 8 / NW) void attn_fwd_dma_kernel(const AttnParams p) {
  constexpr bool TAIL = MODE == 1;
  constexpr bool PERSIST = MODE == 2;
  using M = Mma<T>;
  using frag = typename M::frag;
  constexpr int BN = 64;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int ROWB = D * 2;                 // bytes per tile row
  constexpr int CPR = ROWB / 16;              // 16-byte chunks per row (16 for D=128, 8 for D=64)
  constexpr int RPI = 64 / CPR;               // tile rows filled by one wave instruction (4 or 8)
  constexpr int TILEB = BN * ROWB;            // bytes per tile
  constexpr int NINST = BN / RPI;             // wave instructions per tile (16 or 8)
  // NW = 8 is the anti-phase form: the workgroup's two wavefronts on a SIMD (w and w + 4) run the same tile loop
  // half a tile apart, held there by a second barrier between the stages, so one's stage A (exp2 and the other
  // vector work, with the next scores' MFMAs) always meets the other's stage B (MFMAs and LDS reads only). Wavefronts
  // 0-3 fetch the K tiles, 4-7 the V tiles, each group at the start of its own stage A.
  constexpr bool PP = NW == 8;
  static_assert(!(PP && PERSIST), "the persistent form has no anti-phase variant");
  constexpr int NWL = PP ? 4 : NW;              // wavefronts that fetch one tile
  constexpr int IPW = (NINST + NWL - 1) / NWL;  // ... per wavefront
  static_assert(NINST % NWL == 0, "tile loads must divide evenly over the wavefronts");
  constexpr int BM = NW * 32;

  __shared__ __attribute__((aligned(1024))) char lds[4 * TILEB];  // K0 K1 V0 V1
  char* const Kb = lds;
  char* const Vb = lds + 2 * TILEB;
  constexpr int kKoff = 0, kVoff = 2 * TILEB;  // the same as byte offsets, for the tile loads' LDS destinations

  const int n_tiles_all = (p.Sk + BN - 1) / BN;
  int pid, jt0 = 0, n_tiles = n_tiles_all;
  const int part = blockIdx.x;
  // persistent form: the unit after the current one (-1: none, or not drawn yet)
  int next_pid = -1;
  __shared__ int next_unit_box;  // thread 0's draw, handed to the workgroup across a tile's barrier
  if constexpr (MODE == 0) {
    pid = xcd_remap(blockIdx.x, p.n_full);
  } else if constexpr (TAIL) {  // this workgroup covers key tiles [jt0, n_tiles) of unit pid (jt0 is even)
    pid = p.n_full + part / p.key_chunks;
    jt0 = (part % p.key_chunks) * p.tiles_per_chunk;
    n_tiles = jt0 + p.tiles_per_chunk < n_tiles_all ? jt0 + p.tiles_per_chunk : n_tiles_all;
  } else {
    // gridDim.x = W workgroups, a multiple of the XCD count, all resident; hardware puts workgroup w on XCD
    // w % 8. XCD x owns units [x_lo, x_hi); its W / 8 workgroups start on the first W / 8 of them.
    const int xcd = part % kNumXcd;
    const int x_lo = static_cast<int>(static_cast<int64_t>(p.n_full) * xcd / kNumXcd);
    const int x_hi = static_cast<int>(static_cast<int64_t>(p.n_full) * (xcd + 1) / kNumXcd);
    pid = x_lo + part / kNumXcd;
    if (pid >= x_hi) return;  // fewer units than workgroups on this XCD (before any barrier: the whole workgroup leaves)
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int wl = PP ? (wave & 3) : wave;     // this wavefront's share of a tile load
  const bool grp1 = PP && wave >= 4;          // second group of the anti-phase form (wave-uniform)

  // ---- the current unit (fixed for MODE 0 and 1, advanced unit by unit in the persistent form) ----
  int h = (pid / p.n_qblocks) % p.H;
  int b = (pid / p.n_qblocks) / p.H;
  int q0 = (pid % p.n_qblocks) * BM + wave * 32;

  // buffer descriptors end right after the last valid key row: later rows read as zeros
  const uint32_t k_bytes = static_cast<uint32_t>(((p.Sk - 1) * p.ks_s + D) * 2);
  // value rows [0, k_split) come from v, rows [k_split, Sk) from v_tail (k_split is a whole number of
  // tiles and both share the row stride): two descriptors, picked per tile with scalar selects
  const int v_split_tiles = p.v_tail != nullptr ? p.k_split / BN : n_tiles_all;
  const int v_rows = p.v_tail != nullptr ? p.k_split : p.Sk;
  const uint32_t v_bytes = static_cast<uint32_t>(((v_rows - 1) * p.vs_s + D) * 2);
  const uint32_t v2_bytes = p.v_tail != nullptr ? static_cast<uint32_t>(((p.Sk - p.k_split - 1) * p.vs_s + D) * 2) : v_bytes;
  // raw buffer descriptors {base[31:0], base[47:32] (stride 0), bytes, dword3 = 0x00020000}
  auto make_rsrc = [](const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4_v r;
    r.x = static_cast<uint32_t>(a); r.y = static_cast<uint32_t>(a >> 32) & 0xffffu; r.z = bytes; r.w = 0x00020000u;
    return r;
  };
  // descriptors of the keys / values / second value tensor of (batch b_, head h_)
  auto k_rsrc_of = [&](int b_, int h_) {
    const int hkv_ = h_ / (ODIT_ARG(H) / ODIT_ARG(Hkv));
    return make_rsrc(static_cast<const T*>(ODIT_ARG(k)) + b_ * ODIT_ARG(ks_b) + hkv_ * ODIT_ARG(ks_h), k_bytes);
  };
  auto v_rsrc_of = [&](int b_, int h_) {
    const int hkv_ = h_ / (ODIT_ARG(H) / ODIT_ARG(Hkv));
    return make_rsrc(static_cast<const T*>(ODIT_ARG(v)) + b_ * ODIT_ARG(vs_b) + hkv_ * ODIT_ARG(vs_h), v_bytes);
  };
  auto v2_rsrc_of = [&](int b_, int h_) {
    const int hkv_ = h_ / (ODIT_ARG(H) / ODIT_ARG(Hkv));
    return make_rsrc(static_cast<const T*>(ODIT_ARG(v_tail)) + b_ * ODIT_ARG(vt_b) + hkv_ * ODIT_ARG(vt_h), v2_bytes);
  };
  u32x4_v krsrc = k_rsrc_of(b, h);
  u32x4_v vrsrc = v_rsrc_of(b, h);
  u32x4_v vrsrc2 = p.v_tail != nullptr ? v2_rsrc_of(b, h) : vrsrc;
  const uint8_t* mrow = p.mask ? p.mask + static_cast<int64_t>(b) * p.Sk : nullptr;
  // persistent form: where the next unit is (valid while next_pid >= 0)
  int n_h = 0, n_b = 0;
  // Thread 0 draws the unit after the current one: the XCD's word is raised to this launch's epoch (a no-op but
  // for the XCD's first draw of the launch), then ticket t names unit x_first + t. Every unit that is run draws
  // once, so the draw with the ticket of the XCD's last unit is the launch's last on this word and puts it back
  // to zero (a launch replayed from a HIP graph carries the same epoch).
  auto draw_next = [&]() {
    if (tid == 0) {
      // the XCD's unit range, worked out again here rather than held in scalar registers for the whole unit
      int xcd = part % kNumXcd;
      asm volatile("" : "+s"(xcd));  // (so that the word's address is formed here, not held in vector registers)
      const int per = static_cast<int>(gridDim.x) / kNumXcd;
      const int x_lo = static_cast<int>(static_cast<int64_t>(p.n_full) * xcd / kNumXcd);
      const int x_hi = static_cast<int>(static_cast<int64_t>(p.n_full) * (xcd + 1) / kNumXcd);
      const int x_first = x_lo + per < x_hi ? x_lo + per : x_hi;  // first unit handed out by ticket
      unsigned long long* word = ODIT_ARG(queue) + xcd * 8;
      __hip_atomic_fetch_max(word, ODIT_ARG(epoch) << 24, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned t = static_cast<unsigned>(__hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) & 0xffffffu;
      if (static_cast<int>(t) == x_hi - x_lo - 1) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int cand = x_first + static_cast<int>(t);
      next_unit_box = cand < x_hi ? cand : -1;
    }
  };
  auto take_next = [&]() {  // behind the barrier that follows draw_next
    next_pid = __builtin_amdgcn_readfirstlane(next_unit_box);
    if (next_pid >= 0) {
      const int bh = next_pid / ODIT_ARG(n_qblocks), heads = ODIT_ARG(H);
      n_h = bh % heads;
      n_b = bh / heads;
    }
  };

  // Per-lane global byte offset of the chunk this lane moves with its wave's FIRST instruction of a tile,
  // relative to the tile's first row; instruction i moves the rows RPI * i further down, which is a scalar
  // term (it goes into the load's scalar offset), and its swizzle differs from the first one's by a constant:
  // for K, row % 16 = (row0 % 16) + (RPI * i) % 16 without a carry (row0 % 16 < RPI), so the chunk index is that
  // of instruction 0 XOR ((RPI * i) % 16 % CPR) - for V (4 * (row % 4), RPI a multiple of 4) it is the same. The
  // XOR is done on the byte offset, which needs row strides that are multiples of the row's own 2 D bytes.
  const int r0 = wl * IPW * RPI + lane / CPR, pc0 = lane % CPR;
  const uint32_t kvoff0 = static_cast<uint32_t>(r0 * p.ks_s * 2) + static_cast<uint32_t>(((pc0 ^ (r0 % 16)) % CPR) * 16);
  const uint32_t vvoff0 = static_cast<uint32_t>(r0 * p.vs_s * 2) + static_cast<uint32_t>(((pc0 ^ (4 * (r0 % 4))) % CPR) * 16);
  const uint32_t k_inst_step = static_cast<uint32_t>(RPI * p.ks_s * 2);
  const uint32_t v_inst_step = static_cast<uint32_t>(RPI * p.vs_s * 2);
  const uint32_t k_tile_step = static_cast<uint32_t>(BN * p.ks_s * 2);
  const uint32_t v_tile_step = static_cast<uint32_t>(BN * p.vs_s * 2);

  // The tile loads are written as inline assembly on purpose. Issued through the compiler's builtin they
  // are known to it as pending LDS writes, and it then puts `s_waitcnt vmcnt(0)` in front of the first V
  // fragment read of every tile (it cannot prove that the XOR-swizzled read addresses miss the buffer
  // being filled): the loads issued at the top of a tile, meant to land a whole tile later, were waited
  // for half a tile after issue. Here the ordering is explicit instead: one `s_waitcnt vmcnt(0)` and one
  // barrier at the end of each tile, before any wave reads the buffers those loads filled.
  // `dst_off` is the tile's byte offset inside the kernel's LDS block: a literal at every call
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_p)lds));
  auto dma_tile = [&](const u32x4_v& rsrc, const bool is_k, uint32_t soff, const int dst_off) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t lds0 = lds_base + static_cast<uint32_t>(dst_off) + static_cast<uint32_t>(wl * IPW * 1024);
    // (the empty asm makes the offset opaque here: otherwise the compiler forms the IPW swizzled offsets once,
    // outside the tile loop, and holds them in registers the loop does not have)
    uint32_t voff0 = is_k ? kvoff0 : vvoff0;
    asm volatile("" : "+v"(voff0));
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds0 + i * 1024);
      const uint32_t voff_i = is_k ? (voff0 ^ static_cast<uint32_t>((((RPI * i) % 16) % CPR) * 16)) : voff0;
      const uint32_t soff_i = soff + static_cast<uint32_t>(i) * (is_k ? k_inst_step : v_inst_step);
      // m0 (the LDS destination of the load) is a reserved register: naming it as clobbered draws a
      // warning per expansion, and leaving it out would hide the write from the compiler
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   :
                   : "s"(m0v), "v"(voff_i), "s"(rsrc), "s"(soff_i)
                   : "memory", "m0");
#pragma clang diagnostic pop
    }
#endif
  };

  auto dma_v = [&](int jt, const int dst) {
    const bool second = jt >= v_split_tiles;
    dma_tile(second ? vrsrc2 : vrsrc, false, static_cast<uint32_t>(second ? jt - v_split_tiles : jt) * v_tile_step, dst);
  };
  // the same for tiles of the NEXT unit (persistent form): descriptors made on the spot from (n_b, n_h), a few
  // scalar instructions per tile instead of a dozen scalar registers held for the whole unit
  auto dma_k_next = [&](int jt, const int dst) {
    dma_tile(k_rsrc_of(n_b, n_h), true, static_cast<uint32_t>(jt) * k_tile_step, dst);
  };
  auto dma_v_next = [&](int jt, const int dst) {
    const bool second = jt >= v_split_tiles;
    dma_tile(second ? v2_rsrc_of(n_b, n_h) : v_rsrc_of(n_b, n_h), false,
             static_cast<uint32_t>(second ? jt - v_split_tiles : jt) * v_tile_step, dst);
  };

  // ---- Q fragments stay in registers ----
  frag qf[KS];
  // (the persistent form calls these two inside the tile loop: they take the lane's position from the thread
  // index again, so that nothing of theirs is carried through the loop)
  auto lane_again = [&](int& l32_, int& hh_) {
    int t = tid;
    if constexpr (PERSIST) asm volatile("" : "+v"(t));
    l32_ = t & 31;
    hh_ = (t >> 5) & 1;
  };
  auto load_q = [&](int b_, int h_, int q0_) {
    int l32, hh;
    lane_again(l32, hh);
    int row = q0_ + l32;
    const int rows = ODIT_ARG(Sq);
    row = row < rows ? row : rows - 1;
    const T* qp = static_cast<const T*>(ODIT_ARG(q)) + b_ * ODIT_ARG(qs_b) + h_ * ODIT_ARG(qs_h) + row * ODIT_ARG(qs_s) + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(qp + ks * 16));
  };
  load_q(b, h, q0);

  f32x16_v o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const float c = p.scale_log2;

  // K fragment (kt, ks): row kt*32 + l32, logical chunk 2*ks + hh  ->  chunk (2*ks) ^ (hh ^ l32 % 16)
  const int k_lane = l32 * ROWB + ((((hh ^ (l32 % 16)) % CPR)) << 4);
  // V transpose read, 16-lane group g = lane/16 (d half dh = g&1, key half = hh), lane s = lane%16:
  // key 4*hh + s/4 (+ tile offsets), logical chunk 4*dt + 2*dh + (s%4)/2, 8-byte half (s%4)%2,
  // physical chunk = logical ^ 4*(s/4)  ->  XOR of the dt field only
  const int sq = (lane & 15) >> 2;
  const int dh = (lane >> 4) & 1;
  const int v_lane = (4 * hh + sq) * ROWB + ((((4 * sq) % CPR) ^ (2 * dh + ((lane & 3) >> 1))) << 4) + ((lane & 1) << 3);

  auto qk_plain = [&](const char* kt_base, f32x16_v(&s)[2]) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kt][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const frag a = __builtin_bit_cast(
            frag, *reinterpret_cast<const u32x4_v*>(kt_base + kt * 32 * ROWB + (k_lane ^ (ks * 32))));
        s[kt] = M::run(a, qf[ks], s[kt]);
      }
  };

  auto mask_and_max = [&](int j, const uint8_t* mrow, f32x16_v(&s)[2]) -> float {
    // branch-free selects: every lane rewrites all its scores, excluded ones with -inf
    if (mrow != nullptr) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int key = j * BN + kt * 32 + g * 8 + hh * 4 + t;
            const int kc = key < p.Sk ? key : p.Sk - 1;
            const bool live = (key < p.Sk) & (mrow[kc] != 0);
            const float x = s[kt][g * 4 + t];
            s[kt][g * 4 + t] = live ? x : -INFINITY;
          }
    } else if ((j + 1) * BN > p.Sk) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int key = j * BN + kt * 32 + g * 8 + hh * 4 + t;
            const float x = s[kt][g * 4 + t];
            s[kt][g * 4 + t] = key < p.Sk ? x : -INFINITY;
          }
    }
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[kt][e]);
    return mx;
  };

  // mx = row maximum over both lane halves
  auto settle_max = [&](float mx) {
    const float m_new = fmaxf(m_run, mx);
    if (__any((m_new - m_run) * c > 8.f)) {
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_safe) * c);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
      m_run = m_new;
    }
  };

  // normalises and stores the finished unit (b, h, q0): the tail of MODE 0 and of every unit of the persistent form
  auto finish_unit = [&]() {
    int l32, hh;
    lane_again(l32, hh);
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = q0 + l32;
    if (row < ODIT_ARG(Sq)) {
      // head of the joint sequence in `o`, tail in `o_tail` (out_row_ptr, with the arguments fetched here)
      T* op;
      void* const o_tail = ODIT_ARG(o_tail);
      const int q_split = ODIT_ARG(q_split);
      if (o_tail != nullptr && row >= q_split) {
        op = static_cast<T*>(o_tail) + b * ODIT_ARG(ts_b) + h * ODIT_ARG(ts_h) + static_cast<int64_t>(row - q_split) * ODIT_ARG(ts_s);
      } else {
        op = static_cast<T*>(ODIT_ARG(o)) + b * ODIT_ARG(os_b) + h * ODIT_ARG(os_h) + static_cast<int64_t>(row) * ODIT_ARG(os_s);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2_v w;
          w.x = M::pack2(o[dt][g * 4 + 0] * inv, o[dt][g * 4 + 1] * inv);
          w.y = M::pack2(o[dt][g * 4 + 2] * inv, o[dt][g * 4 + 3] * inv);
          *reinterpret_cast<u32x2_v*>(op + dt * 32 + g * 8 + hh * 4) = w;
          // (in the persistent form this runs inside the tile loop, with the next unit's queries and first scores
          // live: the values go out one store at a time instead of being formed all at once)
          if constexpr (PERSIST) __builtin_amdgcn_sched_barrier(0);
        }
      float* const lse_out = ODIT_ARG(lse);
      if (lse_out != nullptr && hh == 0) {
        const float lse = l_tot > 0.f ? m_run * ODIT_ARG(scale) + __logf(l_tot) : -INFINITY;
        lse_out[(static_cast<int64_t>(b) * ODIT_ARG(H) + h) * ODIT_ARG(Sq) + row] = lse;
      }
    }
  };

  // Tile j of the current unit. In the persistent form the tile after a unit's last one is tile 0 of the
  // workgroup's next unit (`cross`), and the tile after that its tile 1.
  // `buf` (the LDS buffer pair of this tile: the parity of its running index) is a literal at every call, so the
  // LDS addresses below are compile-time offsets.
  auto tile = [&](int j, const int buf, f32x16_v(&s_cur)[2], f32x16_v(&s_next)[2]) {
    const bool last = j + 1 == n_tiles;
    const bool cross = PERSIST && last && next_pid >= 0;
    const bool has_next = !last || cross;
    // buffers K[buf] (held K(j), consumed last tile) and V[buf^1] (held V(j-1)) are free now
    // (anti-phase form: the first group fetches K, the second V; K(j) was last read by the second group's stage A
    // of tile j - 1, half a tile before the first group gets here, V(j-1) by the second group's own stage B)
    if (!PP || !grp1) {
      if (j + 2 < n_tiles) {
        dma_tile(krsrc, true, static_cast<uint32_t>(j + 2) * k_tile_step, kKoff + buf * TILEB);
      } else if (PERSIST && next_pid >= 0) {
        dma_k_next(j + 2 - n_tiles, kKoff + buf * TILEB);
      }
    }
    if constexpr (PERSIST) {
      if (j == 0) draw_next();  // the answer is in the box when this tile's barrier has been passed
    }
    if (!PP || grp1) {
      if (!last) {
        dma_v(j + 1, kVoff + (buf ^ 1) * TILEB);
      } else if (cross) {
        dma_v_next(0, kVoff + (buf ^ 1) * TILEB);
      }
    }
    // the tile whose scores stage A computes, and the mask row of its unit
    const int jn = last ? 0 : j + 1;
    const uint8_t* mrow_n = cross ? (p.mask ? p.mask + static_cast<int64_t>(n_b) * p.Sk : nullptr) : mrow;  // (p.mask and p.Sk are live in the tile loop anyway)

    const float mc = (m_run == -INFINITY) ? 0.f : m_run * c;
    // (Row sums in fp32 from the unrounded probabilities. Summing the packed pairs with v_dot2c_f32_bf16, one
    // instruction per pair instead of two adds, measured 4 % slower at D = 128, with one chain or four.)
    uint32_t pf[2][2][4];
    float psum = 0.f;
    // Stage A mixes this wave's MFMAs with its exp2 work; giving it issue priority over the SIMD's other
    // wave (which is then mostly in its MFMA + LDS-read stage B) measured +5 % at 32760 keys, +9 % at
    // batch 1 / 4608 keys and nothing lost at the 4352-token, batch-2 shape.
    __builtin_amdgcn_s_setprio(2);
    // ---- stage A ----
    if (has_next) {
      const char* kt_base = Kb + (buf ^ 1) * TILEB;
      // (opaque copy: the KS swizzled variants of the lane offset are formed again in every tile, one XOR each,
      // instead of being carried through the loop in KS registers)
      int k_lane_t = k_lane;
      if constexpr (PERSIST) asm volatile("" : "+v"(k_lane_t));
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s_next[kt][e] = 0.f;
      constexpr int KPF = ODIT_ATTN_KPF;  // K fragments in flight ahead of the MFMA that consumes them
      u32x4_v kfr[KPF + 1];
      auto k_fetch = [&](int i) {
        const int ks = i >> 1, kt = i & 1;
        kfr[i % (KPF + 1)] = *reinterpret_cast<const u32x4_v*>(kt_base + kt * 32 * ROWB + (k_lane_t ^ (ks * 32)));
      };
#pragma unroll
      for (int i = 0; i < KPF; ++i) k_fetch(i);
#pragma unroll
      for (int i = 0; i < 2 * KS; ++i) {
        if (i + KPF < 2 * KS) k_fetch(i + KPF);
        const int ks = i >> 1, kt = i & 1;
        s_next[kt] = M::run(__builtin_bit_cast(frag, kfr[i % (KPF + 1)]), qf[ks], s_next[kt]);
        constexpr int PAIRS = 16 / (2 * KS) > 0 ? 16 / (2 * KS) : 1;
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
          const int pi = i * PAIRS + q;
          if (pi < 16) {
            const int pkt = pi >> 3, e0 = (pi & 7) * 2;
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0], c, -mc));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0 + 1], c, -mc));
            psum += p0 + p1;
            pf[pkt][(pi & 7) >> 2][pi & 3] = M::pack2(p0, p1);
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // pin: fetch(i+KPF), MFMA(i), this step's exp2 work
      }
    } else {
      // (an opaque copy of the offset: were the two branches' exponent arguments the same expressions, the
      // compiler would form all 32 ahead of the branch, out of the MFMAs' shadow and in 32 more registers)
      float mc_t = mc;
      asm volatile("" : "+v"(mc_t));
#pragma unroll
      for (int pi = 0; pi < 16; ++pi) {
        const int pkt = pi >> 3, e0 = (pi & 7) * 2;
        const float p0 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0], c, -mc_t));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0 + 1], c, -mc_t));
        psum += p0 + p1;
        pf[pkt][(pi & 7) >> 2][pi & 3] = M::pack2(p0, p1);
      }
    }
    l_run += psum;
    if constexpr (PERSIST) {
      // The next unit's queries replace this unit's once its last scores have been formed, a tile before they are
      // used: they land behind this tile's closing wait. (Loaded at the top of the tile that uses them, the
      // compiler's own wait for them, which it has to place on every trip through the loop, also waits for the
      // tile loads it does not know of.)
      if (j + 2 == n_tiles && next_pid >= 0)
        load_q(n_b, n_h, (next_pid - (n_b * ODIT_ARG(H) + n_h) * ODIT_ARG(n_qblocks)) * BM + wave * 32);
    }

    __builtin_amdgcn_s_setprio(0);
    if constexpr (PP) {
      // the stages' boundary: the two groups swap roles here. A bare barrier: no wavefront writes LDS, and the tile
      // loads in flight are waited for at the end of the tile, not here.
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- stage B: O^T += V(j)^T P(j)^T ----
    // 4*DT steps, head-dim tile innermost so that consecutive MFMAs hit different accumulators and one
    // P fragment serves DT of them; the two transpose reads of step n + PF are issued before the MFMA
    // of step n, so LDS latency is covered by PF matrix instructions. The in-lane row maximum of
    // S(j+1) — vector work with nothing to wait for — is placed in the shadow of these MFMAs.
    const char* vt_base = Vb + buf * TILEB;
    int v_lane_t = v_lane;  // (opaque copy, as for the key fragments)
    if constexpr (PERSIST) asm volatile("" : "+v"(v_lane_t));
    constexpr int NSTEP = 4 * DT;
    constexpr int PF = ODIT_ATTN_VPF;
    s16x4_d vlo[PF + 1], vhi[PF + 1];
    auto v_fetch = [&](int step) {
      const int dt = step % DT, kt = (step / DT) >> 1, g2 = (step / DT) & 1;
      const char* vp = vt_base + (kt * 32 + g2 * 16) * ROWB + (v_lane_t ^ ((dt * 64) % ROWB));
      vlo[step % (PF + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_p)(vp));
      vhi[step % (PF + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_p)(vp + 8 * ROWB));
    };
    const bool plain_next = has_next && mrow_n == nullptr && (jn + 1) * BN <= p.Sk;  // no exclusions in the next scores
    float mx = -INFINITY;
#pragma unroll
    for (int st = 0; st < PF; ++st) v_fetch(st);
#pragma unroll
    for (int st = 0; st < NSTEP; ++st) {
      if (st + PF < NSTEP) v_fetch(st + PF);
      const int dt = st % DT, kt = (st / DT) >> 1, g2 = (st / DT) & 1;
      const s16x8_d av = __builtin_shufflevector(vlo[st % (PF + 1)], vhi[st % (PF + 1)], 0, 1, 2, 3, 4, 5, 6, 7);
      u32x4_v pb;
      pb.x = pf[kt][g2][0]; pb.y = pf[kt][g2][1]; pb.z = pf[kt][g2][2]; pb.w = pf[kt][g2][3];
      o[dt] = M::run(__builtin_bit_cast(frag, av), __builtin_bit_cast(frag, pb), o[dt]);
      if (st == 1 && plain_next) {  // wave-uniform
        float t = s_next[0][0];
#pragma unroll
        for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
          for (int e = 0; e < 16; ++e) t = fmaxf(t, s_next[kt2][e]);
        mx = fmaxf(t, __shfl_xor(t, 32, 64));
      }
      __builtin_amdgcn_sched_barrier(0);  // keep the reads of step st+PF ahead of this MFMA
    }
    if (has_next && !plain_next) {
      const float t = mask_and_max(jn, mrow_n, s_next);
      mx = fmaxf(t, __shfl_xor(t, 32, 64));
    }
    __builtin_amdgcn_s_waitcnt(0);  // this wave's tile loads have landed in LDS
    __syncthreads();
    if constexpr (PERSIST) {
      if (j == 0) take_next();
      if (last) {
        finish_unit();
        if (cross) {  // the next unit becomes the current one; its running maximum, sum and accumulators start over
          h = n_h; b = n_b;
          q0 = (next_pid - (n_b * ODIT_ARG(H) + n_h) * ODIT_ARG(n_qblocks)) * BM + wave * 32;
          krsrc = k_rsrc_of(b, h);
          vrsrc = v_rsrc_of(b, h);
          vrsrc2 = p.v_tail != nullptr ? v2_rsrc_of(b, h) : vrsrc;
          mrow = mrow_n;
          pid = next_pid;
          next_pid = -1;  // drawn during the new unit's first tile
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
          m_run = -INFINITY;
          l_run = 0.f;
        }
      }
    }
    if (has_next) settle_max(mx);
  };

  // ---- prologue (jt0 is even, so tile j always lives in buffer j & 1) ----
  if (!PP || !grp1) dma_tile(krsrc, true, static_cast<uint32_t>(jt0) * k_tile_step, kKoff);
  if (!PP || grp1) dma_v(jt0, kVoff);
  if ((!PP || !grp1) && jt0 + 1 < n_tiles) dma_tile(krsrc, true, static_cast<uint32_t>(jt0 + 1) * k_tile_step, kKoff + TILEB);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  f32x16_v sa[2], sb[2];
  qk_plain(Kb, sa);
  {
    const float t = mask_and_max(jt0, mrow, sa);
    settle_max(fmaxf(t, __shfl_xor(t, 32, 64)));
  }
  // every wavefront has read the first K tile: the loop's first tile load overwrites it
  __syncthreads();
  if constexpr (PP) {
    // the second group enters the loop one barrier, i.e. half a tile, behind the first (which makes up for it
    // behind the loop)
    if (grp1) asm volatile("s_barrier" ::: "memory");
  }

  if constexpr (PERSIST) {
    // one stream of tiles over all units this workgroup gets; every unit stores itself behind its last tile, and
    // the stream ends behind a unit that found the XCD's range exhausted (every wave sees the same next_pid)
    int j = 0;
    for (;;) {  // a tile's buffer pair is the parity of its index in this stream
      bool done = j + 1 == n_tiles && next_pid < 0;
      tile(j, 0, sa, sb);
      if (done) break;
      j = j + 1 == n_tiles ? 0 : j + 1;
      done = j + 1 == n_tiles && next_pid < 0;
      tile(j, 1, sb, sa);
      if (done) break;
      j = j + 1 == n_tiles ? 0 : j + 1;
    }
    return;
  } else {
    for (int j = jt0; j < n_tiles; j += 2) {  // jt0 is even
      tile(j, 0, sa, sb);
      if (j + 1 < n_tiles) tile(j + 1, 1, sb, sa);
    }
    if constexpr (PP) {
      if (!grp1) asm volatile("s_barrier" ::: "memory");
    }
  }

  // ---- epilogue ----
  if constexpr (TAIL) {
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    // partial result of a key range: unnormalised O (fp32, [BM][D] per part) and the row's (m, l)
    float* wo = p.ws + (static_cast<int64_t>(part) * BM + wave * 32 + l32) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4_v w4;
        w4.x = o[dt][g * 4 + 0]; w4.y = o[dt][g * 4 + 1]; w4.z = o[dt][g * 4 + 2]; w4.w = o[dt][g * 4 + 3];
        *reinterpret_cast<f32x4_v*>(wo + dt * 32 + g * 8 + hh * 4) = w4;
      }
    if (hh == 0) {
      float* ml = p.ws + static_cast<int64_t>(gridDim.x) * BM * D +
                  (static_cast<int64_t>(part) * BM + wave * 32 + l32) * 2;
      ml[0] = m_run;
      ml[1] = l_tot;
    }
    return;
  }
  finish_unit();
}

// The persistent form is a measurement aid, off unless the environment says ODIT_ATTN_PERSISTENT=1 when the
// library makes its first attention launch: with it every shape measured ran 3 to 6 % slower than one workgroup
// per unit (its tile loop is slower than what it saves at the unit boundaries, see the header comment).
#ifndef ODIT_ATTN_PERSISTENT_DEFAULT
#define ODIT_ATTN_PERSISTENT_DEFAULT 0
#endif
static bool persistent_form_on() {
  static const bool on = [] {
    const char* e = getenv("ODIT_ATTN_PERSISTENT");
    return e != nullptr ? e[0] == '1' : ODIT_ATTN_PERSISTENT_DEFAULT != 0;
  }();
  return on;
}

// Workgroups of the persistent form for `units` whole units of `n_tiles` key tiles each on `slots` workgroup
// slots, or 0 when every unit gets a workgroup of its own (no more units than slots, or units too short for the
// next unit to be known before its first tiles are fetched).
static int persistent_workgroups(int units, int n_tiles, int slots, int nw) {
  const int W = slots - slots % kNumXcd;
  if (!persistent_form_on() || nw != 4 || W < kNumXcd || units <= W || n_tiles < 4 || units >= (1 << 26)) return 0;  // tickets have 24 bits
  return W;
}

template <typename T, int D, int NW>
static int launch_dma(AttnParams& p, hipStream_t stream, void* ws, size_t ws_bytes) {
  constexpr int BM = NW * 32;
  p.n_qblocks = (p.Sq + BM - 1) / BM;
  const int64_t total = static_cast<int64_t>(p.n_qblocks) * p.H * p.B;
  if (total > 0x3fffffffll) {
    set_error("odit_attn_fwd: grid of %lld workgroups is too large", static_cast<long long>(total));
    return ODIT_EINVAL;
  }
  p.total_blocks = static_cast<int>(total);
  p.n_full = p.total_blocks; p.key_chunks = 1; p.tiles_per_chunk = 0; p.ws = nullptr;
  p.queue = nullptr; p.epoch = 0;
  TailPlan t{0, 1, 0};
  const int n_tiles = (p.Sk + 63) / 64, slots = device_slots(NW);
  if (ws != nullptr) {
    if ((reinterpret_cast<uintptr_t>(ws) & 15) != 0) {
      set_error("odit_attn_fwd: workspace must be 16-byte aligned");
      return ODIT_EINVAL;
    }
    t = plan_tail(total, n_tiles, slots);
    const size_t need = attn_dma_workspace_bytes(p.B, p.Sq, p.Sk, p.H, D);
    if (ws_bytes < need) {
      set_error("odit_attn_fwd: workspace of %zu bytes given, %zu needed", ws_bytes, need);
      return ODIT_EWORKSPACE;
    }
    if (t.rem > 0) {
      p.n_full = p.total_blocks - t.rem; p.key_chunks = t.key_chunks; p.tiles_per_chunk = t.tiles_per_chunk;
      p.ws = reinterpret_cast<float*>(static_cast<char*>(ws) + kAttnQueueBytes);
    }
  }
  const int n_parts = t.rem * t.key_chunks;
  int rc = ODIT_OK;
  if (p.n_full > 0) {
    // the persistent form draws its units from ticket words at the head of the workspace
    const int W = (ws != nullptr && NW == 4) ? persistent_workgroups(p.n_full, n_tiles, slots, NW) : 0;
    if constexpr (NW == 4) {
      if (W > 0) {
        p.queue = static_cast<unsigned long long*>(ws);
        p.epoch = next_ticket_epoch() & ((1ull << 40) - 1);
        hipLaunchKernelGGL((attn_fwd_dma_kernel<T, D, NW, 2>), dim3(W), dim3(NW * 64), 0, stream, p);
      }
    }
    if (W == 0) {
      hipLaunchKernelGGL((attn_fwd_dma_kernel<T, D, NW, 0>), dim3(p.n_full), dim3(NW * 64), 0, stream, p);
    }
    rc = check_launch("odit_attn_fwd");
  }
  if (rc != ODIT_OK || n_parts == 0) return rc;
  // stream order puts these after the full rounds, when every slot is free again
  hipLaunchKernelGGL((attn_fwd_dma_kernel<T, D, NW, 1>), dim3(n_parts), dim3(NW * 64), 0, stream, p);
  rc = check_launch("odit_attn_fwd (key-split tail)");
  if (rc != ODIT_OK) return rc;
  const int64_t rows = static_cast<int64_t>(t.rem) * BM;
  hipLaunchKernelGGL((attn_merge_kernel<T, D, BM>), dim3(static_cast<unsigned>((rows + 3) / 4)), dim3(256), 0,
                     stream, p, n_parts);
  return check_launch("odit_attn_fwd (merge)");
}

// Wavefronts per workgroup: 4 (two workgroups per compute unit, each on its own) or 8 (one workgroup per compute unit
// whose two halves run in anti-phase). Side by side in one process (bf16, us, 4 / 8 wavefronts; two boxes):
//   D=128  B=2 S=4352 H=24  514 / 491, 492 / 473     B=2 S=4096 H=24  429 / 420, 407 / 402
//          B=1 S=4608 H=24  302 / 297, 289 / 288     B=2 S=32760 H=40  38910 / 38616, 37053 / 36483
//   D=64   B=2 S=4352 H=24  326 / 334, 316 / 328
// so head size 128 takes 8 and head size 64 stays at 4 - from 32 key tiles per unit on: the two halves of an
// 8-wavefront workgroup begin and end their unit together, so the unit's fixed cost (first tiles fetched cold,
// first scores, the store) is not hidden behind another workgroup's tiles as it is with two independent workgroups
// per compute unit, and with few tiles per unit that costs more than the anti-phase gains (B=2, 16384 queries,
// 24 heads, 4 / 8 wavefronts: 512 keys 300 / 334 us, 1024 keys 469 / 496, 2048 keys 823 / 823; Wan's cross-attention,
// 32760 queries x 512 keys x 40 heads, 901 / 947). (With the two halves' roles paired wrongly, wavefronts w and
// w + 1 or w and w + 2 in anti-phase instead of w and w + 4, the same kernel is 10 to 18 % slower: two wavefronts of a
// SIMD in the same stage is what costs, and independent workgroups already avoid it most of the time by themselves.)
// ODIT_ATTN_WAVES in the environment, read at the first attention launch, overrides the choice (for measurements).
static int dma_waves(int D, int Sk) {
  static const int forced = [] {
    const char* e = getenv("ODIT_ATTN_WAVES");
    const int v = e != nullptr ? atoi(e) : 0;
    return (v == 4 || v == 8) ? v : 0;
  }();
  if (forced != 0) return forced;
  return (D == 128 && Sk >= 32 * 64) ? 8 : 4;
}

size_t attn_dma_workspace_bytes(int B, int Sq, int Sk, int H, int D) {
  if (B <= 0 || Sq <= 0 || Sk <= 0 || H <= 0) return 0;
  const int nw = dma_waves(D, Sk);
  const int bm = nw * 32;
  const int64_t units = static_cast<int64_t>((Sq + bm - 1) / bm) * H * B;
  const int n_tiles = (Sk + 63) / 64, slots = device_slots(nw);
  const TailPlan t = plan_tail(units, n_tiles, slots);
  const int64_t main_units = units - t.rem;
  const bool persistent = main_units <= 0x3fffffff && persistent_workgroups(static_cast<int>(main_units), n_tiles, slots, nw) > 0;
  if (t.rem == 0 && !persistent) return 0;
  return kAttnQueueBytes + tail_ws_bytes(t, bm, D);  // ticket words first (zero-filled once), then the tail's partial results
}

// 32-bit buffer offsets: the whole key range of one (batch, head) must be addressable
bool attn_dma_addressable(int Sk, int D, int64_t k_seq_stride, int64_t v_seq_stride) {
  const int64_t k_span = (static_cast<int64_t>(Sk) + 64) * k_seq_stride * 2;
  const int64_t v_span = (static_cast<int64_t>(Sk) + 64) * v_seq_stride * 2;
  // (the tile loads fold their swizzle into the byte offset by an XOR, which needs rows that start on a multiple
  // of their own length of D elements)
  return k_span < (1ll << 31) && v_span < (1ll << 31) && k_seq_stride >= 0 && v_seq_stride >= 0 &&
         k_seq_stride % D == 0 && v_seq_stride % D == 0;
}

int attn_dma_plan(int B, int Sq, int Sk, int H, int D, bool with_workspace, char* text, size_t text_bytes) {
  const int nw = dma_waves(D, Sk), bm = nw * 32;
  const int64_t units = static_cast<int64_t>((Sq + bm - 1) / bm) * H * B;
  const int n_tiles = (Sk + 63) / 64, slots = device_slots(nw);
  TailPlan t{0, 1, 0};
  if (with_workspace) t = plan_tail(units, n_tiles, slots);
  // kernel names as a profiler prints them, with T for the element type
  char main_text[160];
  const int64_t main_units = units - t.rem;
  const int W = (!with_workspace || main_units > 0x3fffffff) ? 0 : persistent_workgroups(static_cast<int>(main_units), n_tiles, slots, nw);
  if (W > 0) {
    snprintf(main_text, sizeof(main_text), "attn_fwd_dma_kernel<T, %d, %d, 2> units=%lld on %d persistent workgroups", D,
             nw, static_cast<long long>(main_units), W);
  } else {
    snprintf(main_text, sizeof(main_text), "attn_fwd_dma_kernel<T, %d, %d, 0> units=%lld", D, nw,
             static_cast<long long>(main_units));
  }
  if (t.rem == 0) {
    snprintf(text, text_bytes, "%s", main_text);
    return 1;
  }
  snprintf(text, text_bytes, "%s; attn_fwd_dma_kernel<T, %d, %d, 1> units=%d x %d key ranges of %d tiles; "
           "attn_merge_kernel<T, %d, %d> rows=%d", main_text, D, nw, t.rem, t.key_chunks, t.tiles_per_chunk, D, bm,
           t.rem * bm);
  return main_units > 0 ? 3 : 2;
}

int launch_attn_dma(AttnParams& p, int dtype, int D, hipStream_t stream, void* ws, size_t ws_bytes) {
  if (!attn_dma_addressable(p.Sk, D, p.ks_s, p.vs_s)) return ODIT_ENOTSUP;
#define ODIT_DMA_GO(T)                                                                     \
  if (dma_waves(D, p.Sk) == 8) {                                                                  \
    if (D == 128) return launch_dma<T, 128, 8>(p, stream, ws, ws_bytes);                   \
    return launch_dma<T, 64, 8>(p, stream, ws, ws_bytes);                                  \
  }                                                                                        \
  if (D == 128) return launch_dma<T, 128, 4>(p, stream, ws, ws_bytes);                     \
  return launch_dma<T, 64, 4>(p, stream, ws, ws_bytes);
  if (dtype == ODIT_BF16) { ODIT_DMA_GO(bf16_t) }
  ODIT_DMA_GO(f16_t)
#undef ODIT_DMA_GO
}

}  // namespace odit
