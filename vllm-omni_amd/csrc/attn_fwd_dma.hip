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
// barrier per tile, XCD-aware workgroup order) is as in attn_fwd_pipe_kernel.
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

typedef short s16x4_d __attribute__((ext_vector_type(4)));
typedef short s16x8_d __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_d* lds_s16x4_p;
typedef __attribute__((address_space(3))) void* lds_void_p;

// TAIL = false: workgroup i owns unit i (a q block of one head of one batch row), all keys.
// TAIL = true:  launched after the full rounds for the units that are left over: workgroup i owns key
//               tiles [jt0, n_tiles) of unit n_full + i / key_chunks and leaves an unnormalised partial
//               result in scratch for attn_merge_kernel. A separate instantiation, so the extra
//               bookkeeping cannot disturb the register allocation of the main kernel.
template <typename T, int D, int NW, bool TAIL>
__global__ __launch_bounds__(NW * 64, 8 / NW) void attn_fwd_dma_kernel(const AttnParams p) {
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
  constexpr int IPW = (NINST + NW - 1) / NW;  // ... per wavefront
  static_assert(NINST % NW == 0, "tile loads must divide evenly over the wavefronts");
  constexpr int BM = NW * 32;

  __shared__ __attribute__((aligned(1024))) char lds[4 * TILEB];  // K0 K1 V0 V1
  char* const Kb = lds;
  char* const Vb = lds + 2 * TILEB;

  const int n_tiles_all = (p.Sk + BN - 1) / BN;
  int pid, jt0 = 0, n_tiles = n_tiles_all;
  const int part = blockIdx.x;
  if constexpr (!TAIL) {
    pid = xcd_remap(blockIdx.x, p.n_full);
  } else {  // this workgroup covers key tiles [jt0, n_tiles) of unit pid (jt0 is even)
    pid = p.n_full + part / p.key_chunks;
    jt0 = (part % p.key_chunks) * p.tiles_per_chunk;
    n_tiles = jt0 + p.tiles_per_chunk < n_tiles_all ? jt0 + p.tiles_per_chunk : n_tiles_all;
  }
  const int qb = pid % p.n_qblocks;
  const int bh = pid / p.n_qblocks;
  const int h = bh % p.H;
  const int b = bh / p.H;
  const int hkv = h / (p.H / p.Hkv);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int q0 = qb * BM + wave * 32;

  const T* qbase = static_cast<const T*>(p.q) + b * p.qs_b + h * p.qs_h;
  const T* kbase = static_cast<const T*>(p.k) + b * p.ks_b + hkv * p.ks_h;
  const T* vbase = static_cast<const T*>(p.v) + b * p.vs_b + hkv * p.vs_h;

  // buffer descriptors end right after the last valid key row: later rows read as zeros
  const uint32_t k_bytes = static_cast<uint32_t>(((p.Sk - 1) * p.ks_s + D) * 2);
  // value rows [0, k_split) come from v, rows [k_split, Sk) from v_tail (k_split is a whole number of
  // tiles and both share the row stride): two descriptors, picked per tile with scalar selects
  const int v_split_tiles = p.v_tail != nullptr ? p.k_split / BN : n_tiles_all;
  const int v_rows = p.v_tail != nullptr ? p.k_split : p.Sk;
  const uint32_t v_bytes = static_cast<uint32_t>(((v_rows - 1) * p.vs_s + D) * 2);
  // raw buffer descriptors {base[31:0], base[47:32] (stride 0), bytes, dword3 = 0x00020000}
  auto make_rsrc = [](const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4_v r;
    r.x = static_cast<uint32_t>(a); r.y = static_cast<uint32_t>(a >> 32) & 0xffffu; r.z = bytes; r.w = 0x00020000u;
    return r;
  };
  const u32x4_v krsrc = make_rsrc(kbase, k_bytes);
  const u32x4_v vrsrc = make_rsrc(vbase, v_bytes);
  u32x4_v vrsrc2 = vrsrc;
  if (p.v_tail != nullptr) {
    const T* vbase2 = static_cast<const T*>(p.v_tail) + b * p.vt_b + hkv * p.vt_h;
    vrsrc2 = make_rsrc(vbase2, static_cast<uint32_t>(((p.Sk - p.k_split - 1) * p.vs_s + D) * 2));
  }

  // per-lane global byte offsets of the chunks this lane moves, relative to the tile's first row
  uint32_t kvoff[IPW], vvoff[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int r = (wave * IPW + i) * RPI + lane / CPR;  // tile row
    const int pc = lane % CPR;
    kvoff[i] = static_cast<uint32_t>(r * p.ks_s * 2) + static_cast<uint32_t>(((pc ^ (r % 16)) % CPR) * 16);
    vvoff[i] = static_cast<uint32_t>(r * p.vs_s * 2) + static_cast<uint32_t>(((pc ^ (4 * (r % 4))) % CPR) * 16);
  }
  const uint32_t k_tile_step = static_cast<uint32_t>(BN * p.ks_s * 2);
  const uint32_t v_tile_step = static_cast<uint32_t>(BN * p.vs_s * 2);

  // The tile loads are written as inline assembly on purpose. Issued through the compiler's builtin they
  // are known to it as pending LDS writes, and it then puts `s_waitcnt vmcnt(0)` in front of the first V
  // fragment read of every tile (it cannot prove that the XOR-swizzled read addresses miss the buffer
  // being filled): the loads issued at the top of a tile, meant to land a whole tile later, were waited
  // for half a tile after issue. Here the ordering is explicit instead: one `s_waitcnt vmcnt(0)` and one
  // barrier at the end of each tile, before any wave reads the buffers those loads filled.
  auto dma_tile = [&](const u32x4_v& rsrc, const uint32_t(&voff)[IPW], uint32_t soff, char* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_p)(dst + wave * IPW * 1024)));
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds0 + i * 1024);
      // m0 (the LDS destination of the load) is a reserved register: naming it as clobbered draws a
      // warning per expansion, and leaving it out would hide the write from the compiler
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   :
                   : "s"(m0v), "v"(voff[i]), "s"(rsrc), "s"(soff)
                   : "memory", "m0");
#pragma clang diagnostic pop
    }
#endif
  };

  auto dma_v = [&](int jt, char* dst) {
    const bool second = jt >= v_split_tiles;
    dma_tile(second ? vrsrc2 : vrsrc, vvoff, static_cast<uint32_t>(second ? jt - v_split_tiles : jt) * v_tile_step, dst);
  };

  // ---- Q fragments stay in registers ----
  frag qf[KS];
  {
    int row = q0 + l32;
    row = row < p.Sq ? row : p.Sq - 1;
    const T* qp = qbase + row * p.qs_s + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(qp + ks * 16));
  }

  f32x16_v o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const float c = p.scale_log2;
  const uint8_t* mrow = p.mask ? p.mask + static_cast<int64_t>(b) * p.Sk : nullptr;

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

  auto mask_and_max = [&](int j, f32x16_v(&s)[2]) -> float {
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

  auto tile = [&](int j, f32x16_v(&s_cur)[2], f32x16_v(&s_next)[2]) {
    const int buf = j & 1;
    const bool has_next = j + 1 < n_tiles;
    // buffers K[buf] (held K(j), consumed last tile) and V[buf^1] (held V(j-1)) are free now
    if (j + 2 < n_tiles) dma_tile(krsrc, kvoff, static_cast<uint32_t>(j + 2) * k_tile_step, Kb + buf * TILEB);
    if (has_next) dma_v(j + 1, Vb + (buf ^ 1) * TILEB);

    const float mc = (m_run == -INFINITY) ? 0.f : m_run * c;
    uint32_t pf[2][2][4];
    float psum = 0.f;
    // Stage A mixes this wave's MFMAs with its exp2 work; giving it issue priority over the SIMD's other
    // wave (which is then mostly in its MFMA + LDS-read stage B) measured +5 % at 32760 keys, +9 % at
    // batch 1 / 4608 keys and nothing lost at the 4352-token, batch-2 shape.
    __builtin_amdgcn_s_setprio(2);
    // ---- stage A ----
    if (has_next) {
      const char* kt_base = Kb + (buf ^ 1) * TILEB;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s_next[kt][e] = 0.f;
      constexpr int KPF = ODIT_ATTN_KPF;  // K fragments in flight ahead of the MFMA that consumes them
      u32x4_v kfr[KPF + 1];
      auto k_fetch = [&](int i) {
        const int ks = i >> 1, kt = i & 1;
        kfr[i % (KPF + 1)] = *reinterpret_cast<const u32x4_v*>(kt_base + kt * 32 * ROWB + (k_lane ^ (ks * 32)));
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
#pragma unroll
      for (int pi = 0; pi < 16; ++pi) {
        const int pkt = pi >> 3, e0 = (pi & 7) * 2;
        const float p0 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0], c, -mc));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(s_cur[pkt][e0 + 1], c, -mc));
        psum += p0 + p1;
        pf[pkt][(pi & 7) >> 2][pi & 3] = M::pack2(p0, p1);
      }
    }
    l_run += psum;

    __builtin_amdgcn_s_setprio(0);
    // ---- stage B: O^T += V(j)^T P(j)^T ----
    // 4*DT steps, head-dim tile innermost so that consecutive MFMAs hit different accumulators and one
    // P fragment serves DT of them; the two transpose reads of step n + PF are issued before the MFMA
    // of step n, so LDS latency is covered by PF matrix instructions. The in-lane row maximum of
    // S(j+1) — vector work with nothing to wait for — is placed in the shadow of these MFMAs.
    const char* vt_base = Vb + buf * TILEB;
    constexpr int NSTEP = 4 * DT;
    constexpr int PF = ODIT_ATTN_VPF;
    s16x4_d vlo[PF + 1], vhi[PF + 1];
    auto v_fetch = [&](int step) {
      const int dt = step % DT, kt = (step / DT) >> 1, g2 = (step / DT) & 1;
      const char* vp = vt_base + (kt * 32 + g2 * 16) * ROWB + (v_lane ^ ((dt * 64) % ROWB));
      vlo[step % (PF + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_p)(vp));
      vhi[step % (PF + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_p)(vp + 8 * ROWB));
    };
    const bool plain_next = has_next && mrow == nullptr && (j + 2) * BN <= p.Sk;  // no exclusions in S(j+1)
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
      const float t = mask_and_max(j + 1, s_next);
      mx = fmaxf(t, __shfl_xor(t, 32, 64));
    }
    __builtin_amdgcn_s_waitcnt(0);  // this wave's tile loads have landed in LDS
    __syncthreads();
    if (has_next) settle_max(mx);
  };

  // ---- prologue (jt0 is even, so tile j always lives in buffer j & 1) ----
  dma_tile(krsrc, kvoff, static_cast<uint32_t>(jt0) * k_tile_step, Kb);
  dma_v(jt0, Vb);
  if (jt0 + 1 < n_tiles) dma_tile(krsrc, kvoff, static_cast<uint32_t>(jt0 + 1) * k_tile_step, Kb + TILEB);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  f32x16_v sa[2], sb[2];
  qk_plain(Kb, sa);
  {
    const float t = mask_and_max(jt0, sa);
    settle_max(fmaxf(t, __shfl_xor(t, 32, 64)));
  }

  for (int j = jt0; j < n_tiles; j += 2) {
    tile(j, sa, sb);
    if (j + 1 < n_tiles) tile(j + 1, sb, sa);
  }

  // ---- epilogue ----
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if constexpr (TAIL) {
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
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const int row = q0 + l32;
  if (row < p.Sq) {
    T* op = out_row_ptr<T>(p, b, h, row);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2_v w;
        w.x = M::pack2(o[dt][g * 4 + 0] * inv, o[dt][g * 4 + 1] * inv);
        w.y = M::pack2(o[dt][g * 4 + 2] * inv, o[dt][g * 4 + 3] * inv);
        *reinterpret_cast<u32x2_v*>(op + dt * 32 + g * 8 + hh * 4) = w;
      }
    if (p.lse != nullptr && hh == 0) {
      const float lse = l_tot > 0.f ? m_run * p.scale + __logf(l_tot) : -INFINITY;
      p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Sq + row] = lse;
    }
  }
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
  TailPlan t{0, 1, 0};
  if (ws != nullptr) {
    t = plan_tail(total, (p.Sk + 63) / 64, device_slots(NW));
    if (t.rem > 0) {
      if (ws_bytes < tail_ws_bytes(t, BM, D)) {
        set_error("odit_attn_fwd: workspace of %zu bytes given, %zu needed", ws_bytes, tail_ws_bytes(t, BM, D));
        return ODIT_EWORKSPACE;
      }
      if ((reinterpret_cast<uintptr_t>(ws) & 15) != 0) {
        set_error("odit_attn_fwd: workspace must be 16-byte aligned");
        return ODIT_EINVAL;
      }
      p.n_full = p.total_blocks - t.rem; p.key_chunks = t.key_chunks; p.tiles_per_chunk = t.tiles_per_chunk;
      p.ws = static_cast<float*>(ws);
    }
  }
  const int n_parts = t.rem * t.key_chunks;
  int rc = ODIT_OK;
  if (p.n_full > 0) {
    hipLaunchKernelGGL((attn_fwd_dma_kernel<T, D, NW, false>), dim3(p.n_full), dim3(NW * 64), 0, stream, p);
    rc = check_launch("odit_attn_fwd");
  }
  if (rc != ODIT_OK || n_parts == 0) return rc;
  // stream order puts these after the full rounds, when every slot is free again
  hipLaunchKernelGGL((attn_fwd_dma_kernel<T, D, NW, true>), dim3(n_parts), dim3(NW * 64), 0, stream, p);
  rc = check_launch("odit_attn_fwd (key-split tail)");
  if (rc != ODIT_OK) return rc;
  const int64_t rows = static_cast<int64_t>(t.rem) * BM;
  hipLaunchKernelGGL((attn_merge_kernel<T, D, BM>), dim3(static_cast<unsigned>((rows + 3) / 4)), dim3(256), 0,
                     stream, p, n_parts);
  return check_launch("odit_attn_fwd (merge)");
}

constexpr int kDmaWaves = 4;  // wavefronts per workgroup (two workgroups per compute unit)

size_t attn_dma_workspace_bytes(int B, int Sq, int Sk, int H, int D) {
  if (B <= 0 || Sq <= 0 || Sk <= 0 || H <= 0) return 0;
  constexpr int nw = kDmaWaves;
  const int bm = nw * 32;
  const int64_t units = static_cast<int64_t>((Sq + bm - 1) / bm) * H * B;
  return tail_ws_bytes(plan_tail(units, (Sk + 63) / 64, device_slots(nw)), bm, D);
}

// 32-bit buffer offsets: the whole key range of one (batch, head) must be addressable
bool attn_dma_addressable(int Sk, int64_t k_seq_stride, int64_t v_seq_stride) {
  const int64_t k_span = (static_cast<int64_t>(Sk) + 64) * k_seq_stride * 2;
  const int64_t v_span = (static_cast<int64_t>(Sk) + 64) * v_seq_stride * 2;
  return k_span < (1ll << 31) && v_span < (1ll << 31) && k_seq_stride >= 0 && v_seq_stride >= 0;
}

int attn_dma_plan(int B, int Sq, int Sk, int H, int D, bool with_workspace, char* text, size_t text_bytes) {
  constexpr int bm = kDmaWaves * 32;
  const int64_t units = static_cast<int64_t>((Sq + bm - 1) / bm) * H * B;
  TailPlan t{0, 1, 0};
  if (with_workspace) t = plan_tail(units, (Sk + 63) / 64, device_slots(kDmaWaves));
  if (t.rem == 0) {
    snprintf(text, text_bytes, "attn_fwd_dma_kernel<T, %d, %d, false> units=%lld", D, kDmaWaves, static_cast<long long>(units));
    return 1;
  }
  // kernel names as a profiler prints them, with T for the element type
  snprintf(text, text_bytes, "attn_fwd_dma_kernel<T, %d, %d, false> units=%lld; attn_fwd_dma_kernel<T, %d, %d, true> "
           "units=%d x %d key ranges of %d tiles; attn_merge_kernel<T, %d, %d> rows=%d", D, kDmaWaves,
           static_cast<long long>(units - t.rem), D, kDmaWaves, t.rem, t.key_chunks, t.tiles_per_chunk, D, bm, t.rem * bm);
  return units - t.rem > 0 ? 3 : 2;
}

int launch_attn_dma(AttnParams& p, int dtype, int D, hipStream_t stream, void* ws, size_t ws_bytes) {
  if (!attn_dma_addressable(p.Sk, p.ks_s, p.vs_s)) return ODIT_ENOTSUP;
#define ODIT_DMA_GO(T)                                                                     \
  if (D == 128) return launch_dma<T, 128, kDmaWaves>(p, stream, ws, ws_bytes);                \
  return launch_dma<T, 64, kDmaWaves>(p, stream, ws, ws_bytes);
  if (dtype == ODIT_BF16) { ODIT_DMA_GO(bf16_t) }
  ODIT_DMA_GO(f16_t)
#undef ODIT_DMA_GO
}

}  // namespace odit
