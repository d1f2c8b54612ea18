// K1 entry points, and the pointer-addressed attention kernel used when the key/value rows of one
// (batch, head) span 2 GiB or more and so cannot be reached through 32-bit buffer offsets (the
// production kernel of attn_fwd_dma.hip). Both kernels share the formulation:
//     S^T = K Q^T          v_mfma_f32_32x32x16:  A = K tile rows (from LDS), B = Q rows (registers)
//     O^T = V^T P^T        v_mfma_f32_32x32x16:  A = V^T rows (from LDS),  B = P^T (registers)
// In the 32x32 accumulator layout lane l owns column (l & 31) — one QUERY — and 16 rows — KEYS
// 8g + 4(l>>5) + t, g,t in 0..3.  So a query's running max / sum need only in-lane work plus one
// exchange between lanes l and l^32, and the P^T accumulators are, after conversion to 16-bit,
// already in B-operand order for the second product as long as V^T is read from LDS with the same
// permutation of the summation (key) index.  P never touches LDS.
//
// Work decomposition: grid = B * H * ceil(Sq / BM) workgroups; each wavefront owns 32 queries and
// streams all keys in tiles of 64 through a double-buffered LDS stage. Workgroup ids are remapped so
// that the q-blocks of one (batch, head) — which share K/V — land on the same XCD and hit its L2.
//
// Algorithmic work: 4 * B * H * Sq * Sk * D flop; minimum traffic 2 * (2*B*Sq*H*D + 2*B*Sk*Hkv*D) bytes.
#include "attn_common.h"

#include <string.h>

namespace odit {

// ------------------------------------------------------------------------------------------------
// Pointer-addressed, software-pipelined kernel (one 32-query tile per wavefront; tiles are staged
// through registers with ordinary 64-bit addressed loads, so any tensor extent works).
//
// Per key tile j a wavefront runs two stages:
//   A:  S(j+1)^T = K(j+1) Q^T on the matrix cores   while the vector ALU turns S(j) into P(j)
//       (exp2, row sums, 16-bit packing) — the two instruction streams are independent and are
//       written interleaved, one MFMA per seven vector instructions;
//   B:  O^T += V(j)^T P(j)^T.
// The row maximum of S(j+1) and the (rare) rescale of O are settled between B and the next A.
// K runs one tile ahead of V through the double-buffered LDS stage, so one barrier per tile is
// enough. V stays row-major in LDS; its transposed A fragments come from ds_read_b64_tr_b16, whose
// 16-lane transpose delivers, for lane i of a group, element (i % 4) of the 8-byte words fetched by
// lanes 4k + i/4 (k = 0..3): four consecutive keys of one head-dim column.
// ------------------------------------------------------------------------------------------------
typedef short s16x4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4_v* lds_s16x4_ptr;

template <typename T, int D, int NW>
__global__ __launch_bounds__(NW * 64, 8 / NW) void attn_fwd_pipe_kernel(const AttnParams p) {
  using M = Mma<T>;
  using frag = typename M::frag;
  constexpr int BN = 64;
  constexpr int NT = NW * 64;
  constexpr int BM = NW * 32;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int KROW = D + 8;    // +16 B per row: the 16 lanes of a quarter-wave b128 read cover all banks
  constexpr int VROW = D + 32;   // +64 B per row: the 4 keys x 4 words of a transpose read cover disjoint banks
  constexpr int CPR = D / 8;
  constexpr int TCH = BN * CPR;  // 16-byte chunks per tile
  constexpr int TPT = (TCH + NT - 1) / NT;

  __shared__ __attribute__((aligned(16))) T Ks[2][BN * KROW];
  __shared__ __attribute__((aligned(16))) T Vs[2][BN * VROW];

  const int pid = xcd_remap(blockIdx.x, p.total_blocks);
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

  frag qf[KS];
  {
    int row = q0 + l32;
    row = row < p.Sq ? row : p.Sq - 1;
    const T* qp = qbase + row * p.qs_s + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks] = __builtin_bit_cast(frag, *reinterpret_cast<const u32x4_v*>(qp + ks * 16));
  }

  u32x4_v kreg[TPT], vreg[TPT];
  auto gload = [&](const T* base, int64_t stride_s, int j, u32x4_v(&reg)[TPT]) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int c = tid + i * NT;
      if (TCH % NT == 0 || c < TCH) {
        int key = j * BN + c / CPR;
        key = key < p.Sk ? key : p.Sk - 1;
        reg[i] = *reinterpret_cast<const u32x4_v*>(base + key * stride_s + (c % CPR) * 8);
      }
    }
  };
  auto sstore = [&](T* dst, int pitch, const u32x4_v(&reg)[TPT]) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int c = tid + i * NT;
      if (TCH % NT == 0 || c < TCH)
        *reinterpret_cast<u32x4_v*>(dst + (c / CPR) * pitch + (c % CPR) * 8) = reg[i];
    }
  };

  f32x16_v o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int n_tiles = (p.Sk + BN - 1) / BN;
  const float c = p.scale_log2;
  const uint8_t* mrow = p.mask ? p.mask + static_cast<int64_t>(b) * p.Sk : nullptr;
  const int k_off = l32 * KROW + hh * 8;                                       // K fragment, per lane
  const int v_off = (((lane & 15) >> 2) + 4 * hh) * VROW + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // S^T tile = K(tile in Ks[buf]) Q^T, no softmax work to overlap (prologue only)
  auto qk_plain = [&](int buf, f32x16_v(&s)[2]) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kt][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const frag a = __builtin_bit_cast(
            frag, *reinterpret_cast<const u32x4_v*>(&Ks[buf][kt * 32 * KROW + k_off + ks * 16]));
        s[kt] = M::run(a, qf[ks], s[kt]);
      }
  };

  // exclusions (keys past Sk, padding mask), then the lane-local part of the row maximum
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

  // move the reference maximum (and rescale O, l) only when some query outgrew it by more than 2^8
  auto settle_max = [&](float mx) {
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
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

  // one tile: s_cur holds S(j) (max already settled); s_next receives S(j+1)
  auto tile = [&](int j, f32x16_v(&s_cur)[2], f32x16_v(&s_next)[2]) {
    const int buf = j & 1;
    const bool has_next = j + 1 < n_tiles;
    if (j + 2 < n_tiles) gload(kbase, p.ks_s, j + 2, kreg);
    if (has_next) gload(vbase, p.vs_s, j + 1, vreg);

    const float mc = (m_run == -INFINITY) ? 0.f : m_run * c;
    uint32_t pf[2][2][4];
    float psum = 0.f;
    // ---- stage A ----
    if (has_next) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s_next[kt][e] = 0.f;
#pragma unroll
      for (int i = 0; i < 2 * KS; ++i) {
        const int ks = i >> 1, kt = i & 1;
        const frag a = __builtin_bit_cast(
            frag, *reinterpret_cast<const u32x4_v*>(&Ks[buf ^ 1][kt * 32 * KROW + k_off + ks * 16]));
        s_next[kt] = M::run(a, qf[ks], s_next[kt]);
        // 32 / (2*KS) score pairs of S(j) per MFMA
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

    // ---- stage B: O^T += V(j)^T P(j)^T ----
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int g2 = 0; g2 < 2; ++g2) {
          T* vp = &Vs[buf][(kt * 32 + g2 * 16) * VROW + dt * 32 + v_off];
          const s16x4_v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(vp));
          const s16x4_v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(vp + 8 * VROW));
          typedef short s16x8_v __attribute__((ext_vector_type(8)));
          const s16x8_v av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          u32x4_v pb;
          pb.x = pf[kt][g2][0]; pb.y = pf[kt][g2][1]; pb.z = pf[kt][g2][2]; pb.w = pf[kt][g2][3];
          o[dt] = M::run(__builtin_bit_cast(frag, av), __builtin_bit_cast(frag, pb), o[dt]);
        }

    float mx = -INFINITY;
    if (has_next) mx = mask_and_max(j + 1, s_next);
    if (j + 2 < n_tiles) sstore(&Ks[buf][0], KROW, kreg);
    if (has_next) sstore(&Vs[buf ^ 1][0], VROW, vreg);
    __syncthreads();
    if (has_next) settle_max(mx);
  };

  // ---- prologue: K(0), V(0), K(1) staged; S(0) computed and its maximum settled ----
  gload(kbase, p.ks_s, 0, kreg);
  gload(vbase, p.vs_s, 0, vreg);
  sstore(&Ks[0][0], KROW, kreg);
  sstore(&Vs[0][0], VROW, vreg);
  if (n_tiles > 1) {
    gload(kbase, p.ks_s, 1, kreg);
    sstore(&Ks[1][0], KROW, kreg);
  }
  __syncthreads();
  f32x16_v sa[2], sb[2];
  qk_plain(0, sa);
  settle_max(mask_and_max(0, sa));

  for (int j = 0; j < n_tiles; j += 2) {
    tile(j, sa, sb);
    if (j + 1 < n_tiles) tile(j + 1, sb, sa);
  }

  // ---- epilogue ----
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
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
static int launch_attn_pipe(AttnParams& p, hipStream_t stream) {
  constexpr int BM = NW * 32;
  p.n_qblocks = (p.Sq + BM - 1) / BM;
  const int64_t total = static_cast<int64_t>(p.n_qblocks) * p.H * p.B;
  if (total > 0x7fffffffll) {
    set_error("odit_attn_fwd: grid of %lld workgroups is too large", static_cast<long long>(total));
    return ODIT_EINVAL;
  }
  p.total_blocks = static_cast<int>(total);
  hipLaunchKernelGGL((attn_fwd_pipe_kernel<T, D, NW>), dim3(p.total_blocks), dim3(NW * 64), 0, stream, p);
  return check_launch("odit_attn_fwd");
}

}  // namespace odit

extern "C" int odit_attn_fwd_ex(const void* q, const void* k, const void* v, const void* v_tail, int k_split,
                                void* o, void* o_tail, int q_split, const uint8_t* key_mask, float* lse,
                                int B, int Sq, int Sk, int H, int Hkv, int D, const int64_t q_strides[3],
                                const int64_t k_strides[3], const int64_t v_strides[3],
                                const int64_t v_tail_strides[3], const int64_t o_strides[3],
                                const int64_t o_tail_strides[3], float scale, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream);

extern "C" int odit_attn_fwd(const void* q, const void* k, const void* v, void* o,
                             const uint8_t* key_mask, float* lse, int B, int Sq, int Sk, int H,
                             int Hkv, int D, const int64_t q_strides[3], const int64_t k_strides[3],
                             const int64_t v_strides[3], const int64_t o_strides[3], float scale,
                             int dtype, void* stream) {
  return odit_attn_fwd_ex(q, k, v, nullptr, 0, o, nullptr, 0, key_mask, lse, B, Sq, Sk, H, Hkv, D, q_strides,
                          k_strides, v_strides, nullptr, o_strides, nullptr, scale, dtype, nullptr, 0, stream);
}

extern "C" size_t odit_attn_fwd_workspace_bytes(int B, int Sq, int Sk, int H, int D) {
  if (D != 64 && D != 128) return 0;
  return odit::attn_dma_workspace_bytes(B, Sq, Sk, H, D);
}

extern "C" int odit_attn_fwd_plan(int B, int Sq, int Sk, int H, int D, int64_t k_seq_stride, int64_t v_seq_stride,
                                  int with_workspace, char* text, size_t text_bytes) {
  using namespace odit;
  ODIT_CHECK_ARG(text != nullptr && text_bytes > 0, "odit_attn_fwd_plan: no text buffer");
  ODIT_CHECK_ARG(B > 0 && Sq > 0 && Sk > 0 && H > 0 && (D == 64 || D == 128), "odit_attn_fwd_plan: bad shape");
  if (attn_dma_addressable(Sk, D, k_seq_stride, v_seq_stride))
    return attn_dma_plan(B, Sq, Sk, H, D, with_workspace != 0, text, text_bytes);
  const int64_t units = static_cast<int64_t>((Sq + 255) / 256) * H * B;
  snprintf(text, text_bytes, "attn_fwd_pipe_kernel<T, %d, 8> units=%lld", D, static_cast<long long>(units));
  return 1;
}

extern "C" int odit_attn_fwd_ex(const void* q, const void* k, const void* v, const void* v_tail, int k_split,
                                void* o, void* o_tail, int q_split, const uint8_t* key_mask, float* lse,
                                int B, int Sq, int Sk, int H, int Hkv, int D, const int64_t q_strides[3],
                                const int64_t k_strides[3], const int64_t v_strides[3],
                                const int64_t v_tail_strides[3], const int64_t o_strides[3],
                                const int64_t o_tail_strides[3], float scale, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream) {
  using namespace odit;
  if (o_tail != nullptr) {
    ODIT_CHECK_ARG(o_tail_strides != nullptr, "odit_attn_fwd_ex: o_tail given without strides");
    ODIT_CHECK_ARG(q_split >= 0 && q_split <= Sq, "odit_attn_fwd_ex: q_split=%d outside [0, Sq=%d]", q_split, Sq);
    ODIT_CHECK_ARG(aligned16(o_tail) && o_tail_strides[0] % 8 == 0 && o_tail_strides[1] % 8 == 0 &&
                       o_tail_strides[2] % 8 == 0,
                   "odit_attn_fwd_ex: o_tail must be 16-byte aligned with strides multiple of 8");
  }
  if (v_tail != nullptr) {
    ODIT_CHECK_ARG(v_tail_strides != nullptr && v_strides != nullptr, "odit_attn_fwd_ex: v_tail given without strides");
    ODIT_CHECK_ARG(k_split > 0 && k_split < Sk && k_split % 64 == 0,
                   "odit_attn_fwd_ex: k_split=%d must be a multiple of 64 inside (0, Sk=%d)", k_split, Sk);
    ODIT_CHECK_ARG(v_tail_strides[1] == v_strides[1],
                   "odit_attn_fwd_ex: v and v_tail must share the row stride (%lld vs %lld)",
                   static_cast<long long>(v_strides[1]), static_cast<long long>(v_tail_strides[1]));
    ODIT_CHECK_ARG(aligned16(v_tail) && v_tail_strides[0] % 8 == 0 && v_tail_strides[2] % 8 == 0,
                   "odit_attn_fwd_ex: v_tail must be 16-byte aligned with strides multiple of 8");
  }
  ODIT_CHECK_ARG(q && k && v && o, "odit_attn_fwd: q/k/v/o must not be null");
  ODIT_CHECK_ARG(q_strides && k_strides && v_strides && o_strides, "odit_attn_fwd: null strides");
  ODIT_CHECK_ARG(B >= 0 && Sq >= 0 && Sk >= 0 && H > 0 && Hkv > 0, "odit_attn_fwd: bad shape");
  ODIT_CHECK_ARG(H % Hkv == 0, "odit_attn_fwd: H=%d is not a multiple of Hkv=%d", H, Hkv);
  ODIT_CHECK_ARG(scale > 0.f, "odit_attn_fwd: softmax scale must be positive (got %g)", scale);
  if (dtype != ODIT_BF16 && dtype != ODIT_F16) {
    set_error("odit_attn_fwd: dtype code %d unsupported (bf16 and fp16 only)", dtype);
    return ODIT_ENOTSUP;
  }
  if (D != 64 && D != 128) {
    set_error("odit_attn_fwd: head size %d unsupported (64 and 128 only)", D);
    return ODIT_ENOTSUP;
  }
  ODIT_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o),
                 "odit_attn_fwd: q/k/v/o must be 16-byte aligned");
  for (int i = 0; i < 3; ++i) {
    ODIT_CHECK_ARG(q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 &&
                       o_strides[i] % 8 == 0,
                   "odit_attn_fwd: strides must be multiples of 8 elements");
  }
  if (B == 0 || Sq == 0) return ODIT_OK;
  ODIT_CHECK_ARG(Sk > 0, "odit_attn_fwd: Sk must be positive when there are queries");

  AttnParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.mask = key_mask; p.lse = lse;
  p.B = B; p.Sq = Sq; p.Sk = Sk; p.H = H; p.Hkv = Hkv;
  p.qs_b = q_strides[0]; p.qs_s = q_strides[1]; p.qs_h = q_strides[2];
  p.ks_b = k_strides[0]; p.ks_s = k_strides[1]; p.ks_h = k_strides[2];
  p.vs_b = v_strides[0]; p.vs_s = v_strides[1]; p.vs_h = v_strides[2];
  p.os_b = o_strides[0]; p.os_s = o_strides[1]; p.os_h = o_strides[2];
  p.scale = scale;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.o_tail = o_tail; p.q_split = q_split;
  p.ts_b = o_tail ? o_tail_strides[0] : 0; p.ts_s = o_tail ? o_tail_strides[1] : 0; p.ts_h = o_tail ? o_tail_strides[2] : 0;

  p.v_tail = v_tail; p.k_split = v_tail ? k_split : 0;
  p.vt_b = v_tail ? v_tail_strides[0] : 0; p.vt_h = v_tail ? v_tail_strides[2] : 0;

  p.n_full = 0; p.key_chunks = 1; p.tiles_per_chunk = 0; p.ws = nullptr;

  hipStream_t st = static_cast<hipStream_t>(stream);
  const int rc = launch_attn_dma(p, dtype, D, st, workspace, workspace_bytes);
  if (rc != ODIT_ENOTSUP) return rc;
  // key/value spans of 2 GiB or more per (batch, head): the pointer-addressed kernel
  if (v_tail != nullptr) {
    set_error("odit_attn_fwd_ex: values in two tensors need key/value spans below 2 GiB per batch and head");
    return ODIT_ENOTSUP;
  }
  constexpr int kPtrWaves = 8;
  if (dtype == ODIT_BF16) {
    return D == 128 ? launch_attn_pipe<bf16_t, 128, kPtrWaves>(p, st) : launch_attn_pipe<bf16_t, 64, kPtrWaves>(p, st);
  }
  return D == 128 ? launch_attn_pipe<f16_t, 128, kPtrWaves>(p, st) : launch_attn_pipe<f16_t, 64, kPtrWaves>(p, st);
}
