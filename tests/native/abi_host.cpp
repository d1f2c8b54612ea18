// A host program with no Python and no torch in it: it links libomni_dit_hip.so through include/omni_dit.h,
// owns its device buffers through the HIP runtime, and checks five entry points against loops written here
// (double precision on the CPU). It is what a non-Python caller of the C ABI looks like; the GPU test
// tests/test_gpu_native_host.py runs it as a child process and reads its exit status.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "omni_dit.h"

#define HIP_OK(call)                                                                          \
  do {                                                                                        \
    const hipError_t e__ = (call);                                                            \
    if (e__ != hipSuccess) {                                                                  \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e__));                 \
      return 2;                                                                               \
    }                                                                                         \
  } while (0)
#define ODIT_OK_OR_FAIL(call)                                                                 \
  do {                                                                                        \
    const int rc__ = (call);                                                                  \
    if (rc__ != 0) {                                                                          \
      std::fprintf(stderr, "%s returned %d: %s\n", #call, rc__, odit_last_error());           \
      return 3;                                                                               \
    }                                                                                         \
  } while (0)

static uint32_t g_state = 12345u;
static float next_uniform() {  // (-1, 1), same sequence on every run
  g_state = g_state * 1664525u + 1013904223u;
  return static_cast<float>(g_state >> 8) * (2.0f / 16777216.0f) - 1.0f;
}
static uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}
static float from_bf16(uint16_t h) {
  const uint32_t u = static_cast<uint32_t>(h) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

template <typename T> struct DeviceBuffer {
  T* p = nullptr;
  ~DeviceBuffer() { if (p) (void)hipFree(p); }
  hipError_t alloc(size_t n) { return hipMalloc(reinterpret_cast<void**>(&p), n * sizeof(T)); }
};

static int check_rel_l1(hipStream_t st) {
  const int B = 2;
  const int64_t n = 5000;  // not a multiple of the vector width
  std::vector<uint16_t> cur(B * n), prev(B * n);
  for (auto& v : cur) v = to_bf16(next_uniform());
  for (auto& v : prev) v = to_bf16(next_uniform());
  DeviceBuffer<uint16_t> d_cur, d_prev;
  DeviceBuffer<double> d_sums;
  DeviceBuffer<char> d_ws;
  const size_t ws = odit_rel_l1_workspace_bytes(B, n);
  HIP_OK(d_cur.alloc(cur.size())); HIP_OK(d_prev.alloc(prev.size())); HIP_OK(d_sums.alloc(2 * B));
  HIP_OK(d_ws.alloc(ws > 0 ? ws : 16));
  HIP_OK(hipMemset(d_ws.p, 0, ws > 0 ? ws : 16));  // the ticket counters start at zero; calls keep them there
  HIP_OK(hipMemcpy(d_cur.p, cur.data(), cur.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_prev.p, prev.data(), prev.size() * 2, hipMemcpyHostToDevice));
  double got[4], first[4];
  for (int rep = 0; rep < 2; ++rep) {  // the second call reuses the workspace as the first one left it
    ODIT_OK_OR_FAIL(odit_rel_l1(d_cur.p, d_prev.p, d_sums.p, d_ws.p, ws, B, n, n, n, ODIT_BF16, 0, st));
    HIP_OK(hipStreamSynchronize(st));
    HIP_OK(hipMemcpy(got, d_sums.p, sizeof(got), hipMemcpyDeviceToHost));
    if (rep == 0) std::memcpy(first, got, sizeof(got));
  }
  if (std::memcmp(first, got, sizeof(got)) != 0) {
    std::fprintf(stderr, "rel_l1: two calls on one workspace differ\n");
    return 1;
  }
  for (int b = 0; b < B; ++b) {
    double sd = 0.0, sp = 0.0;
    for (int64_t i = 0; i < n; ++i) {
      const double c = from_bf16(cur[b * n + i]), p = from_bf16(prev[b * n + i]);
      sd += std::fabs(c - p);
      sp += std::fabs(p);
    }
    if (std::fabs(got[2 * b] - sd) > 1e-5 * sd || std::fabs(got[2 * b + 1] - sp) > 1e-5 * sp) {
      std::fprintf(stderr, "rel_l1 row %d: got (%.9g, %.9g), want (%.9g, %.9g)\n", b, got[2 * b], got[2 * b + 1], sd, sp);
      return 1;
    }
  }
  std::printf("odit_rel_l1: ok\n");
  return 0;
}

static int check_gated_residual(hipStream_t st) {
  const int B = 2, S = 7, C = 40;
  std::vector<float> h(B * S * C), y(B * S * C), gate(B * C), out(B * S * C);
  for (auto& v : h) v = next_uniform();
  for (auto& v : y) v = next_uniform();
  for (auto& v : gate) v = next_uniform();
  DeviceBuffer<float> d_h, d_y, d_g, d_o;
  HIP_OK(d_h.alloc(h.size())); HIP_OK(d_y.alloc(y.size())); HIP_OK(d_g.alloc(gate.size())); HIP_OK(d_o.alloc(out.size()));
  HIP_OK(hipMemcpy(d_h.p, h.data(), h.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_y.p, y.data(), y.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_g.p, gate.data(), gate.size() * 4, hipMemcpyHostToDevice));
  const int64_t dense[2] = {static_cast<int64_t>(S) * C, C}, per_batch[2] = {C, 0};
  ODIT_OK_OR_FAIL(odit_gated_residual(d_h.p, d_y.p, d_g.p, nullptr, d_o.p, B, S, C, dense, dense, dense, per_batch,
                                      ODIT_F32, ODIT_F32, 0, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(out.data(), d_o.p, out.size() * 4, hipMemcpyDeviceToHost));
  for (int b = 0; b < B; ++b)
    for (int s = 0; s < S; ++s)
      for (int c = 0; c < C; ++c) {
        const int i = (b * S + s) * C + c;
        const double want = static_cast<double>(h[i]) + static_cast<double>(gate[b * C + c]) * y[i];
        if (std::fabs(out[i] - want) > 1e-6) {
          std::fprintf(stderr, "gated_residual (%d,%d,%d): got %.9g, want %.9g\n", b, s, c, out[i], want);
          return 1;
        }
      }
  std::printf("odit_gated_residual: ok\n");
  return 0;
}

static int check_attention(hipStream_t st) {
  const int B = 1, Sq = 70, Sk = 130, H = 2, D = 64;  // ragged in queries and keys
  const float scale = 0.125f;
  std::vector<uint16_t> q(B * Sq * H * D), k(B * Sk * H * D), v(B * Sk * H * D), o(B * Sq * H * D);
  for (auto& x : q) x = to_bf16(2.0f * next_uniform());
  for (auto& x : k) x = to_bf16(2.0f * next_uniform());
  for (auto& x : v) x = to_bf16(next_uniform());
  DeviceBuffer<uint16_t> d_q, d_k, d_v, d_o;
  HIP_OK(d_q.alloc(q.size())); HIP_OK(d_k.alloc(k.size())); HIP_OK(d_v.alloc(v.size())); HIP_OK(d_o.alloc(o.size()));
  HIP_OK(hipMemcpy(d_q.p, q.data(), q.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_k.p, k.data(), k.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_v.p, v.data(), v.size() * 2, hipMemcpyHostToDevice));
  const int64_t qs[3] = {static_cast<int64_t>(Sq) * H * D, H * D, D}, ks[3] = {static_cast<int64_t>(Sk) * H * D, H * D, D};
  ODIT_OK_OR_FAIL(odit_attn_fwd(d_q.p, d_k.p, d_v.p, d_o.p, nullptr, nullptr, B, Sq, Sk, H, H, D, qs, ks, ks, qs, scale,
                                ODIT_BF16, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(o.data(), d_o.p, o.size() * 2, hipMemcpyDeviceToHost));
  double worst = 0.0;
  std::vector<double> s(Sk);
  for (int h = 0; h < H; ++h)
    for (int i = 0; i < Sq; ++i) {
      double m = -1e300;
      for (int j = 0; j < Sk; ++j) {
        double acc = 0.0;
        for (int d = 0; d < D; ++d) acc += static_cast<double>(from_bf16(q[(i * H + h) * D + d])) * from_bf16(k[(j * H + h) * D + d]);
        s[j] = acc * scale;
        m = s[j] > m ? s[j] : m;
      }
      double l = 0.0;
      for (int j = 0; j < Sk; ++j) { s[j] = std::exp(s[j] - m); l += s[j]; }
      for (int d = 0; d < D; ++d) {
        double acc = 0.0;
        for (int j = 0; j < Sk; ++j) acc += s[j] * from_bf16(v[(j * H + h) * D + d]);
        const double err = std::fabs(from_bf16(o[(i * H + h) * D + d]) - acc / l);
        worst = err > worst ? err : worst;
      }
    }
  if (!(worst <= 2e-2)) {  // bf16 output, probabilities rounded to bf16 inside the kernel
    std::fprintf(stderr, "attention: max abs error %.4g\n", worst);
    return 1;
  }
  // an unsupported head size must be refused before any launch, with a message
  const int rc = odit_attn_fwd(d_q.p, d_k.p, d_v.p, d_o.p, nullptr, nullptr, B, Sq, Sk, H, H, 96, qs, ks, ks, qs, scale, ODIT_BF16, st);
  if (rc == 0 || std::strlen(odit_last_error()) == 0) {
    std::fprintf(stderr, "attention: head size 96 was not refused\n");
    return 1;
  }
  std::printf("odit_attn_fwd: ok (max abs error %.4g; head size 96 refused: %s)\n", worst, odit_last_error());
  return 0;
}

static int check_adaln(hipStream_t st) {
  const int B = 2, S = 5, C = 96;
  const float eps = 1e-6f;
  std::vector<float> x(B * S * C), shift(B * C), scale(B * C), out(B * S * C);
  for (auto& v : x) v = 3.0f * next_uniform() + 0.5f;
  for (auto& v : shift) v = 0.5f * next_uniform();
  for (auto& v : scale) v = 0.5f * next_uniform();
  DeviceBuffer<float> d_x, d_sh, d_sc, d_o;
  HIP_OK(d_x.alloc(x.size())); HIP_OK(d_sh.alloc(shift.size())); HIP_OK(d_sc.alloc(scale.size())); HIP_OK(d_o.alloc(out.size()));
  HIP_OK(hipMemcpy(d_x.p, x.data(), x.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_sh.p, shift.data(), shift.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_sc.p, scale.data(), scale.size() * 4, hipMemcpyHostToDevice));
  const int64_t dense[2] = {static_cast<int64_t>(S) * C, C};
  ODIT_OK_OR_FAIL(odit_adaln_modulate(d_x.p, d_o.p, d_sh.p, d_sc.p, nullptr, nullptr, nullptr, nullptr, nullptr, B, S, C,
                                      dense, dense, C, 0, eps, ODIT_F32, ODIT_F32, 0, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(out.data(), d_o.p, out.size() * 4, hipMemcpyDeviceToHost));
  for (int b = 0; b < B; ++b)
    for (int s = 0; s < S; ++s) {
      const float* row = &x[(b * S + s) * C];
      double mean = 0.0, var = 0.0;
      for (int c = 0; c < C; ++c) mean += row[c];
      mean /= C;
      for (int c = 0; c < C; ++c) var += (row[c] - mean) * (row[c] - mean);
      const double rstd = 1.0 / std::sqrt(var / C + eps);
      for (int c = 0; c < C; ++c) {
        const double want = (row[c] - mean) * rstd * (1.0 + scale[b * C + c]) + shift[b * C + c];
        if (std::fabs(out[(b * S + s) * C + c] - want) > 1e-4) {
          std::fprintf(stderr, "adaln (%d,%d,%d): got %.9g, want %.9g\n", b, s, c, out[(b * S + s) * C + c], want);
          return 1;
        }
      }
    }
  std::printf("odit_adaln_modulate: ok\n");
  return 0;
}

static int check_qknorm_rope(hipStream_t st) {
  // q and k are two thirds of a fused [B,S,3,H,D] projection output; they land at rows off.. of joint buffers
  const int B = 2, S = 9, H = 3, D = 64, off = 4, S_total = S + off;
  const float eps = 1e-6f;
  std::vector<float> qkv(B * S * 3 * H * D), wq(D), wk(D), cs(S * D / 2), sn(S * D / 2);
  std::vector<float> jq(B * S_total * H * D, 0.f), jk(jq);
  for (auto& v : qkv) v = 2.0f * next_uniform();
  for (auto& v : wq) v = 1.0f + 0.2f * next_uniform();
  for (auto& v : wk) v = 1.0f + 0.2f * next_uniform();
  for (int i = 0; i < S * D / 2; ++i) { const float a = 3.0f * next_uniform(); cs[i] = std::cos(a); sn[i] = std::sin(a); }
  DeviceBuffer<float> d_qkv, d_wq, d_wk, d_cs, d_sn, d_jq, d_jk;
  HIP_OK(d_qkv.alloc(qkv.size())); HIP_OK(d_wq.alloc(D)); HIP_OK(d_wk.alloc(D)); HIP_OK(d_cs.alloc(cs.size()));
  HIP_OK(d_sn.alloc(sn.size())); HIP_OK(d_jq.alloc(jq.size())); HIP_OK(d_jk.alloc(jk.size()));
  HIP_OK(hipMemcpy(d_qkv.p, qkv.data(), qkv.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_wq.p, wq.data(), D * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_wk.p, wk.data(), D * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_cs.p, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_sn.p, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(d_jq.p, 0, jq.size() * 4));
  HIP_OK(hipMemset(d_jk.p, 0, jk.size() * 4));
  const int64_t in_strides[2] = {static_cast<int64_t>(S) * 3 * H * D, 3 * H * D};
  ODIT_OK_OR_FAIL(odit_qknorm_rope(d_qkv.p, d_qkv.p + H * D, nullptr, d_jq.p, d_jk.p, nullptr, d_wq.p, d_wk.p, d_cs.p, d_sn.p,
                                   B, S, H, D, D, in_strides, off, S_total, eps, ODIT_NORM_HEAD, ODIT_F32, ODIT_F32, 0, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(jq.data(), d_jq.p, jq.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(jk.data(), d_jk.p, jk.size() * 4, hipMemcpyDeviceToHost));
  for (int part = 0; part < 2; ++part) {
    const std::vector<float>& got = part == 0 ? jq : jk;
    const std::vector<float>& w = part == 0 ? wq : wk;
    for (int b = 0; b < B; ++b)
      for (int s = 0; s < S_total; ++s)
        for (int h = 0; h < H; ++h) {
          const float* g = &got[((b * S_total + s) * H + h) * D];
          if (s < off) {  // rows in front of the offset belong to another stream: untouched
            for (int d = 0; d < D; ++d) if (g[d] != 0.f) { std::fprintf(stderr, "qknorm: row %d written\n", s); return 1; }
            continue;
          }
          const float* in = &qkv[(((b * S + (s - off)) * 3 + part) * H + h) * D];
          double ms = 0.0;
          for (int d = 0; d < D; ++d) ms += static_cast<double>(in[d]) * in[d];
          const double rstd = 1.0 / std::sqrt(ms / D + eps);
          for (int i = 0; i < D / 2; ++i) {
            const double x0 = in[2 * i] * rstd * w[2 * i], x1 = in[2 * i + 1] * rstd * w[2 * i + 1];
            const double c = cs[(s - off) * (D / 2) + i], sv = sn[(s - off) * (D / 2) + i];
            if (std::fabs(g[2 * i] - (x0 * c - x1 * sv)) > 1e-4 || std::fabs(g[2 * i + 1] - (x1 * c + x0 * sv)) > 1e-4) {
              std::fprintf(stderr, "qknorm part %d (%d,%d,%d,%d)\n", part, b, s, h, i);
              return 1;
            }
          }
        }
  }
  std::printf("odit_qknorm_rope: ok\n");
  return 0;
}

// odit_linear_rows on the hand-written kernel: x [2 x 96, 128] W [192, 128]^T, bf16, one float32 gate vector per
// 96 rows, pre-scaled bias, accumulated onto a residual; checked against a double-precision loop.
static int check_linear_rows(hipStream_t st) {
  const int B = 2, S = 96, M = B * S, N = 192, K = 128;
  std::vector<uint16_t> x(M * K), w(N * K), res(M * N), out(M * N);
  std::vector<float> gate(B * N), gbias(B * N);
  for (auto& v : x) v = to_bf16(next_uniform());
  for (auto& v : w) v = to_bf16(0.1f * next_uniform());
  for (auto& v : res) v = to_bf16(next_uniform());
  for (auto& v : gate) v = next_uniform();
  for (auto& v : gbias) v = 0.1f * next_uniform();
  DeviceBuffer<uint16_t> d_x, d_w, d_r, d_o;
  DeviceBuffer<float> d_g, d_b;
  DeviceBuffer<unsigned char> d_ws;
  const size_t ws = odit_linear_workspace_bytes();
  HIP_OK(d_x.alloc(x.size())); HIP_OK(d_w.alloc(w.size())); HIP_OK(d_r.alloc(res.size())); HIP_OK(d_o.alloc(out.size()));
  HIP_OK(d_g.alloc(gate.size())); HIP_OK(d_b.alloc(gbias.size())); HIP_OK(d_ws.alloc(ws));
  HIP_OK(hipMemset(d_ws.p, 0, ws));  // the contract: zero-filled once before the first use
  HIP_OK(hipMemcpy(d_x.p, x.data(), x.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_w.p, w.data(), w.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_r.p, res.data(), res.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_g.p, gate.data(), gate.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_b.p, gbias.data(), gbias.size() * 4, hipMemcpyHostToDevice));
  int handwritten = 0, launches = 0;
  ODIT_OK_OR_FAIL(odit_linear_rows_plan(d_x.p, d_w.p, d_b.p, d_o.p, d_r.p, d_g.p, M, N, K, K, K, N, N,
                                        ODIT_EPI_GATED_RESIDUAL_PRE, ODIT_F32, ODIT_BF16, S, N, ODIT_LINEAR_HANDWRITTEN,
                                        d_ws.p, ws, &handwritten, &launches));
  if (handwritten != 1 || launches != 1) {
    std::fprintf(stderr, "linear_rows plan: handwritten %d launches %d, want 1 and 1\n", handwritten, launches);
    return 1;
  }
  for (int rep = 0; rep < 2; ++rep)  // twice: the second call finds the counters as the first left them
    ODIT_OK_OR_FAIL(odit_linear_rows(d_x.p, d_w.p, d_b.p, d_o.p, d_r.p, d_g.p, M, N, K, K, K, N, N,
                                     ODIT_EPI_GATED_RESIDUAL_PRE, ODIT_F32, ODIT_BF16, S, N, ODIT_LINEAR_HANDWRITTEN,
                                     d_ws.p, ws, st));
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipMemcpy(out.data(), d_o.p, out.size() * 2, hipMemcpyDeviceToHost));
  double worst = 0.0;
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += static_cast<double>(from_bf16(x[m * K + k])) * from_bf16(w[n * K + k]);
      const int b = m / S;
      const double want = from_bf16(res[m * N + n]) + gate[b * N + n] * acc + gbias[b * N + n];
      const double err = std::fabs(from_bf16(out[m * N + n]) - want);
      worst = err > worst ? err : worst;
      if (err > 0.02 + 0.01 * std::fabs(want)) {
        std::fprintf(stderr, "linear_rows (%d,%d): got %.6g, want %.6g\n", m, n, from_bf16(out[m * N + n]), want);
        return 1;
      }
    }
  std::printf("odit_linear_rows: ok (hand-written kernel, one launch, max abs error %.4g)\n", worst);
  return 0;
}

int main() {
  if (odit_version() != ODIT_VERSION) {
    std::fprintf(stderr, "library version %d, header %d\n", odit_version(), ODIT_VERSION);
    return 1;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  int rc = check_rel_l1(st);
  if (rc == 0) rc = check_gated_residual(st);
  if (rc == 0) rc = check_adaln(st);
  if (rc == 0) rc = check_qknorm_rope(st);
  if (rc == 0) rc = check_attention(st);
  if (rc == 0) rc = check_linear_rows(st);
  (void)hipStreamDestroy(st);
  return rc;
}
