"""Dense projections with fused epilogues (odit_linear) against a float64 CPU product followed by the
oracle's elementwise ops: bias, GELU(tanh) (checked in fp32, where the tanh form and the erf form are
distinguishable), gated residual with per-batch-row gates, strided operands, and the tuning call."""

import pytest
import torch

from oracle import ops

pytestmark = pytest.mark.gpu


def _mk(M, N, K, dtype, seed=0, lead=()):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(*lead, M, K, generator=g) * 0.5).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    b = (torch.randn(N, generator=g) * 0.1).to(dtype)
    return x, w, b


def _ref(x, w, b):
    y = x.double() @ w.double().t()
    return y + b.double() if b is not None else y


def _tol(dtype):
    return {torch.bfloat16: 2e-2, torch.float16: 3e-3, torch.float32: 2e-4}[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(512, 768, 1024), (77, 200, 136), (1, 64, 64)])
def test_linear_bias_and_plain(gpu, dtype, M, N, K):
    from vllm_omni_amd import kernels

    x, w, b = _mk(M, N, K, dtype)
    print(f"linear {dtype} {M}x{N}x{K}", flush=True)
    got = kernels.linear(x.to(gpu), w.to(gpu), b.to(gpu))
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, b), atol=_tol(dtype), rtol=_tol(dtype))
    got = kernels.linear(x.to(gpu), w.to(gpu), None)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, None), atol=_tol(dtype), rtol=_tol(dtype))


def test_linear_gelu_epilogue_is_the_tanh_form(gpu):
    from vllm_omni_amd import kernels

    x, w, b = _mk(256, 512, 256, torch.float32, seed=1)
    x = x * 4  # spread pre-activations over [-4, 4], where tanh and erf forms differ by up to 5e-4
    pre = _ref(x, w, b)
    want_tanh = ops.gelu_tanh(pre)
    want_erf = torch.nn.functional.gelu(pre)
    got = kernels.linear(x.to(gpu), w.to(gpu), b.to(gpu), activation="gelu_tanh").double().cpu()
    err_tanh = (got - want_tanh).abs().max().item()
    err_erf = (got - want_erf).abs().max().item()
    print(f"GELU epilogue: max err vs tanh form {err_tanh:.2e}, vs erf form {err_erf:.2e}", flush=True)
    assert err_tanh < 5e-5 < err_erf
    # 16-bit, with and without bias
    for dtype in (torch.bfloat16, torch.float16):
        x, w, b = _mk(300, 384, 256, dtype, seed=2)
        for bias in (b, None):
            got = kernels.linear(x.to(gpu), w.to(gpu), None if bias is None else bias.to(gpu), activation="gelu_tanh")
            torch.testing.assert_close(got.double().cpu(), ops.gelu_tanh(_ref(x, w, bias)), atol=_tol(dtype),
                                       rtol=_tol(dtype))


@pytest.mark.parametrize("dtype,gate_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                              (torch.float16, torch.float16), (torch.float32, torch.float32)])
def test_linear_gated_residual(gpu, dtype, gate_dtype):
    from vllm_omni_amd import kernels

    B, S, N, K = 2, 130, 256, 384
    x, w, b = _mk(S, N, K, dtype, seed=3, lead=(B,))
    g = torch.Generator().manual_seed(4)
    h = torch.randn(B, S, N, generator=g).to(dtype)
    gate = torch.randn(B, N, generator=g).to(gate_dtype)
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, b)
    xg, wg, bg, hg, gg = (t.to(gpu) for t in (x, w, b, h, gate))
    got = kernels.linear(xg, wg, bg, residual=hg, gate=gg)
    torch.testing.assert_close(got.double().cpu(), want, atol=2 * _tol(dtype), rtol=_tol(dtype))
    assert torch.equal(hg.cpu(), h), "the residual operand is not written unless it is also the output"
    # [B,1,N] gate, in place on the residual
    h2 = hg.clone()
    got2 = kernels.linear(xg, wg, bg, residual=h2, gate=gg[:, None, :], out=h2)
    assert got2.data_ptr() == h2.data_ptr() and torch.equal(got2, got)
    # no gate = plain residual add; no bias
    got3 = kernels.linear(xg, wg, None, residual=hg)
    torch.testing.assert_close(got3.double().cpu(), h.double() + _ref(x, w, None), atol=2 * _tol(dtype), rtol=_tol(dtype))
    # gate chunk of a wider modulation tensor (row stride 6N), as the blocks pass it
    mod = torch.randn(B, 6 * N, generator=g).to(gate_dtype).to(gpu)
    got4 = kernels.linear(xg, wg, bg, residual=hg, gate=mod[:, 2 * N:3 * N])
    want4 = h.double() + mod[:, 2 * N:3 * N].double().cpu()[:, None, :] * _ref(x, w, b)
    torch.testing.assert_close(got4.double().cpu(), want4, atol=2 * _tol(dtype), rtol=_tol(dtype))


def test_linear_prescaled_gate_rows_and_autotune(gpu):
    """Caller-made float32 gate and gate*bias rows (no helper launch) give the same result as the form
    that derives them per call; autotuning on first use does not disturb in-place accumulation."""
    from vllm_omni_amd import kernels

    B, S, N, K = 2, 96, 256, 512
    x, w, b = _mk(S, N, K, torch.bfloat16, seed=9, lead=(B,))
    g = torch.Generator().manual_seed(10)
    h = torch.randn(B, S, N, generator=g).bfloat16()
    gate = torch.randn(B, N, generator=g).bfloat16()
    xg, wg, bg, hg, gg = (t.to(gpu) for t in (x, w, b, h, gate))
    per_call = kernels.linear(xg, wg, bg, residual=hg, gate=gg)
    g32 = gg.float()
    pre = kernels.linear(xg, wg, None, residual=hg, gate=g32, gate_bias=g32 * bg.float(), prescaled=True)
    assert torch.equal(pre, per_call)
    nobias = kernels.linear(xg, wg, None, residual=hg, gate=g32, prescaled=True)
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, None)
    torch.testing.assert_close(nobias.double().cpu(), want, atol=4e-2, rtol=2e-2)
    kernels.set_linear_autotune(3)
    try:
        h2 = hg.clone()
        tuned = kernels.linear(xg, wg, None, residual=h2, gate=g32, gate_bias=g32 * bg.float(), prescaled=True, out=h2)
    finally:
        kernels.set_linear_autotune(0)
    torch.testing.assert_close(tuned.float(), per_call.float(), atol=4e-2, rtol=2e-2)
    # the tuning record is keyed by the whole problem: all B * S rows, S rows per gate vector
    assert any(k[1:4] == (B * S, N, K) and k[-1] == S for k in kernels.linear_tuning_report())
    with pytest.raises(TypeError):
        kernels.linear(xg, wg, None, residual=hg, gate=gg, prescaled=True)


def test_linear_strided_operands_and_split_projection(gpu):
    """proj(cat([a, m])) as two calls on the two column ranges of one weight, the second accumulating
    through the residual form; x given as a 2-D view with a row stride."""
    from vllm_omni_amd import kernels

    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(6)
    M, Ca, Cm, N = 200, 128, 512, 128
    a = torch.randn(M, Ca, generator=g).to(dtype)
    m = torch.randn(M, Cm, generator=g).to(dtype)
    W = (torch.randn(N, Ca + Cm, generator=g) * 0.05).to(dtype)
    b = (torch.randn(N, generator=g) * 0.1).to(dtype)
    want = _ref(torch.cat([a, m], dim=1), W, b)
    Wg = W.to(gpu)
    wide = torch.cat([a, m], dim=1).to(gpu)           # rows of 640, the two inputs are column ranges of it
    y = kernels.linear(wide[:, Ca:], Wg[:, Ca:], b.to(gpu))
    y = kernels.linear(wide[:, :Ca], Wg[:, :Ca], None, residual=y, out=y)
    torch.testing.assert_close(y.double().cpu(), want, atol=4e-2, rtol=2e-2)


def test_linear_tune_keeps_results_and_reports_a_time(gpu):
    from vllm_omni_amd import kernels

    x, w, b = _mk(1024, 1024, 512, torch.bfloat16, seed=7)
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    before = kernels.linear(xg, wg, bg, activation="gelu_tanh")
    us = kernels.linear(xg, wg, bg, activation="gelu_tanh", tune_iters=5)
    print(f"tuned 1024x1024x512 GELU GEMM: {us:.1f} us", flush=True)
    assert 0 < us < 1e4
    after = kernels.linear(xg, wg, bg, activation="gelu_tanh")
    torch.testing.assert_close(after.float(), before.float(), atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(after.double().cpu(), ops.gelu_tanh(_ref(x, w, b)), atol=2e-2, rtol=2e-2)


def test_linear_argument_errors(gpu):
    from vllm_omni_amd import kernels

    x, w, b = _mk(8, 16, 32, torch.bfloat16)
    with pytest.raises(ValueError):
        kernels.linear(x.to(gpu), w.to(gpu)[:, :16], b.to(gpu))
    with pytest.raises(ValueError):
        kernels.linear(x.to(gpu), w.to(gpu), b.to(gpu), gate=torch.ones(16, device=gpu, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        kernels.linear(x, w, b)  # CPU tensors: no fallback


# ---------------------------------------------------------------------------- hand-written stream-K kernel
@pytest.fixture
def handwritten(gpu):
    from vllm_omni_amd import kernels

    kernels.set_linear_engine("handwritten")
    yield kernels
    kernels.set_linear_engine("auto")


def _counters_are_zero(kernels):
    return all(int(ws[:32768].view(torch.int32).abs().max().item()) == 0 for ws in kernels._LINEAR_SCRATCH.values())


@pytest.mark.parametrize("M,N,K", [
    (512, 768, 1024),    # 4 row tiles x 4 feature tiles
    (200, 392, 448),     # ragged row and feature tiles (N a multiple of 8 only)
    (64, 192, 64),       # one tile, one step
    (1024, 200, 4096),   # 8 row tiles, 2 feature tiles, every tile shared by 16 workgroups
    (512, 3072, 3072),   # text-stream output projection of the headline workload
    (512, 3072, 12288),  # text-stream MLP down-projection of the headline workload: where the kernel runs in the step
])
def test_streamk_gemm_matches_fp64_product(handwritten, gpu, M, N, K):
    x, w, b = _mk(M, N, K, torch.bfloat16, seed=M + N)
    print(f"stream-K {M}x{N}x{K}", flush=True)
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    got = handwritten.linear(xg, wg, bg)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, b), atol=2e-2, rtol=2e-2)
    again = handwritten.linear(xg, wg, bg)
    assert torch.equal(got, again), "the order of the partial sums must not depend on arrival order"
    assert _counters_are_zero(handwritten)
    got = handwritten.linear(xg, wg, None, activation="gelu_tanh")
    torch.testing.assert_close(got.double().cpu(), ops.gelu_tanh(_ref(x, w, None)), atol=2e-2, rtol=2e-2)
    # agreement with the library kernel on the same operands (both accumulate in fp32)
    handwritten.set_linear_engine("library")
    lib = handwritten.linear(xg, wg, bg)
    handwritten.set_linear_engine("handwritten")
    torch.testing.assert_close(handwritten.linear(xg, wg, bg).float(), lib.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("gate_dtype", [torch.bfloat16, torch.float32])
def test_streamk_gemm_gates_per_batch_row_in_one_launch(handwritten, gpu, gate_dtype):
    B, S, N, K = 2, 256, 384, 1536
    x, w, b = _mk(S, N, K, torch.bfloat16, seed=21, lead=(B,))
    g = torch.Generator().manual_seed(22)
    h = torch.randn(B, S, N, generator=g).bfloat16()
    mod = torch.randn(B, 6 * N, generator=g).to(gate_dtype)   # the gate is a column range of a wider tensor
    gate = mod[:, 2 * N:3 * N]
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, b)
    xg, wg, bg, hg, mg = (t.to(gpu) for t in (x, w, b, h, mod))
    got = handwritten.linear(xg, wg, bg, residual=hg, gate=mg[:, 2 * N:3 * N])
    torch.testing.assert_close(got.double().cpu(), want, atol=4e-2, rtol=2e-2)
    assert torch.equal(hg.cpu(), h)
    h2 = hg.clone()
    inplace = handwritten.linear(xg, wg, bg, residual=h2, gate=mg[:, 2 * N:3 * N], out=h2)
    assert inplace.data_ptr() == h2.data_ptr() and torch.equal(inplace, got)
    if gate_dtype == torch.float32:
        g32 = mg[:, 2 * N:3 * N]
        gb = torch.zeros_like(mg)                      # gate * bias rows with the gate's row stride
        gb[:, 2 * N:3 * N] = g32 * bg.float()
        pre = handwritten.linear(xg, wg, None, residual=hg, gate=g32, gate_bias=gb[:, 2 * N:3 * N], prescaled=True)
        torch.testing.assert_close(pre.double().cpu(), want, atol=4e-2, rtol=2e-2)
    assert _counters_are_zero(handwritten)


def test_streamk_gemm_refuses_what_it_does_not_take(handwritten, gpu):
    from vllm_omni_amd._lib import OmniDitKernelError

    x, w, b = _mk(77, 200, 136, torch.bfloat16)      # K not a multiple of 64
    with pytest.raises(OmniDitKernelError):
        handwritten.linear(x.to(gpu), w.to(gpu), b.to(gpu))
    x, w, b = _mk(4096, 250, 256, torch.bfloat16)    # N not a multiple of 8: neither hand-written kernel
    with pytest.raises(OmniDitKernelError):
        handwritten.linear(x.to(gpu), w.to(gpu), b.to(gpu))
    handwritten.set_linear_engine("auto")
    got = handwritten.linear(x.to(gpu), w.to(gpu), b.to(gpu))
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, b), atol=2e-2, rtol=2e-2)


def test_streamk_gemm_headline_problem_with_row_group_gates(handwritten, gpu):
    """The launch the Qwen step makes once per block: M = 2 x 256 text rows, N = 3072, K = 12288, float32
    gate and gate * bias rows per batch entry, accumulated onto the residual in place."""
    B, S, N, K = 2, 256, 3072, 12288
    x, w, b = _mk(S, N, K, torch.bfloat16, seed=41, lead=(B,))
    g = torch.Generator().manual_seed(42)
    h = torch.randn(B, S, N, generator=g).bfloat16()
    gate = torch.randn(B, N, generator=g)
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, b)
    xg, wg, hg, gg = (t.to(gpu) for t in (x, w, h, gate))
    gb = gg * b.to(gpu).float()
    assert handwritten.linear(xg, wg, None, residual=hg, gate=gg, gate_bias=gb, prescaled=True, plan_only=True) == (True, 1)
    got = handwritten.linear(xg, wg, None, residual=hg, gate=gg, gate_bias=gb, prescaled=True)
    torch.testing.assert_close(got.double().cpu(), want, atol=4e-2, rtol=2e-2)
    assert _counters_are_zero(handwritten)


def test_streamk_gemm_overrides_stale_ticket_words(handwritten, gpu):
    """Ticket words that an earlier launch left behind (as one that never finished would) carry an older launch
    number: the next launch raises them to its own and still reduces every tile."""
    x, w, b = _mk(1024, 200, 4096, torch.bfloat16, seed=43)   # every tile shared by 16 workgroups
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    want = handwritten.linear(xg, wg, bg)
    torch.cuda.synchronize()
    ws = handwritten._LINEAR_SCRATCH[(gpu.index or 0, torch.cuda.current_stream().cuda_stream)]
    words = ws[:16 * 8].view(torch.int64)   # the ticket words of this problem's 8 x 2 output tiles
    words.copy_(torch.randint(1, 14, words.shape, device=gpu))   # launch number 0, 1..13 tickets drawn
    got = handwritten.linear(xg, wg, bg)
    assert torch.equal(got, want)
    assert _counters_are_zero(handwritten)


@pytest.mark.parametrize("B,S", [(3, 96), (2, 160)])
@pytest.mark.parametrize("engine", ["handwritten", "library"])
def test_gated_rows_that_straddle_tiles_and_a_ragged_group(gpu, B, S, engine):
    """Groups of rows whose ends fall inside a 128-row tile, and B * S not a multiple of the tile: the
    hand-written kernel picks the gate row per output row, the library runs one launch per group."""
    from vllm_omni_amd import kernels

    N, K = 192, 256
    x, w, b = _mk(S, N, K, torch.bfloat16, seed=51 + B, lead=(B,))
    g = torch.Generator().manual_seed(52)
    h = torch.randn(B, S, N, generator=g).bfloat16()
    gate = torch.randn(B, N, generator=g).bfloat16()
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, b)
    got = kernels.linear(x.to(gpu), w.to(gpu), b.to(gpu), residual=h.to(gpu), gate=gate.to(gpu), engine=engine)
    torch.testing.assert_close(got.double().cpu(), want, atol=4e-2, rtol=2e-2)


# ---------------------------------------------------------------------------- hand-written tile kernel (many rows)
@pytest.mark.parametrize("M,N,K", [
    (2048, 512, 256),     # 8 x 2 tiles of 256 x 256, four steps
    (1280, 384, 64),      # 192-wide tiles, one step
    (1100, 200, 192),     # ragged last row tile and last feature tile (N a multiple of 8 only), three steps
    (4096, 768, 3072),    # 16 x 4 tiles of 256 x 192, the headline reduction length
])
def test_tile_gemm_matches_fp64_product(handwritten, gpu, M, N, K):
    x, w, b = _mk(M, N, K, torch.bfloat16, seed=M + N + 1)
    print(f"tile kernel {M}x{N}x{K}", flush=True)
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    assert handwritten.linear(xg, wg, bg, plan_only=True) == (True, 1)
    got = handwritten.linear(xg, wg, bg)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, b), atol=2e-2, rtol=2e-2)
    assert torch.equal(got, handwritten.linear(xg, wg, bg))
    got = handwritten.linear(xg, wg, None)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, None), atol=2e-2, rtol=2e-2)
    got = handwritten.linear(xg, wg, bg, activation="gelu_tanh")
    torch.testing.assert_close(got.double().cpu(), ops.gelu_tanh(_ref(x, w, b)), atol=2e-2, rtol=2e-2)
    lib = handwritten.linear(xg, wg, bg, engine="library")
    torch.testing.assert_close(handwritten.linear(xg, wg, bg).float(), lib.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("gate_dtype", [torch.bfloat16, torch.float32])
def test_tile_gemm_gates_per_batch_row_in_one_launch(handwritten, gpu, gate_dtype):
    B, S, N, K = 2, 1152, 384, 512     # groups of 1152 rows: the second starts inside row tile 4
    x, w, b = _mk(S, N, K, torch.bfloat16, seed=61, lead=(B,))
    g = torch.Generator().manual_seed(62)
    h = torch.randn(B, S, N, generator=g).bfloat16()
    mod = torch.randn(B, 6 * N, generator=g).to(gate_dtype)
    gate = mod[:, 2 * N:3 * N]
    want = h.double() + gate.double()[:, None, :] * _ref(x, w, b)
    xg, wg, bg, hg, mg = (t.to(gpu) for t in (x, w, b, h, mod))
    assert handwritten.linear(xg, wg, bg, residual=hg, gate=mg[:, 2 * N:3 * N], plan_only=True) == (True, 1)
    got = handwritten.linear(xg, wg, bg, residual=hg, gate=mg[:, 2 * N:3 * N])
    torch.testing.assert_close(got.double().cpu(), want, atol=4e-2, rtol=2e-2)
    assert torch.equal(hg.cpu(), h)
    h2 = hg.clone()
    inplace = handwritten.linear(xg, wg, bg, residual=h2, gate=mg[:, 2 * N:3 * N], out=h2)
    assert inplace.data_ptr() == h2.data_ptr() and torch.equal(inplace, got)
    if gate_dtype == torch.float32:
        g32 = mg[:, 2 * N:3 * N]
        gb = torch.zeros_like(mg)
        gb[:, 2 * N:3 * N] = g32 * bg.float()
        pre = handwritten.linear(xg, wg, None, residual=hg, gate=g32, gate_bias=gb[:, 2 * N:3 * N], prescaled=True)
        torch.testing.assert_close(pre.double().cpu(), want, atol=4e-2, rtol=2e-2)


def test_tile_gemm_on_a_column_range_of_the_weight(handwritten, gpu):
    """W as a column range of a wider weight (row stride > K), x and out as column ranges too."""
    M, N, K = 1536, 256, 128
    g = torch.Generator().manual_seed(71)
    wide_w = (torch.randn(N, 3 * K, generator=g) * 0.05).bfloat16()
    wide_x = torch.randn(M, 2 * K, generator=g).bfloat16()
    x, w = wide_x[:, K:], wide_w[:, K:2 * K]
    xg, wg = wide_x.to(gpu)[:, K:], wide_w.to(gpu)[:, K:2 * K]
    got = handwritten.linear(xg, wg, None)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, None), atol=2e-2, rtol=2e-2)


def test_linear_tune_compares_both_engines(gpu):
    from vllm_omni_amd import kernels

    x, w, b = _mk(512, 768, 3072, torch.bfloat16, seed=31)
    xg, wg, bg = x.to(gpu), w.to(gpu), b.to(gpu)
    us = kernels.linear(xg, wg, bg, tune_iters=5)
    print(f"tuned 512x768x3072: best of both engines {us:.1f} us", flush=True)
    assert 0 < us < 1e4
    got = kernels.linear(xg, wg, bg)
    torch.testing.assert_close(got.double().cpu(), _ref(x, w, b), atol=2e-2, rtol=2e-2)
