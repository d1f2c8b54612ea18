"""Parity of every HIP kernel (called through the C ABI) against the CPU oracle on seeded inputs.

Tolerances: bf16/fp16 results are compared with the oracle evaluated in fp32 on the same (already
16-bit-rounded) inputs; the bound is a few units of the output format's rounding step. With
reference rounding switched on, elementwise results must match the oracle's 16-bit torch path
bit for bit up to a stated number of ulps where reduction order differs.
"""

import math

import pytest
import torch

from oracle import ops

pytestmark = pytest.mark.gpu


def _rand(*shape, seed=0, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _cos_sin(S, half, seed=0):
    g = torch.Generator().manual_seed(seed)
    ang = torch.rand(S, half, generator=g) * 6.0 - 3.0
    return torch.cos(ang), torch.sin(ang)


def _close(got, want, atol, rtol=0.0, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert bool((err <= bound).all()), f"{what}: max err {err.max().item():.3e} (bound {atol}+{rtol}*|x|)"


def _cosine(a, b):
    a, b = a.float().flatten().cpu(), b.float().flatten().cpu()
    return float(torch.dot(a, b) / (a.norm() * b.norm()))


# ========================================================================================= K3
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,C", [(2, 33, 3072), (1, 7, 256), (2, 5, 5120), (3, 4, 40), (1, 3, 1000), (2, 3, 37)])
def test_adaln_modulate(gpu, dtype, B, S, C):
    from vllm_omni_amd import kernels

    x = _rand(B, S, C, seed=1, dtype=dtype, scale=2.0) + 0.5
    mod = _rand(B, 3 * C, seed=2, dtype=dtype, scale=0.5)
    want, _ = ops.ada_layer_norm(x.float(), mod.float())
    shift, scale, _ = mod.to(gpu).chunk(3, dim=-1)
    got = kernels.adaln_modulate(x.to(gpu), shift, scale)
    tol = {torch.bfloat16: 2e-2, torch.float16: 3e-3, torch.float32: 2e-5}[dtype]
    _close(got, want, atol=tol, rtol=tol, what="adaln")
    if dtype != torch.float32:
        # reference rounding: LN -> dtype, (1+scale) -> dtype, product -> dtype, sum -> dtype
        want_rr, _ = ops.ada_layer_norm(x, mod)
        got_rr = kernels.adaln_modulate(x.to(gpu), shift, scale, ref_rounding=True)
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        # 16-bit roundings after a reduction whose order differs: the product may move by one of ITS
        # ulps, which after cancellation against the shift is several ulps of a smaller output
        _close(got_rr, want_rr, atol=8 * ulp, rtol=4.2 * ulp, what="adaln ref-rounding")
        frac_equal = (got_rr.cpu() == want_rr).float().mean().item()
        assert frac_equal > 0.97, f"only {frac_equal:.3f} of elements bit-identical"


@pytest.mark.parametrize("C", [3072, 5120, 1000])
def test_adaln_ill_conditioned_rows(gpu, C):
    """Rows where a one-pass variance is at risk, in float32 against a float64 LayerNorm: a mean 600 times the
    standard deviation, constant rows (variance exactly zero: the output is the shift), one outlier channel of
    1e4 among unit-scale values, and a row of values near 1e-3."""
    from vllm_omni_amd import kernels

    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 6, C, generator=g)
    x[0, 0] = 300.0 + 0.5 * x[0, 0]
    x[0, 1] = 7.25
    x[0, 2] = 0.0
    x[0, 3, C // 3] = 1.0e4
    x[0, 4] = 1.0e-3 * x[0, 4]
    shift, scale = 0.3 * torch.randn(1, C, generator=g), 0.3 * torch.randn(1, C, generator=g)
    want = torch.nn.functional.layer_norm(x.double(), (C,), eps=1e-6) * (1 + scale.double()[:, None]) + shift.double()[:, None]
    got = kernels.adaln_modulate(x.to(gpu), shift.to(gpu), scale.to(gpu)).cpu()
    assert torch.isfinite(got).all()
    assert torch.equal(got[0, 1], shift[0]) and torch.equal(got[0, 2], shift[0])
    for r, tol in ((0, 2e-4), (3, 1e-4), (4, 1e-4), (5, 1e-5)):
        err = (got[0, r].double() - want[0, r]).abs().max().item()
        assert err <= tol * max(1.0, want[0, r].abs().max().item()), (r, err)
    # the same rows in bf16 (the mean-300 row then carries 2^-8 * 300 of input rounding: checked against the
    # LayerNorm of the ROUNDED input)
    xb = x.bfloat16()
    wantb = torch.nn.functional.layer_norm(xb.double(), (C,), eps=1e-6) * (1 + scale.bfloat16().double()[:, None]) \
        + shift.bfloat16().double()[:, None]
    gotb = kernels.adaln_modulate(xb.to(gpu), shift.bfloat16().to(gpu), scale.bfloat16().to(gpu)).cpu()
    assert torch.isfinite(gotb.float()).all()
    rel = (gotb.double() - wantb).abs() / (wantb.abs() + 1.0)
    assert rel.max().item() <= 2 ** -7, rel.max().item()


def test_adaln_index_fp32_params_affine_and_strides(gpu):
    from vllm_omni_amd import kernels

    B, S, C = 2, 9, 512
    x = _rand(B, S, C, seed=3)
    mod = _rand(2 * B, 3 * C, seed=4, scale=0.3)
    index = (torch.arange(B * S).reshape(B, S) % 3 == 0).int()
    want, _ = ops.ada_layer_norm(x.float(), mod.float(), index)
    shift, scale, _ = mod.to(gpu).chunk(3, dim=-1)
    got = kernels.adaln_modulate(x.to(gpu), shift, scale, index=index.to(gpu))
    _close(got, want, atol=2e-2, rtol=2e-2, what="adaln index")
    # fp32 modulation on bf16 activations, LayerNorm affine (Wan's norm2 / fp32 modulation path)
    modf = _rand(B, 2 * C, seed=5, dtype=torch.float32, scale=0.3)
    lw, lb = _rand(C, seed=6, dtype=torch.float32) + 1, _rand(C, seed=7, dtype=torch.float32)
    ln = torch.nn.functional.layer_norm(x.float(), (C,), lw, lb, 1e-6)
    want2 = ln * (1 + modf[:, None, C:]) + modf[:, None, :C]
    mg = modf.to(gpu)
    got2 = kernels.adaln_modulate(x.to(gpu), mg[:, :C], mg[:, C:], ln_weight=lw.to(gpu), ln_bias=lb.to(gpu))
    _close(got2, want2, atol=2e-2, rtol=1e-2, what="adaln fp32 params + affine")
    # strided input rows (a slice of a wider buffer) and no modulation at all
    wide = _rand(B, S, 2 * C, seed=8)
    got3 = kernels.adaln_modulate(wide.to(gpu)[:, :, C:], None, None)
    _close(got3, torch.nn.functional.layer_norm(wide[:, :, C:].float(), (C,), eps=1e-6), atol=2e-2, what="plain LN")


@pytest.mark.parametrize("C", [256, 3072, 5120, 100])
def test_adaln_and_gate_with_per_token_rows_and_tables(gpu, C):
    """Per-token modulation rows (views of a [B,S,6,C] tensor, token stride 6C) plus float32 [C] tables
    added in-kernel, against the expression the reference evaluates: (table + temb.float()) chunks, fp32
    LayerNorm, modulate; (h.float() + y * gate). C = 100 takes the kernels' unvectorised paths."""
    from vllm_omni_amd import kernels

    B, S = 2, 11
    x, y = _rand(B, S, C, seed=1), _rand(B, S, C, seed=2)
    temb = _rand(B, S, 6, C, seed=3, scale=0.3)
    table = _rand(6, C, seed=4, dtype=torch.float32, scale=0.3)
    mods = (table[None, None] + temb.float()).unbind(2)
    ln = torch.nn.functional.layer_norm(x.float(), (C,), eps=1e-6)
    tg, tabg = temb.to(gpu), table.to(gpu)
    got = kernels.adaln_modulate(x.to(gpu), tg[:, :, 0], tg[:, :, 1], shift_bias=tabg[0], scale_bias=tabg[1])
    _close(got, ln * (1 + mods[1]) + mods[0], atol=2e-2, rtol=1e-2, what="per-token adaln + tables")
    # rows only / tables only (the table alone is then the modulation of every token)
    got = kernels.adaln_modulate(x.to(gpu), tg[:, :, 3], tg[:, :, 4])
    _close(got, ln * (1 + temb[:, :, 4].float()) + temb[:, :, 3].float(), atol=2e-2, rtol=1e-2, what="per-token adaln")
    got = kernels.adaln_modulate(x.to(gpu), None, None, shift_bias=tabg[0], scale_bias=tabg[1])
    _close(got, ln * (1 + table[1]) + table[0], atol=2e-2, rtol=1e-2, what="tables only")
    got = kernels.gated_residual(x.to(gpu), y.to(gpu), tg[:, :, 2], gate_bias=tabg[2])
    _close(got, x.float() + y.float() * mods[2], atol=1e-6, rtol=2 ** -8, what="per-token gate + table")
    got = kernels.gated_residual(x.to(gpu), y.to(gpu), None, gate_bias=tabg[5])
    _close(got, x.float() + y.float() * table[5], atol=1e-6, rtol=2 ** -8, what="table as the gate")
    with pytest.raises(ValueError, match="exclude"):
        kernels.adaln_modulate(x.to(gpu), tg[:, :, 0], tg[:, :, 1], index=torch.zeros(B, S, dtype=torch.int32, device=gpu))


# ========================================================================================= K4
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gated_residual(gpu, dtype):
    from vllm_omni_amd import kernels

    B, S, C = 2, 17, 3072
    h, y = _rand(B, S, C, seed=1, dtype=dtype), _rand(B, S, C, seed=2, dtype=dtype)
    mod = _rand(B, 3 * C, seed=3, dtype=dtype)
    gate = mod.chunk(3, dim=-1)[2]
    want = ops.gated_residual(h.float(), y.float(), gate.float()[:, None])
    got = kernels.gated_residual(h.to(gpu), y.to(gpu), mod.to(gpu).chunk(3, dim=-1)[2].unsqueeze(1))
    tol = {torch.bfloat16: 2 ** -8, torch.float16: 2 ** -11, torch.float32: 1e-6}[dtype]
    _close(got, want, atol=1e-6, rtol=tol, what="gated residual")
    if dtype != torch.float32:
        want_rr = ops.gated_residual(h, y, gate[:, None])
        got_rr = kernels.gated_residual(h.to(gpu), y.to(gpu), gate.to(gpu), ref_rounding=True)
        assert torch.equal(got_rr.cpu(), want_rr), "reference-rounding path must be bit-exact"
    # gate = 0 is the identity, gate = None a plain residual, in-place output, per-token fp32 gate
    z = torch.zeros(B, C, dtype=dtype, device=gpu)
    assert torch.equal(kernels.gated_residual(h.to(gpu), y.to(gpu), z).cpu(), h)
    _close(kernels.gated_residual(h.to(gpu), y.to(gpu), None), h.float() + y.float(), atol=1e-6, rtol=tol)
    hg = h.to(gpu).clone()
    gtok = _rand(B, S, C, seed=4, dtype=torch.float32)
    out = kernels.gated_residual(hg, y.to(gpu), gtok.to(gpu), out=hg)
    assert out.data_ptr() == hg.data_ptr()
    _close(hg, h.float() + gtok * y.float(), atol=1e-6, rtol=tol, what="per-token fp32 gate, in place")


def test_gated_residual_odd_sizes(gpu):
    from vllm_omni_amd import kernels

    h, y, g = _rand(2, 3, 37, seed=1), _rand(2, 3, 37, seed=2), _rand(2, 37, seed=3)
    _close(kernels.gated_residual(h.to(gpu), y.to(gpu), g.to(gpu)),
           h.float() + g.float()[:, None] * y.float(), atol=1e-6, rtol=2 ** -8)


# ========================================================================================= K5
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,n", [(2, 64 * 3072), (1, 4096 * 3072), (3, 1000), (2, 8 * 1024 * 8 + 5)])
def test_rel_l1(gpu, dtype, B, n):
    from vllm_omni_amd import kernels
    from vllm_omni_amd.cache.teacache.hook import rel_l1_from_sums

    prev = _rand(B, n, seed=1, dtype=dtype)
    cur = (prev.float() * 1.04 + 0.03 * _rand(B, n, seed=2, dtype=torch.float32)).to(dtype)
    sums = kernels.rel_l1_sums(cur.to(gpu), prev.to(gpu), ref_rounding=True).cpu()
    for b in range(B):
        sd = (cur[b] - prev[b]).abs().double().sum().item()   # difference rounded to dtype, as torch does
        sp = prev[b].abs().double().sum().item()
        assert sums[b, 0].item() == pytest.approx(sd, rel=5e-6)
        assert sums[b, 1].item() == pytest.approx(sp, rel=5e-6)
        # the scalar TeaCache thresholds is IDENTICAL to the reference expression's
        want = ops.rel_l1(cur[b:b + 1], prev[b:b + 1])
        got = rel_l1_from_sums(sums[b, 0].item(), sums[b, 1].item(), n, dtype)
        if dtype == torch.bfloat16:
            assert got == want
        else:
            assert got == pytest.approx(want, rel=1e-5)
    # deterministic: a second launch gives bit-identical sums
    again = kernels.rel_l1_sums(cur.to(gpu), prev.to(gpu), ref_rounding=True).cpu()
    assert torch.equal(again, sums)


def test_rel_l1_one_workspace_serves_changing_shapes(gpu):
    """The reduction is one launch whose last workgroup per row adds the row's partials and hands the row's ticket
    counter back at zero: calls of different (B, n) through one cached workspace, back to back on one stream,
    each equal to the same call on a fresh workspace."""
    from vllm_omni_amd import kernels

    shapes = [(2, 4096 * 3072), (1, 1000), (3, 64 * 3072 + 3), (2, 4096 * 3072), (4, 17), (2, 300000)]
    data = {}
    for B, n in set(shapes):
        prev = _rand(B, n, seed=B + n % 97)
        cur = (prev.float() * 1.1 + 0.01).bfloat16()
        data[(B, n)] = (cur.to(gpu), prev.to(gpu))
    kernels._REL_L1_SCRATCH.clear()
    kernels.rel_l1_sums(*data[(4, 4096 * 3072)] if (4, 4096 * 3072) in data else data[(2, 4096 * 3072)])  # sizes the workspace
    shared = [kernels.rel_l1_sums(*data[s_]) for s_ in shapes for _ in range(3)]
    torch.cuda.synchronize()
    fresh = []
    for s_ in shapes:
        kernels._REL_L1_SCRATCH.clear()
        fresh.append(kernels.rel_l1_sums(*data[s_]))
    for i, s_ in enumerate(shapes):
        for r in range(3):
            assert torch.equal(shared[3 * i + r], fresh[i]), f"shape {s_}, repetition {r}"
        cur, prev = data[s_]
        want = (cur.float() - prev.float()).bfloat16().float().abs().double().sum(dim=1)
        assert torch.allclose(fresh[i][:, 0], want, rtol=5e-6)


def test_rel_l1_workspace_rows_grow_and_stale_ticket_words(gpu):
    """One workspace through the C ABI: a call with few rows and many workgroups per row (its partials fill the
    bytes behind the ticket words), then a call with many rows (whose ticket words must not be those bytes), then
    ticket words left as by a launch that never finished (an older launch number, some tickets drawn): each call
    equals the same call on a fresh zeroed workspace."""
    from vllm_omni_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    few = (2, 4096 * 3072)
    many = (100, 3000)
    need = max(int(lib.odit_rel_l1_workspace_bytes(*few)), int(lib.odit_rel_l1_workspace_bytes(*many)))
    ws = torch.zeros(need, dtype=torch.uint8, device=gpu)

    def run(cur, prev, workspace):
        B, n = cur.shape
        sums = torch.full((B, 2), -1.0, dtype=torch.float64, device=gpu)
        rc = lib.odit_rel_l1(cur.data_ptr(), prev.data_ptr(), sums.data_ptr(), workspace.data_ptr(), workspace.numel(),
                             B, n, n, n, 0, 1, st)
        assert rc == 0, lib.odit_last_error()
        return sums

    data = {}
    for B, n in (few, many):
        prev = _rand(B, n, seed=B)
        data[(B, n)] = ((prev.float() * 1.1 + 0.01).bfloat16().to(gpu), prev.to(gpu))
    fresh = {k: run(*v, torch.zeros(need, dtype=torch.uint8, device=gpu)) for k, v in data.items()}
    got_few = run(*data[few], ws)
    got_many = run(*data[many], ws)
    torch.cuda.synchronize()
    assert torch.equal(got_few, fresh[few]) and torch.equal(got_many, fresh[many])
    # stale words: launch number 0 with 1..99 tickets drawn in every row's word
    words = ws[:8 * 100].view(torch.int64)   # the words of the rows these calls use
    words.copy_(torch.randint(1, 100, words.shape, device=gpu))
    # ... and in the group words of the two long rows (8 per row, 1 KiB apart, behind the 65536 row words)
    groups = ws[65536 * 8:65536 * 8 + 2 * 8 * 1024].view(torch.int64).view(16, 128)[:, 0]
    groups.copy_(torch.randint(1, 16, groups.shape, device=gpu))
    assert torch.equal(run(*data[many], ws), fresh[many])
    assert torch.equal(run(*data[few], ws), fresh[few])
    torch.cuda.synchronize()
    assert int(ws[:8 * 100].view(torch.int64).abs().max().item()) == 0   # handed back at zero
    assert int(groups.abs().max().item()) == 0


def test_rel_l1_closed_forms(gpu):
    from vllm_omni_amd import kernels

    prev = (_rand(2, 5000, seed=3, dtype=torch.float32).abs() + 0.5)
    s = kernels.rel_l1_sums(prev.to(gpu), prev.to(gpu)).cpu()
    assert torch.all(s[:, 0] == 0)
    s = kernels.rel_l1_sums((1.5 * prev).to(gpu), prev.to(gpu), ref_rounding=False).cpu()
    assert torch.allclose(s[:, 0] / s[:, 1], torch.full((2,), 0.5, dtype=torch.float64), rtol=1e-6)


# ========================================================================================= K2
@pytest.mark.parametrize("C", [3072, 2048, 1536, 1160])
def test_adaln_many_rows_two_per_wavefront(gpu, C):
    """From 6144 rows on the per-block form puts two rows on a wavefront: an odd row count (the last wavefront
    has one row), 3, 4, 5 and 6 vectors per lane, alone and as a pair whose second problem starts in the middle of
    the first wavefronts' second rows; against the oracle and, bit for bit, against calls of few rows each."""
    from vllm_omni_amd import kernels

    B, S = 1, 6145
    x = _rand(B, S, C, seed=11, dtype=torch.bfloat16, scale=1.5).to(gpu)
    mod = (_rand(B, 3 * C, seed=12, dtype=torch.bfloat16) * 0.3).to(gpu)
    got = kernels.adaln_modulate(x, mod[:, :C], mod[:, C:2 * C], eps=1e-6)
    want = ops.ada_layer_norm(x.float().cpu(), mod.float().cpu(), eps=1e-6)[0]
    _close(got, want, atol=2e-2, rtol=2e-2, what="adaln, two rows per wavefront")
    few = torch.cat([kernels.adaln_modulate(x[:, i:i + 1000], mod[:, :C], mod[:, C:2 * C], eps=1e-6)
                     for i in range(0, S, 1000)], dim=1)
    assert torch.equal(got, few), "a row's result depends on how many rows the call has"
    x2 = _rand(B, 77, C, seed=13, dtype=torch.bfloat16).to(gpu)
    mod2 = (_rand(B, 3 * C, seed=14, dtype=torch.bfloat16) * 0.3).to(gpu)
    a, b = kernels.adaln_modulate_pair((x, mod[:, :C], mod[:, C:2 * C]), (x2, mod2[:, :C], mod2[:, C:2 * C]), eps=1e-6)
    assert torch.equal(a, got)
    assert torch.equal(b, kernels.adaln_modulate(x2, mod2[:, :C], mod2[:, C:2 * C], eps=1e-6))


# ---- two problems in one launch (the image and the text stream of a dual-stream block) ----------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("C,S0,S1", [(3072, 70, 9), (256, 5, 33), (37, 4, 6)])
@pytest.mark.parametrize("ref_rounding", [False, True])
def test_adaln_modulate_pair_equals_two_calls(gpu, dtype, C, S0, S1, ref_rounding):
    """odit_adaln_modulate_pair against odit_adaln_modulate, bit for bit (C = 37 takes the any-width kernel),
    with strided inputs and modulation rows that are views of one [B, 6C] tensor, and against the oracle."""
    from vllm_omni_amd import kernels

    B = 2
    xs = [_rand(B, S, 2 * C, seed=3 + i, dtype=dtype, scale=2.0).to(gpu)[:, :, C:] if C % 8 == 0
          else _rand(B, S, C, seed=3 + i, dtype=dtype, scale=2.0).to(gpu) for i, S in enumerate((S0, S1))]
    mods = [(_rand(B, 6 * C, seed=7 + i, dtype=dtype) * 0.3).to(gpu) for i in range(2)]
    probs = [(x, m[:, :C], m[:, C:2 * C]) for x, m in zip(xs, mods)]
    got = kernels.adaln_modulate_pair(probs[0], probs[1], eps=1e-6, ref_rounding=ref_rounding)
    for (x, shift, scale), m, g in zip(probs, mods, got):
        one = kernels.adaln_modulate(x, shift, scale, eps=1e-6, ref_rounding=ref_rounding)
        assert torch.equal(g, one), "pair launch differs from the single call"
        want = ops.ada_layer_norm(x.float().cpu(), m[:, :3 * C].float().cpu(), eps=1e-6)[0]
        tol = {torch.bfloat16: 2e-2, torch.float16: 3e-3, torch.float32: 2e-5}[dtype]
        _close(g, want, atol=tol, rtol=tol, what="adaln pair vs oracle")
    # an empty problem leaves the other one
    empty = (xs[1][:, :0], probs[1][1], probs[1][2])
    g0, g1 = kernels.adaln_modulate_pair(probs[0], empty, eps=1e-6, ref_rounding=ref_rounding)
    assert torch.equal(g0, got[0]) and g1.shape[1] == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("ref_rounding", [False, True])
def test_qknorm_rope_pair_equals_two_calls(gpu, dtype, with_v, ref_rounding):
    """odit_qknorm_rope_pair against two odit_qknorm_rope calls into the same joint buffers, bit for bit:
    different lengths, weights, tables and row offsets per problem; also with whole-row statistics (one launch
    per problem inside the call) and without rotary tables."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD, ODIT_NORM_NONE, ODIT_NORM_ROW

    B, H, D, S_txt, S_img = 2, 4, 64, 11, 150
    S = S_txt + S_img
    qkv = [_rand(B, n, 3, H, D, seed=30 + i, dtype=dtype).to(gpu) for i, n in enumerate((S_txt, S_img))]
    tabs = [tuple(t.to(gpu) for t in _cos_sin(n, D // 2, seed=40 + i)) for i, n in enumerate((S_txt, S_img))]
    for mode, wn in ((ODIT_NORM_HEAD, D), (ODIT_NORM_ROW, H * D), (ODIT_NORM_NONE, D)):
        ws = [((_rand(wn, seed=50 + i, dtype=torch.float32) * 0.2 + 1).to(dtype).to(gpu),
               (_rand(wn, seed=60 + i, dtype=torch.float32) * 0.2 + 1).to(dtype).to(gpu)) for i in range(2)]
        for rotary in (True, False):
            outs = []
            for paired in (False, True):
                jq = torch.zeros(B, S, H, D, dtype=dtype, device=gpu)
                jk = torch.zeros_like(jq)
                jv = torch.zeros_like(jq) if with_v else None
                probs = []
                for i, off in enumerate((0, S_txt)):
                    t = qkv[i]
                    cs = tabs[i] if rotary else (None, None)
                    probs.append((t[:, :, 0], t[:, :, 1], t[:, :, 2] if with_v else None, ws[i][0], ws[i][1],
                                  cs[0], cs[1], off))
                if paired:
                    kernels.qknorm_rope_pair(probs[0], probs[1], jq, jk, jv, eps=1e-6, norm_mode=mode,
                                             ref_rounding=ref_rounding)
                else:
                    for (q, k, v, wq, wk, c, s_, off) in probs:
                        kernels.qknorm_rope(q, k, v, jq, jk, jv, wq, wk, c, s_, eps=1e-6, out_seq_offset=off,
                                            norm_mode=mode, ref_rounding=ref_rounding)
                outs.append((jq, jk, jv))
            for a, b in zip(*outs):
                assert (a is None and b is None) or torch.equal(a, b), f"pair launch differs (mode {mode}, rotary {rotary})"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H,D", [(24, 128), (4, 64)])
def test_qknorm_rope_joint(gpu, dtype, H, D):
    """Fused QKV slices of an image and a text stream -> joint [txt;img] buffers."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD

    B, S_img, S_txt = 2, 50, 11
    wq = (_rand(D, seed=1, dtype=torch.float32) * 0.2 + 1).to(dtype)
    wk = (_rand(D, seed=2, dtype=torch.float32) * 0.2 + 1).to(dtype)
    streams = {}
    for name, S, seed in (("txt", S_txt, 10), ("img", S_img, 20)):
        qkv = _rand(B, S, 3, H, D, seed=seed, dtype=dtype)
        cos, sin = _cos_sin(S, D // 2, seed=seed + 1)
        streams[name] = (qkv, cos, sin)
    S = S_txt + S_img
    jq = torch.zeros(B, S, H, D, dtype=dtype, device=gpu)
    jk, jv = torch.zeros_like(jq), torch.zeros_like(jq)
    want_q, want_k, want_v, want_q_rr, want_k_rr = [], [], [], [], []
    off = 0
    for name in ("txt", "img"):
        qkv, cos, sin = streams[name]
        g = qkv.to(gpu)
        kernels.qknorm_rope(g[:, :, 0], g[:, :, 1], g[:, :, 2], jq, jk, jv, wq.to(gpu), wk.to(gpu),
                            cos.to(gpu), sin.to(gpu), eps=1e-6, out_seq_offset=off, norm_mode=ODIT_NORM_HEAD)
        off += qkv.shape[1]
        f = qkv.float()
        want_q.append(ops.apply_rotary(ops.rms_norm_head(f[:, :, 0], wq.float()), cos, sin))
        want_k.append(ops.apply_rotary(ops.rms_norm_head(f[:, :, 1], wk.float()), cos, sin))
        want_v.append(qkv[:, :, 2])
        want_q_rr.append(ops.apply_rotary(ops.rms_norm_head(qkv[:, :, 0], wq), cos.to(dtype), sin.to(dtype)))
        want_k_rr.append(ops.apply_rotary(ops.rms_norm_head(qkv[:, :, 1], wk), cos.to(dtype), sin.to(dtype)))
    tol = {torch.bfloat16: 2e-2, torch.float16: 3e-3, torch.float32: 2e-5}[dtype]
    _close(jq, torch.cat(want_q, 1), atol=tol, rtol=tol, what="joint q")
    _close(jk, torch.cat(want_k, 1), atol=tol, rtol=tol, what="joint k")
    assert torch.equal(jv.cpu(), torch.cat(want_v, 1)), "v must be copied bit for bit"
    if dtype != torch.float32:
        off = 0
        for name in ("txt", "img"):
            qkv, cos, sin = streams[name]
            g = qkv.to(gpu)
            kernels.qknorm_rope(g[:, :, 0], g[:, :, 1], g[:, :, 2], jq, jk, jv, wq.to(gpu), wk.to(gpu),
                                cos.to(gpu), sin.to(gpu), eps=1e-6, out_seq_offset=off,
                                norm_mode=ODIT_NORM_HEAD, ref_rounding=True)
            off += qkv.shape[1]
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        _close(jq, torch.cat(want_q_rr, 1), atol=2 * ulp, rtol=2.1 * ulp, what="joint q, ref rounding")
        _close(jk, torch.cat(want_k_rr, 1), atol=2 * ulp, rtol=2.1 * ulp, what="joint k, ref rounding")
        assert (jq.cpu() == torch.cat(want_q_rr, 1)).float().mean().item() > 0.95


def test_qknorm_rope_q_alone_and_offsets_beyond_31_bits(gpu):
    """q without k, and the same inputs as views whose batch stride exceeds 2^31 elements (the kernel's 64-bit
    indexing, which ordinary shapes never reach): identical bits to the compact call."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD

    B, S, H, D, off = 2, 37, 3, 128, 5
    dtype = torch.bfloat16
    qkv = _rand(B, S, 3, H, D, seed=31, dtype=dtype).to(gpu)
    w = (_rand(D, seed=32, dtype=torch.float32) * 0.2 + 1).to(dtype).to(gpu)
    cos, sin = (t.to(gpu) for t in _cos_sin(S, D // 2, seed=33))

    def run(q, k, v):
        outs = [torch.zeros(B, S + off, H, D, dtype=dtype, device=gpu) if t is not None else None for t in (q, k, v)]
        kernels.qknorm_rope(q, k, v, outs[0], outs[1], outs[2], w, w, cos, sin, eps=1e-6, out_seq_offset=off,
                            norm_mode=ODIT_NORM_HEAD)
        return outs

    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    full = run(q, k, v)
    want_q = ops.apply_rotary(ops.rms_norm_head(q.float().cpu(), w.float().cpu()), cos.cpu(), sin.cpu())
    _close(full[0][:, off:], want_q, atol=2e-2, rtol=2e-2, what="q of the q+k+v call")
    alone = run(q, None, None)
    assert torch.equal(alone[0], full[0])
    pair = run(q, k, None)
    assert torch.equal(pair[0], full[0]) and torch.equal(pair[1], full[1])
    # batch stride 2^31 + 4096 elements: one 4.3 GB buffer holding both batch rows far apart
    row = S * 3 * H * D
    stride_b = (1 << 31) + 4096
    big = torch.empty(stride_b + row, dtype=dtype, device=gpu)
    far = torch.as_strided(big, (B, S, 3, H, D), (stride_b, 3 * H * D, H * D, D, 1))
    far.copy_(qkv)
    got = run(far[:, :, 0], far[:, :, 1], far[:, :, 2])
    del big, far
    for a, b, name in zip(got, full, "qkv"):
        assert torch.equal(a, b), name


def test_rotary_layer_and_neox_and_partial(gpu):
    from vllm_omni_amd.layers.rope import RotaryEmbedding

    B, S, H, D = 2, 13, 3, 128
    x = _rand(B, S, H, D, seed=1)
    cos, sin = _cos_sin(S, D // 2, seed=2)
    for neox in (False, True):
        layer = RotaryEmbedding(is_neox_style=neox)
        got = layer(x.to(gpu), cos.to(gpu), sin.to(gpu))
        _close(got, ops.apply_rotary(x.float(), cos, sin, interleaved=not neox), atol=2e-2, rtol=1e-2,
               what=f"rotary neox={neox}")
    # [B,S,rot/2] tables use the first batch row; rot < D leaves the tail alone
    c3, s3 = cos[:, :32].expand(B, S, 32), sin[:, :32].expand(B, S, 32)
    got = RotaryEmbedding()(x.to(gpu), c3.to(gpu), s3.to(gpu))
    _close(got, ops.apply_rotary(x.float(), cos[:, :32], sin[:, :32]), atol=2e-2, rtol=1e-2, what="partial rotary")
    assert torch.equal(got[..., 64:].cpu(), x[..., 64:])
    # identity tables (text rows of the joint-attention config) return x bit for bit
    same = RotaryEmbedding()(x.to(gpu), torch.ones(S, 64, device=gpu), torch.zeros(S, 64, device=gpu))
    assert torch.equal(same.cpu(), x)


def test_rmsnorm_layer_row_mode_and_wan_qknorm(gpu):
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_ROW
    from vllm_omni_amd.layers.rmsnorm import RMSNorm

    # txt_norm: 3584-wide rows
    x = _rand(2, 19, 3584, seed=1)
    layer = RMSNorm(3584).to(gpu).to(torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_((_rand(3584, seed=2, dtype=torch.float32) * 0.1 + 1).to(gpu))
    _close(layer(x.to(gpu)), ops.rms_norm_head(x.float(), layer.weight.float().cpu()), atol=2e-2, rtol=1e-2,
           what="RMSNorm 3584")
    # Wan: whole-row RMS over H*D = 5120 with fp32 weights, then rotary with half tables
    B, S, H, D = 1, 21, 40, 128
    qkv = _rand(B, S, 3, H, D, seed=3)
    wq, wk = _rand(H * D, seed=4, dtype=torch.float32) * 0.1 + 1, _rand(H * D, seed=5, dtype=torch.float32) * 0.1 + 1
    cos, sin = _cos_sin(S, D // 2, seed=6)
    g = qkv.to(gpu)
    q_out = torch.empty(B, S, H, D, dtype=torch.bfloat16, device=gpu)
    k_out, v_out = torch.empty_like(q_out), torch.empty_like(q_out)
    kernels.qknorm_rope(g[:, :, 0], g[:, :, 1], g[:, :, 2], q_out, k_out, v_out, wq.to(gpu), wk.to(gpu),
                        cos.to(gpu), sin.to(gpu), eps=1e-6, norm_mode=ODIT_NORM_ROW)
    fc = cos.repeat_interleave(2, -1).view(1, S, 1, D)
    fs = sin.repeat_interleave(2, -1).view(1, S, 1, D)
    for got, src, w in ((q_out, qkv[:, :, 0], wq), (k_out, qkv[:, :, 1], wk)):
        n = ops.rms_norm_row_fp32(src.float().flatten(2), w).unflatten(2, (H, D))
        _close(got, ops.apply_rotary_wan(n, fc, fs), atol=2e-2, rtol=1e-2, what="wan qk norm+rope")
    assert torch.equal(v_out.cpu(), qkv[:, :, 2])


# ========================================================================================= activations
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_activations(gpu, dtype):
    from vllm_omni_amd import kernels

    x = _rand(3, 1001, seed=1, dtype=dtype, scale=3.0)
    tol = 2 ** -8 if dtype == torch.bfloat16 else 2e-6
    _close(kernels.gelu_tanh(x.to(gpu)), ops.gelu_tanh(x.float()), atol=tol, rtol=tol, what="gelu")
    _close(kernels.silu(x.to(gpu)), torch.nn.functional.silu(x.float()), atol=tol, rtol=tol, what="silu")
    big = torch.tensor([-100.0, -20.0, 0.0, 20.0, 100.0], dtype=dtype)
    _close(kernels.gelu_tanh(big.to(gpu)), ops.gelu_tanh(big.float()), atol=1e-6, rtol=tol, what="gelu tails")


# ========================================================================================= K1
def _attn_inputs(B, Sq, Sk, H, Hkv, D, seed, dtype=torch.bfloat16):
    q = _rand(B, Sq, H, D, seed=seed, dtype=dtype)
    k = _rand(B, Sk, Hkv, D, seed=seed + 1, dtype=dtype)
    v = _rand(B, Sk, Hkv, D, seed=seed + 2, dtype=dtype)
    return q, k, v


def _far_apart_rows(t, gpu):
    """The same [B,S,H,D] values on the GPU as a view whose sequence stride is so large that the rows of one
    (batch, head) span 2 GiB: the library then has to address them through 64-bit pointers (its second attention
    kernel) instead of 32-bit buffer offsets."""
    B, S, H, D = t.shape
    stride = -(-(1 << 30) // (S + 64))
    stride = max((stride + 7) // 8 * 8, H * D)
    big = torch.empty((B, S, stride), dtype=t.dtype, device=gpu)
    view = big[:, :, : H * D].view(B, S, H, D)
    view.copy_(t)
    return view


def _kv_for_path(path, k, v, gpu):
    from vllm_omni_amd import kernels

    if path == "pointer":
        if k.shape[1] == 1:
            pytest.skip("a single key row has no row stride to stretch")
        kg, vg = _far_apart_rows(k, gpu), _far_apart_rows(v, gpu)
    else:
        kg, vg = k.to(gpu), v.to(gpu)
    B, Sk, H, D = k.shape
    plan = kernels.attn_plan(B, 64, Sk, H, D, kg.stride(1), vg.stride(1))
    assert plan.startswith("attn_fwd_pipe_kernel" if path == "pointer" else "attn_fwd_dma_kernel"), plan
    return kg, vg


ATTN_PATHS = ["buffer", "pointer"]   # which of the library's two attention kernels the strides select

ATTN_SHAPES = [
    # B, Sq, Sk, H, Hkv, D
    (2, 64, 64, 8, 8, 64),       # the reference's own test shape (tests/diffusion/attention/test_flash_attn.py)
    (1, 320, 320, 4, 4, 128),    # tiny config-like
    (2, 300, 300, 3, 3, 128),    # ragged: tails in both q blocks and key tiles
    (1, 1, 1, 1, 1, 128),        # smallest possible
    (1, 70, 515, 2, 2, 64),      # cross-attention shape, ragged keys
    (1, 257, 129, 4, 2, 128),    # grouped KV heads
]


@pytest.mark.parametrize("path", ATTN_PATHS)
@pytest.mark.parametrize("shape", ATTN_SHAPES)
def test_attention_parity(gpu, path, shape):
    from vllm_omni_amd import kernels

    B, Sq, Sk, H, Hkv, D = shape
    q, k, v = _attn_inputs(B, Sq, Sk, H, Hkv, D, seed=42)
    scale = 1.0 / math.sqrt(D)
    print(f"attn path={path} shape={shape}", flush=True)
    kg, vg = _kv_for_path(path, k, v, gpu)
    got, lse = kernels.attn_fwd(q.to(gpu), kg, vg, scale, return_lse=True)
    torch.cuda.synchronize()
    want = ops.sdpa(q.float(), k.float(), v.float(), scale)
    # bf16 output of values in [-~3, 3]: error budget = P rounded to bf16 inside + one output rounding
    _close(got, want, atol=2e-2, rtol=2e-2, what="attention")
    assert _cosine(got, want) >= 0.9995
    # the reference's own thresholds for backend agreement (test_flash_attn.py:144-147)
    d = (got.float().cpu() - want).abs()
    assert d.max() < 0.1 and d.mean() < 0.01
    kf = k.float().repeat_interleave(H // Hkv, dim=2)
    s = torch.einsum("bqhd,bkhd->bhqk", q.float(), kf) * scale
    _close(lse, torch.logsumexp(s, dim=-1), atol=2e-2, rtol=1e-3, what="lse")


@pytest.mark.parametrize("path", ATTN_PATHS)
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("order", ["rising", "falling", "random"])
def test_attention_peaked_logits(gpu, path, D, order):
    """Logits with a standard deviation of about 16 and a row maximum that keeps rising (or falling) from one key
    tile to the next: the running-maximum update, the rescaling of the accumulators that is skipped while the
    maximum grows by less than 2^8, and probabilities that underflow to zero, against an fp64 softmax."""
    from vllm_omni_amd import kernels

    B, Sq, Sk, H = 1, 200, 700, 2
    q, k, v = _attn_inputs(B, Sq, Sk, H, H, D, seed=77)
    ramp = torch.linspace(0.5, 7.5, Sk).view(1, Sk, 1, 1)
    if order == "falling":
        ramp = ramp.flip(1)
    elif order == "random":
        ramp = ramp[:, torch.randperm(Sk, generator=torch.Generator().manual_seed(5))]
    k = (k.float() * ramp).bfloat16()
    q = (q.float() * 4.0).bfloat16()
    scale = 1.0 / math.sqrt(D)
    kg, vg = _kv_for_path(path, k, v, gpu)
    got, lse = kernels.attn_fwd(q.to(gpu), kg, vg, scale, return_lse=True)
    s = torch.einsum("bqhd,bkhd->bhqk", q.double(), k.double()) * scale
    assert s.std() > 10 and s.max() > 80            # far outside what N(0,1) inputs reach
    want = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, dim=-1), v.double())
    _close(got, want.float(), atol=2e-2, rtol=2e-2, what=f"peaked attention ({order})")
    _close(lse, torch.logsumexp(s, dim=-1).float(), atol=2e-2, rtol=1e-3, what="lse")


def test_attention_fp16_and_strided_views(gpu):
    from vllm_omni_amd import kernels

    B, S, H, D = 2, 200, 4, 128
    qkv = _rand(B, S, 3, H, D, seed=7, dtype=torch.float16)
    g = qkv.to(gpu)
    got = kernels.attn_fwd(g[:, :, 0], g[:, :, 1], g[:, :, 2], 0.09)   # views of a fused buffer, no copies
    want = ops.sdpa(qkv[:, :, 0].float(), qkv[:, :, 1].float(), qkv[:, :, 2].float(), 0.09)
    _close(got, want, atol=3e-3, rtol=3e-3, what="fp16 strided attention")


def test_attention_key_mask_equals_deleting_keys(gpu):
    """The reference's padding-equivalence property (test_flash_attn.py:60-147)."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd.attention.backends.abstract import AttentionMetadata
    from vllm_omni_amd.attention.layer import Attention

    B, S, H, D, pad = 2, 84, 8, 64, 20
    q, k, v = _attn_inputs(B, S, S, H, H, D, seed=123)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[:, S - pad:] = False
    layer = Attention(num_heads=H, head_size=D, causal=False, softmax_scale=0.125)
    got = layer(q.to(gpu), k.to(gpu), v.to(gpu), AttentionMetadata(attn_mask=mask.to(gpu)))
    unpadded = kernels.attn_fwd(q.to(gpu), k[:, :S - pad].to(gpu), v[:, :S - pad].to(gpu), 0.125)
    assert torch.equal(got.cpu(), unpadded.cpu()), "masking keys must equal removing them"
    _close(got, ops.sdpa(q.float(), k.float(), v.float(), 0.125, key_mask=mask), atol=2e-2, rtol=2e-2)
    # scattered mask, different per batch row
    g = torch.Generator().manual_seed(5)
    m2 = torch.rand(B, S, generator=g) > 0.3
    m2[:, 0] = True
    got2 = kernels.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu), 0.125, key_mask=m2.to(gpu))
    _close(got2, ops.sdpa(q.float(), k.float(), v.float(), 0.125, key_mask=m2), atol=2e-2, rtol=2e-2)
    # single excluded keys at tile edges, a fully excluded first tile, everything but one key excluded
    for S2, cut in ((64, [63]), (128, [0, 64, 127]), (128, list(range(0, 64))), (200, list(range(1, 200)))):
        q2, k2, v2 = _attn_inputs(1, S2, S2, 2, 2, 64, seed=S2)
        m3 = torch.ones(1, S2, dtype=torch.bool)
        m3[:, cut] = False
        got3 = kernels.attn_fwd(q2.to(gpu), k2.to(gpu), v2.to(gpu), 0.125, key_mask=m3.to(gpu))
        _close(got3, ops.sdpa(q2.float(), k2.float(), v2.float(), 0.125, key_mask=m3), atol=2e-2, rtol=2e-2,
               what=f"mask S={S2} cut={cut[:3]}")
    # a batch row with every key excluded returns zeros (and a log-sum-exp of -inf); the other row is untouched
    m4 = torch.ones(B, S, dtype=torch.bool)
    m4[1] = False
    got4, lse4 = kernels.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu), 0.125, key_mask=m4.to(gpu), return_lse=True)
    assert torch.count_nonzero(got4[1]) == 0 and bool(torch.isneginf(lse4[1]).all())
    assert torch.equal(got4[0].cpu(), layer(q.to(gpu), k.to(gpu), v.to(gpu))[0].cpu())
    # an all-true mask is dropped and gives the unmasked result bit for bit
    ones = AttentionMetadata(attn_mask=torch.ones(B, S, dtype=torch.bool, device=gpu))
    assert torch.equal(layer(q.to(gpu), k.to(gpu), v.to(gpu), ones).cpu(),
                       layer(q.to(gpu), k.to(gpu), v.to(gpu)).cpu())


@pytest.mark.parametrize("path", ATTN_PATHS)
@pytest.mark.parametrize("split", [0, 1, 37, 64, 299, 300])
def test_attention_split_output_equals_slices(gpu, path, split):
    """Two dense outputs written by the kernel == slices of the single output, bit for bit."""
    from vllm_omni_amd import kernels

    B, S, H, D = 2, 300, 3, 128
    q, k, v = _attn_inputs(B, S, S, H, H, D, seed=77)
    q = q.to(gpu)
    k, v = _kv_for_path(path, k, v, gpu)
    print(f"attn split path={path} split={split}", flush=True)
    whole, lse = kernels.attn_fwd(q, k, v, 0.09, return_lse=True)
    head, tail, lse2 = kernels.attn_fwd(q, k, v, 0.09, return_lse=True, split=split)
    assert head.shape == (B, split, H, D) and tail.shape == (B, S - split, H, D)
    assert head.is_contiguous() and tail.is_contiguous()
    assert torch.equal(head.cpu(), whole[:, :split].cpu())
    assert torch.equal(tail.cpu(), whole[:, split:].cpu())
    assert torch.equal(lse.cpu(), lse2.cpu())
    with pytest.raises(ValueError):
        kernels.attn_fwd(q, k, v, 0.09, split=S + 1)


KEY_SPLIT_SHAPES = [
    # B, Sq, Sk, H, Hkv, D: few workgroups, many key tiles -> the last (only) round is cut along the keys
    (1, 300, 1100, 3, 3, 128),    # ragged queries and keys; ranges of 10 + 8 tiles
    (2, 64, 4352, 8, 8, 64),      # one q block per head, 68 tiles in up to 8 ranges
    (1, 130, 2048, 4, 2, 128),    # grouped KV heads, second q block almost empty
    (1, 1, 1030, 1, 1, 128),      # a single query row, 17 tiles in two ranges
]


@pytest.mark.parametrize("shape", KEY_SPLIT_SHAPES)
def test_attention_key_split_tail(gpu, shape):
    """The launch that cuts its last round of workgroups into key ranges and merges them must agree with
    the single-pass launch and with the oracle: plain, with a key mask, with LSE and with two outputs."""
    from vllm_omni_amd import _lib, kernels

    B, Sq, Sk, H, Hkv, D = shape
    assert _lib.load().odit_attn_fwd_workspace_bytes(B, Sq, Sk, H, D) > 0, "shape does not exercise the key split"
    assert "attn_merge_kernel" in kernels.attn_plan(B, Sq, Sk, H, D)
    assert "attn_merge_kernel" not in kernels.attn_plan(B, Sq, Sk, H, D, use_workspace=False)
    q, k, v = _attn_inputs(B, Sq, Sk, H, Hkv, D, seed=5)
    scale = 1.0 / math.sqrt(D)
    print(f"attn key-split shape={shape}", flush=True)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    one, lse1 = kernels.attn_fwd(qg, kg, vg, scale, return_lse=True, use_workspace=False)
    two, lse2 = kernels.attn_fwd(qg, kg, vg, scale, return_lse=True)
    torch.cuda.synchronize()
    want = ops.sdpa(q.float(), k.float(), v.float(), scale)
    _close(two, want, atol=2e-2, rtol=2e-2, what="key-split attention vs oracle")
    assert _cosine(two, want) >= 0.9995
    _close(two, one, atol=8e-3, rtol=8e-3, what="key-split vs single pass")   # one bf16 ulp of O(1) values
    _close(lse2, lse1, atol=1e-4, rtol=1e-5, what="lse")
    again = kernels.attn_fwd(qg, kg, vg, scale)
    assert torch.equal(again, two), "the partition is fixed: repeated calls are bit-identical"
    # key mask: scattered, plus one whole key range excluded (its partial must get weight zero)
    g = torch.Generator().manual_seed(8)
    m = torch.rand(B, Sk, generator=g) > 0.3
    m[:, : min(Sk // 2, 640)] = False
    m[:, -1] = True
    got_m = kernels.attn_fwd(qg, kg, vg, scale, key_mask=m.to(gpu))
    _close(got_m, ops.sdpa(q.float(), k.float(), v.float(), scale, key_mask=m), atol=2e-2, rtol=2e-2,
           what="key-split with mask")
    none = torch.zeros(B, Sk, dtype=torch.bool, device=gpu)
    got0, lse0 = kernels.attn_fwd(qg, kg, vg, scale, key_mask=none, return_lse=True)
    assert torch.count_nonzero(got0) == 0 and bool(torch.isneginf(lse0).all()), "every key excluded: zeros"
    if Sq > 2:
        cut = Sq // 3
        head, tail = kernels.attn_fwd(qg, kg, vg, scale, split=cut)
        assert torch.equal(head, two[:, :cut]) and torch.equal(tail, two[:, cut:])
    # peaked logits whose row maximum rises along the keys: the last key range outweighs the others by far
    # more than 2^126, so the merge has to take weights of exactly zero without producing NaN
    ramp = torch.linspace(0.5, 7.5, Sk).view(1, Sk, 1, 1)
    kp, qp = (k.float() * ramp).bfloat16(), (q.float() * 4.0).bfloat16()
    sp = torch.einsum("bqhd,bkhd->bhqk", qp.double(), kp.double().repeat_interleave(H // Hkv, dim=2)) * scale
    wantp = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(sp, dim=-1), v.double().repeat_interleave(H // Hkv, dim=2))
    gotp, lsep = kernels.attn_fwd(qp.to(gpu), kp.to(gpu), vg, scale, return_lse=True)
    _close(gotp, wantp.float(), atol=2e-2, rtol=2e-2, what="key-split, peaked logits")
    _close(lsep, torch.logsumexp(sp, dim=-1).float(), atol=2e-2, rtol=1e-3, what="key-split, peaked logits, lse")


_PERSISTENT_CHILD = """
import sys, torch
from vllm_omni_amd import kernels
d = torch.load(sys.argv[1])
q, k, v, m = (d[n].cuda() for n in ("q", "k", "v", "m"))
assert "persistent workgroups" in kernels.attn_plan(q.shape[0], q.shape[1], k.shape[1], q.shape[2], q.shape[3])
out = {}
for rep in range(3):            # the ticket words are back at zero after every launch
    out[f"plain{rep}"], out[f"lse{rep}"] = (t.cpu() for t in kernels.attn_fwd(q, k, v, d["scale"], return_lse=True))
out["masked"] = kernels.attn_fwd(q, k, v, d["scale"], key_mask=m).cpu()
torch.save(out, sys.argv[2])
"""


def test_attention_persistent_form_matches_the_default_form(gpu, tmp_path):
    """The measurement mode ODIT_ATTN_PERSISTENT=1 (resident workgroups that draw unit after unit from ticket words
    in the scratch) gives the default form's results bit for bit, also on repeated launches over the same ticket
    words, with a key mask, and with a last round that is cut along the keys. The variable is read once per
    process, so the persistent form runs in a child process."""
    import os
    import subprocess
    import sys

    from vllm_omni_amd import kernels

    B, Sq, S, H, D = 2, 2816, 1408, 24, 128  # 22 query blocks x 48 = 1056 units on 512 slots (two rounds + 32), 22 key tiles
    q, k, v = _attn_inputs(B, Sq, S, H, H, D, seed=91)
    m = torch.rand(B, S, generator=torch.Generator().manual_seed(3)) > 0.2
    scale = 1.0 / math.sqrt(D)
    plan = kernels.attn_plan(B, Sq, S, H, D)
    assert "persistent" not in plan and "attn_merge_kernel" in plan
    want, want_lse = kernels.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu), scale, return_lse=True)
    want_m = kernels.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu), scale, key_mask=m.to(gpu))
    torch.save({"q": q, "k": k, "v": v, "m": m, "scale": scale}, tmp_path / "in.pt")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    # (the persistent form exists for workgroups of 4 wavefronts; the rows of this shape that fall into the last,
    # key-split round are the same for workgroups of 4 and of 8 wavefronts, so the results can be compared bit for bit)
    env = dict(os.environ, ODIT_ATTN_PERSISTENT="1", ODIT_ATTN_WAVES="4", PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    proc = subprocess.run([sys.executable, "-c", _PERSISTENT_CHILD, str(tmp_path / "in.pt"), str(tmp_path / "out.pt")],
                          env=env, capture_output=True, text=True, timeout=100)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = torch.load(tmp_path / "out.pt")
    for rep in range(3):
        assert torch.equal(got[f"plain{rep}"], want.cpu()), rep
        assert torch.equal(got[f"lse{rep}"], want_lse.cpu()), rep
    assert torch.equal(got["masked"], want_m.cpu())


@pytest.mark.parametrize("shape,cut", [((2, 300, 300, 4, 4, 128), 64), ((1, 1100, 1100, 3, 3, 64), 256),
                                       ((2, 130, 2048, 4, 2, 128), 1024), ((1, 300, 1100, 3, 3, 128), 192),
                                       ((2, 200, 200, 2, 2, 128), 70)])
def test_attention_values_in_two_tensors(gpu, shape, cut):
    """Value rows of keys [0, cut) and [cut, Sk) taken from two tensors (strided views of two wider
    buffers, like the value thirds of two fused-QKV outputs) give the result of the concatenated tensor bit
    for bit: plain, masked, with two outputs, and on launches that split their last round by keys. A cut
    that is not a multiple of 64 (last case) goes through a concatenation inside the wrapper, which counts it."""
    from vllm_omni_amd import kernels

    B, Sq, Sk, H, Hkv, D = shape
    copies_before = kernels.HIDDEN_COPIES["attn_value_pair_concatenated"]
    q, k, v = _attn_inputs(B, Sq, Sk, H, Hkv, D, seed=11)
    scale = 1.0 / math.sqrt(D)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    wide_a = torch.zeros(B, cut, 3, Hkv, D, dtype=v.dtype, device=gpu)
    wide_b = torch.zeros(B, Sk - cut, 3, Hkv, D, dtype=v.dtype, device=gpu)
    wide_a[:, :, 2], wide_b[:, :, 2] = vg[:, :cut], vg[:, cut:]
    pair = (wide_a[:, :, 2], wide_b[:, :, 2])
    want = kernels.attn_fwd(qg, kg, vg, scale)
    assert torch.equal(kernels.attn_fwd(qg, kg, pair, scale), want)
    assert kernels.HIDDEN_COPIES["attn_value_pair_concatenated"] - copies_before == (0 if cut % 64 == 0 else 1)
    m = torch.rand(B, Sk, generator=torch.Generator().manual_seed(12)) > 0.3
    m[:, -1] = True
    assert torch.equal(kernels.attn_fwd(qg, kg, pair, scale, key_mask=m.to(gpu)),
                       kernels.attn_fwd(qg, kg, vg, scale, key_mask=m.to(gpu)))
    head, tail = kernels.attn_fwd(qg, kg, pair, scale, split=Sq // 3)
    assert torch.equal(head, want[:, :Sq // 3]) and torch.equal(tail, want[:, Sq // 3:])
    _close(want, ops.sdpa(q.float(), k.float(), v.float(), scale), atol=2e-2, rtol=2e-2, what="attention vs oracle")
    with pytest.raises(ValueError, match="does not cover"):
        kernels.attn_fwd(qg, kg, (pair[0], pair[1][:, :-1]), scale)


def test_attention_workspace_too_small_is_an_error(gpu):
    from vllm_omni_amd import _lib

    lib = _lib.load()
    B, Sq, Sk, H, D = 1, 128, 2048, 2, 128
    need = lib.odit_attn_fwd_workspace_bytes(B, Sq, Sk, H, D)
    assert need > 0
    q = torch.zeros(B, Sq, H, D, device=gpu, dtype=torch.bfloat16)
    o = torch.empty_like(q)
    ws = torch.empty(need, device=gpu, dtype=torch.uint8)
    st = _lib.i64_array(q.stride()[:3])
    rc = lib.odit_attn_fwd_ex(q.data_ptr(), q.data_ptr(), q.data_ptr(), None, 0, o.data_ptr(), None, 0, None, None,
                              B, Sq, Sq, H, H, D, st, st, st, None, st, None, 0.1, 0, ws.data_ptr(), 16, None)
    assert rc == 0  # Sk = 128: nothing to split, any workspace size is fine
    k = torch.zeros(B, Sk, H, D, device=gpu, dtype=torch.bfloat16)
    sk = _lib.i64_array(k.stride()[:3])
    rc = lib.odit_attn_fwd_ex(q.data_ptr(), k.data_ptr(), k.data_ptr(), None, 0, o.data_ptr(), None, 0, None, None,
                              B, Sq, Sk, H, H, D, st, sk, sk, None, st, None, 0.1, 0, ws.data_ptr(), need - 1, None)
    assert rc == -4 and b"workspace" in lib.odit_last_error()
    # values in two tensors: the cut must be a whole number of 64-key tiles, the row strides equal
    rc = lib.odit_attn_fwd_ex(q.data_ptr(), k.data_ptr(), k.data_ptr(), k.data_ptr(), 100, o.data_ptr(), None, 0, None,
                              None, B, Sq, Sk, H, H, D, st, sk, sk, sk, st, None, 0.1, 0, None, 0, None)
    assert rc == -1 and b"multiple of 64" in lib.odit_last_error()
    bad = _lib.i64_array((k.stride(0), 2 * k.stride(1), k.stride(2)))
    rc = lib.odit_attn_fwd_ex(q.data_ptr(), k.data_ptr(), k.data_ptr(), k.data_ptr(), 64, o.data_ptr(), None, 0, None,
                              None, B, Sq, Sk, H, H, D, st, sk, sk, bad, st, None, 0.1, 0, None, 0, None)
    assert rc == -1 and b"row stride" in lib.odit_last_error()
    torch.cuda.synchronize()


def test_attention_fp32_goes_to_sdpa(gpu):
    from vllm_omni_amd.attention.layer import Attention

    q, k, v = _attn_inputs(1, 40, 40, 2, 2, 64, seed=9, dtype=torch.float32)
    layer = Attention(num_heads=2, head_size=64, causal=False, softmax_scale=0.125)
    _close(layer(q.to(gpu), k.to(gpu), v.to(gpu)), ops.sdpa(q, k, v, 0.125), atol=1e-4, rtol=1e-4)


def test_attention_full_size_properties(gpu):
    """BASELINE config 2 shape (B=2, 24 heads x 128, 4096 image + 256 text tokens): properties that
    do not need the full CPU product, plus the oracle on two heads."""
    from vllm_omni_amd import kernels

    B, S, H, D = 2, 4352, 24, 128
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator(device="cpu").manual_seed(0)
    q = torch.randn(B, S, H, D, generator=g).bfloat16().to(gpu)
    k = torch.randn(B, S, H, D, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, S, H, D, generator=g).bfloat16().to(gpu)
    out, lse = kernels.attn_fwd(q, k, v, scale, return_lse=True)
    # (1) V = 1 -> every output is exactly 1 up to the final rounding of sum(P)/sum(P)
    ones = kernels.attn_fwd(q, k, torch.ones_like(v), scale)
    _close(ones, torch.ones(1), atol=2 ** -7, what="rows of P sum to 1")
    # (2) permuting keys with their values leaves the result unchanged (to rounding)
    perm = torch.randperm(S, generator=g).to(gpu)
    outp = kernels.attn_fwd(q, k[:, perm].contiguous(), v[:, perm].contiguous(), scale)
    _close(outp, out, atol=2e-2, what="key permutation invariance")
    # (3) split keys in two halves and merge with the LSE identity
    oa, la = kernels.attn_fwd(q, k[:, :2000], v[:, :2000], scale, return_lse=True)
    ob, lb = kernels.attn_fwd(q, k[:, 2000:], v[:, 2000:], scale, return_lse=True)
    merged, lse_m = ops.merge_lse(oa.float(), la, ob.float(), lb)
    _close(merged, out, atol=2e-2, what="split-K + LSE merge")
    _close(lse_m, lse, atol=1e-2, what="merged lse")
    # (4) oracle on two (batch, head) slices
    for b, h in ((0, 0), (1, 23)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].float().cpu()  # noqa: E731
        want = ops.sdpa(sl(q), sl(k), sl(v), scale)
        _close(out[b:b + 1, :, h:h + 1], want, atol=2e-2, rtol=2e-2, what=f"head ({b},{h})")
        assert _cosine(out[b:b + 1, :, h:h + 1], want) >= 0.9995


def test_attention_wan_sequence_properties(gpu):
    """BASELINE config 4's self-attention shape (B=2, 40 heads x 128, 32 760 video tokens = 511 key tiles of
    64 and a ragged one of 56; 256 query blocks per head with the last one ragged too): size-independent
    properties plus the oracle on slices (rows from the first, a middle and the ragged last query block of
    two (batch, head) pairs against all 32 760 keys)."""
    from vllm_omni_amd import kernels

    B, S, H, D = 2, 32760, 40, 128
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator(device=gpu).manual_seed(4)
    q, k, v = (torch.randn(B, S, H, D, generator=g, device=gpu, dtype=torch.float32).bfloat16() for _ in range(3))
    print(f"wan attention plan: {kernels.attn_plan(B, S, S, H, D)}", flush=True)
    out, lse = kernels.attn_fwd(q, k, v, scale, return_lse=True)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out.float()).all()) and bool(torch.isfinite(lse).all())
    # (1) V = 1: every output is 1 up to the final rounding
    ones = kernels.attn_fwd(q, k, torch.ones_like(v), scale)
    err1 = (ones.float() - 1).abs().max().item()
    assert err1 <= 2 ** -7, f"rows of P sum to 1: {err1}"
    del ones
    # (2) permuting keys with their values changes nothing (to rounding: the order of the key sum moves)
    perm = torch.randperm(S, generator=g, device=gpu)
    outp = kernels.attn_fwd(q, k[:, perm].contiguous(), v[:, perm].contiguous(), scale)
    errp = (outp.float() - out.float()).abs().max().item()
    assert errp <= 2e-2, f"key permutation invariance: {errp}"
    del outp
    # (3) keys cut at 16 001 (inside a tile) and merged with the log-sum-exp identity
    cut = 16001
    oa, la = kernels.attn_fwd(q, k[:, :cut], v[:, :cut], scale, return_lse=True)
    ob, lb = kernels.attn_fwd(q, k[:, cut:], v[:, cut:], scale, return_lse=True)
    w_a = torch.exp(la - torch.maximum(la, lb)).transpose(1, 2).unsqueeze(-1)     # [B,S,H,1]
    w_b = torch.exp(lb - torch.maximum(la, lb)).transpose(1, 2).unsqueeze(-1)
    merged = (oa.float() * w_a + ob.float() * w_b) / (w_a + w_b)
    errm = (merged - out.float()).abs().max().item()
    lse_m = torch.maximum(la, lb) + torch.log(torch.exp(la - torch.maximum(la, lb)) + torch.exp(lb - torch.maximum(la, lb)))
    assert errm <= 2e-2 and (lse_m - lse).abs().max().item() <= 1e-2, f"split-K + LSE merge: {errm}"
    del oa, ob, merged
    # (4) the oracle, fp32 on the CPU, on query rows of three blocks of two (batch, head) pairs
    rows = torch.cat([torch.arange(0, 256), torch.arange(16384, 16384 + 256), torch.arange(S - 200, S)])
    worst, worst_cos = 0.0, 1.0
    for b, h in ((0, 0), (1, 39)):
        qs = q[b:b + 1, rows, h:h + 1].float().cpu()
        ks, vs = k[b:b + 1, :, h:h + 1].float().cpu(), v[b:b + 1, :, h:h + 1].float().cpu()
        want = ops.sdpa(qs, ks, vs, scale)
        got = out[b:b + 1, rows, h:h + 1]
        _close(got, want, atol=2e-2, rtol=2e-2, what=f"wan-sequence attention, head ({b},{h})")
        worst = max(worst, (got.float().cpu() - want).abs().max().item())
        worst_cos = min(worst_cos, _cosine(got, want))
        s = torch.einsum("bqhd,bkhd->bhqk", qs, ks) * scale
        _close(lse[b:b + 1, h:h + 1][:, :, rows], torch.logsumexp(s, dim=-1), atol=2e-2, rtol=1e-3, what="lse")
    print(f"wan-sequence attention: V=1 err {err1:.2e}, permutation {errp:.2e}, split+merge {errm:.2e}, "
          f"oracle max-abs {worst:.2e}, cosine {worst_cos:.6f}", flush=True)
    assert worst_cos >= 0.9995


def test_joint_attention_composed_at_full_size(gpu):
    """BASELINE config 2 end to end: fused-QKV outputs of the image stream (4096 tokens, 64x64 grid) and the
    text stream (256 tokens), per-head QK-RMSNorm (eps 1e-6), rotary on the image rows from the model's own
    3-axis tables (theta 10000; frame axis at position 0, rows and columns centred), text rows unrotated
    (cos = 1, sin = 0), written into the joint [text; image] buffers by the fused kernel, then the joint
    attention over 4352 tokens with the values read in place from the two projection outputs — against
    sdpa(rotary(rms_norm(.))) of the oracle on two heads per batch row."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD
    from vllm_omni_amd.blocks.qwen_image import QwenEmbedRope

    B, S_img, S_txt, H, D = 2, 4096, 256, 24, 128
    S = S_img + S_txt
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator(device=gpu).manual_seed(6)
    img_qkv = torch.randn(B, S_img, 3, H, D, generator=g, device=gpu).bfloat16()
    txt_qkv = torch.randn(B, S_txt, 3, H, D, generator=g, device=gpu).bfloat16()
    w = [(torch.randn(D, generator=g, device=gpu) * 0.2 + 1).bfloat16() for _ in range(4)]   # q, k, added q, added k
    vid, _ = QwenEmbedRope(theta=10000, axes_dim=[16, 56, 56], scale_rope=True)([(1, 64, 64)], [S_txt], gpu)
    img_cos, img_sin = vid.real.contiguous(), vid.imag.contiguous()
    txt_cos, txt_sin = torch.ones(S_txt, D // 2, device=gpu), torch.zeros(S_txt, D // 2, device=gpu)
    jq = torch.empty(B, S, H, D, dtype=torch.bfloat16, device=gpu)
    jk = torch.empty_like(jq)
    kernels.qknorm_rope(txt_qkv[:, :, 0], txt_qkv[:, :, 1], None, jq, jk, None, w[2], w[3], txt_cos, txt_sin,
                        eps=1e-6, out_seq_offset=0, norm_mode=ODIT_NORM_HEAD)
    kernels.qknorm_rope(img_qkv[:, :, 0], img_qkv[:, :, 1], None, jq, jk, None, w[0], w[1], img_cos, img_sin,
                        eps=1e-6, out_seq_offset=S_txt, norm_mode=ODIT_NORM_HEAD)
    copies = dict(kernels.HIDDEN_COPIES)
    txt_o, img_o = kernels.attn_fwd(jq, jk, (txt_qkv[:, :, 2], img_qkv[:, :, 2]), scale, split=S_txt)
    torch.cuda.synchronize()
    assert kernels.HIDDEN_COPIES == copies, "the values must be read where the projections left them"
    assert txt_o.shape == (B, S_txt, H, D) and img_o.shape == (B, S_img, H, D)
    c = lambda t: t.float().cpu()  # noqa: E731
    worst, worst_cos = 0.0, 1.0
    for b, h in ((0, 0), (0, 13), (1, 5), (1, 23)):
        hs = slice(h, h + 1)

        def prep(col, w_img, w_txt):
            xi = ops.apply_rotary(ops.rms_norm_head(c(img_qkv[b:b + 1, :, col, hs]), c(w_img)), c(img_cos), c(img_sin))
            xt = ops.rms_norm_head(c(txt_qkv[b:b + 1, :, col, hs]), c(w_txt))          # text rows are not rotated
            return torch.cat([xt, xi], dim=1)

        want = ops.sdpa(prep(0, w[0], w[2]), prep(1, w[1], w[3]),
                        torch.cat([c(txt_qkv[b:b + 1, :, 2, hs]), c(img_qkv[b:b + 1, :, 2, hs])], dim=1), scale)
        got = torch.cat([txt_o[b:b + 1, :, hs], img_o[b:b + 1, :, hs]], dim=1)
        _close(got, want, atol=2e-2, rtol=2e-2, what=f"composed joint attention, head ({b},{h})")
        worst = max(worst, (c(got) - want).abs().max().item())
        worst_cos = min(worst_cos, _cosine(got, want))
    print(f"composed joint attention at 4352 tokens: max-abs {worst:.2e}, cosine {worst_cos:.6f}", flush=True)
    assert worst_cos >= 0.9995
