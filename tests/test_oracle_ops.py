"""Pins the oracle's per-op functions WITHOUT retyping their formulas: library routines, closed
forms, brute force on tiny inputs and invariants, each chosen so a dropped term / wrong sign / wrong
index / transposed operand fails."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ops


def _rand(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


# ----------------------------------------------------------------------------------- attention
def test_sdpa_matches_library_routine():
    # torch SDPA on CPU fp32 is the very call the reference's SDPA backend makes
    for seed, (B, S, H, D) in [(42, (2, 64, 8, 64)), (123, (1, 37, 3, 128))]:
        q, k, v = (_rand(B, S, H, D, seed=seed + i) for i in range(3))
        ref = F.scaled_dot_product_attention(*(t.transpose(1, 2) for t in (q, k, v)), scale=0.3).transpose(1, 2)
        assert torch.allclose(ops.sdpa(q, k, v, 0.3), ref, atol=2e-6, rtol=1e-5)


def test_sdpa_brute_force_fp64_tiny():
    B, S, H, D = 1, 5, 2, 4
    q, k, v = (_rand(B, S, H, D, seed=i).double() for i in range(3))
    out = torch.zeros(B, S, H, D, dtype=torch.float64)
    for h in range(H):
        for i in range(S):
            w = [math.exp(0.5 * float(q[0, i, h] @ k[0, j, h])) for j in range(S)]
            z = sum(w)
            for j in range(S):
                out[0, i, h] += (w[j] / z) * v[0, j, h]
    assert torch.allclose(ops.sdpa(q.float(), k.float(), v.float(), 0.5).double(), out, atol=1e-5)


def test_sdpa_invariants():
    B, S, H, D = 2, 48, 3, 32
    q, k, v = (_rand(B, S, H, D, seed=10 + i) for i in range(3))
    # rows of P sum to one
    assert torch.allclose(ops.sdpa(q, k, torch.ones_like(v), 0.2), torch.ones_like(v), atol=1e-6)
    # permuting keys together with values changes nothing
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(5))
    assert torch.allclose(ops.sdpa(q, k[:, perm], v[:, perm], 0.2), ops.sdpa(q, k, v, 0.2), atol=1e-5)
    # a key mask equals deleting the masked keys (the reference's own padding-equivalence property,
    # tests/diffusion/attention/test_flash_attn.py:60-147)
    mask = torch.ones(B, S, dtype=torch.bool)
    mask[:, 30:] = False
    assert torch.allclose(ops.sdpa(q, k, v, 0.2, key_mask=mask), ops.sdpa(q, k[:, :30], v[:, :30], 0.2), atol=1e-6)


def test_tiled_online_softmax_and_lse_merge():
    B, S, H, D = 1, 100, 2, 16
    q, k, v = (_rand(B, S, H, D, seed=20 + i) for i in range(3))
    full = ops.sdpa(q, k, v, 0.25)
    tiled, lse = ops.sdpa_tiled(q, k, v, 0.25, tile=32)
    assert torch.allclose(tiled, full, atol=1e-5)
    # lse against logsumexp of the explicit score matrix
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) * 0.25
    assert torch.allclose(lse, torch.logsumexp(s, dim=-1), atol=1e-5)
    # split keys in two, merge with the ring-attention identity, compare to unsplit
    oa, la = ops.sdpa_tiled(q, k[:, :40], v[:, :40], 0.25)
    ob, lb = ops.sdpa_tiled(q, k[:, 40:], v[:, 40:], 0.25)
    merged, lse_m = ops.merge_lse(oa, la, ob, lb)
    assert torch.allclose(merged, full, atol=1e-5)
    assert torch.allclose(lse_m, lse, atol=1e-5)


# ----------------------------------------------------------------------------------- RMSNorm
def test_rms_norm_properties():
    x = _rand(3, 7, 4, 64, seed=1)
    w = _rand(64, seed=2).abs() + 0.5
    y = ops.rms_norm_head(x, w, eps=0.0)
    # ||y / w||_2 = sqrt(D) for every head row; scale invariance
    assert torch.allclose((y / w).norm(dim=-1), torch.full((3, 7, 4), 8.0), atol=1e-4)
    assert torch.allclose(ops.rms_norm_head(3.7 * x, w, eps=0.0), y, atol=1e-5)
    # against torch's own rms_norm (library routine)
    assert torch.allclose(ops.rms_norm_head(x, w, 1e-6), F.rms_norm(x, (64,), w, 1e-6), atol=1e-6)
    # row variant agrees with the library routine over the whole row
    xr = _rand(2, 5, 256, seed=3)
    wr = _rand(256, seed=4)
    assert torch.allclose(ops.rms_norm_row_fp32(xr, wr, 1e-6), F.rms_norm(xr, (256,), wr, 1e-6), atol=1e-5)


def test_rms_norm_cast_order_bf16():
    # normalised value is rounded to bf16 BEFORE the weight multiply (two roundings, not one)
    x = _rand(1, 1, 1, 64, seed=5).bfloat16()
    w = (_rand(64, seed=6) * 0.1 + 1.0).bfloat16()
    n = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    assert torch.equal(ops.rms_norm_head(x, w, 1e-6), n * w)


# ----------------------------------------------------------------------------------- rotary
def _tables(S, half, seed=0):
    ang = _rand(S, half, seed=seed) * 3.0
    return torch.cos(ang), torch.sin(ang), torch.polar(torch.ones_like(ang), ang)


def test_rotary_against_complex_product_and_invariants():
    B, S, H, D = 2, 9, 3, 16
    x = _rand(B, S, H, D, seed=7)
    cos, sin, freqs = _tables(S, D // 2, seed=8)
    y = ops.apply_rotary(x, cos, sin, interleaved=True)
    assert torch.allclose(y, ops.apply_rotary_complex(x, freqs), atol=1e-6)
    # per-pair norms are preserved, and rotating back by -theta is the identity
    pn = lambda t: t.unflatten(-1, (-1, 2)).norm(dim=-1)  # noqa: E731
    assert torch.allclose(pn(y), pn(x), atol=1e-5)
    assert torch.allclose(ops.apply_rotary(y, cos, -sin, interleaved=True), x, atol=1e-5)
    # cos = 1, sin = 0 is the identity (unrotated text rows)
    assert torch.equal(ops.apply_rotary(x, torch.ones_like(cos), torch.zeros_like(sin)), x)
    # partial rotary leaves the tail untouched
    yp = ops.apply_rotary(x, cos[:, :4], sin[:, :4])
    assert torch.equal(yp[..., 8:], x[..., 8:]) and not torch.allclose(yp[..., :8], x[..., :8])


def test_rotary_relative_position_property():
    # <rope(q, m), rope(k, n)> depends on m - n only
    D = 32
    inv = 1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))
    pos = torch.arange(12).float()
    ang = torch.outer(pos, inv)
    q = _rand(1, 1, 1, D, seed=9).expand(1, 12, 1, D)
    k = _rand(1, 1, 1, D, seed=10).expand(1, 12, 1, D)
    rq = ops.apply_rotary(q, ang.cos(), ang.sin())
    rk = ops.apply_rotary(k, ang.cos(), ang.sin())
    dots = torch.einsum("bmhd,bnhd->mn", rq, rk)
    for d in (-3, 0, 5):
        diag = torch.diagonal(dots, offset=d)
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-4)


def test_rotary_neox_is_interleaved_on_permuted_axes():
    B, S, H, D = 1, 4, 2, 8
    x = _rand(B, S, H, D, seed=11)
    cos, sin, _ = _tables(S, D // 2, seed=12)
    # de-interleave: neox on [evens | odds] equals interleaved on the original, re-split the same way
    xi = x
    xn = torch.cat((x[..., 0::2], x[..., 1::2]), dim=-1)
    yi = ops.apply_rotary(xi, cos, sin, interleaved=True)
    yn = ops.apply_rotary(xn, cos, sin, interleaved=False)
    assert torch.allclose(yn, torch.cat((yi[..., 0::2], yi[..., 1::2]), dim=-1), atol=1e-6)


def test_rotary_wan_equals_interleaved_with_half_tables():
    B, S, H, D = 1, 6, 2, 8
    x = _rand(B, S, H, D, seed=13)
    cos, sin, _ = _tables(S, D // 2, seed=14)
    fc = cos.repeat_interleave(2, dim=-1).view(1, S, 1, D)
    fs = sin.repeat_interleave(2, dim=-1).view(1, S, 1, D)
    assert torch.allclose(ops.apply_rotary_wan(x, fc, fs), ops.apply_rotary(x, cos, sin), atol=1e-6)


# ----------------------------------------------------------------------------------- adaLN / residual
def test_ada_layer_norm_against_library_and_closed_forms():
    B, S, C = 2, 5, 48
    x = _rand(B, S, C, seed=15) * 3 + 1
    mod = _rand(B, 3 * C, seed=16)
    out, gate = ops.ada_layer_norm(x, mod)
    shift, scale, g = mod[:, :C], mod[:, C:2 * C], mod[:, 2 * C:]
    ln = F.layer_norm(x, (C,), eps=1e-6)
    assert torch.allclose(out, ln * (1 + scale[:, None]) + shift[:, None], atol=1e-6)
    assert torch.equal(gate, g[:, None])
    # scale = shift = 0 -> zero-mean, unit-variance rows
    z, _ = ops.ada_layer_norm(x, torch.zeros(B, 3 * C))
    assert torch.allclose(z.mean(-1), torch.zeros(B, S), atol=1e-5)
    assert torch.allclose(z.var(-1, unbiased=False), torch.ones(B, S), atol=1e-3)
    # the chunk order is (shift, scale, gate): a pure shift moves the mean, a pure scale does not
    only_shift = torch.cat([torch.full((B, C), 2.0), torch.zeros(B, 2 * C)], dim=1)
    assert torch.allclose(ops.ada_layer_norm(x, only_shift)[0].mean(-1), torch.full((B, S), 2.0), atol=1e-5)


def test_ada_layer_norm_index_is_a_gather():
    B, S, C = 2, 6, 16
    x = _rand(B, S, C, seed=17)
    mod = _rand(2 * B, 3 * C, seed=18)
    index = torch.tensor([[0, 1, 0, 0, 1, 1], [1, 1, 0, 1, 0, 0]])
    out, gate = ops.ada_layer_norm(x, mod, index)
    for b in range(B):
        for s in range(S):
            row = b if index[b, s] == 0 else b + B
            ref, g = ops.ada_layer_norm(x[b:b + 1, s:s + 1], mod[row:row + 1])
            assert torch.allclose(out[b, s], ref[0, 0], atol=1e-6)
            assert torch.equal(gate[b, s], g[0, 0])


def test_gated_residual_and_gelu():
    h, y = _rand(2, 3, 8, seed=19), _rand(2, 3, 8, seed=20)
    g = _rand(2, 1, 8, seed=21)
    assert torch.equal(ops.gated_residual(h, y, torch.zeros_like(g)), h)
    assert torch.allclose(ops.gated_residual(h, y, g), torch.addcmul(h, g.expand_as(y), y))
    x = torch.linspace(-6, 6, 101)
    ref = 0.5 * x * (1 + torch.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3)))
    assert torch.allclose(ops.gelu_tanh(x), ref, atol=1e-6)


# ----------------------------------------------------------------------------------- TeaCache scalar
def test_rel_l1_closed_forms():
    prev = _rand(1, 64, 32, seed=22) + 0.1
    assert ops.rel_l1(prev.clone(), prev) == 0.0
    assert abs(ops.rel_l1(1.25 * prev, prev) - 0.25) < 1e-6
    delta = 0.01
    cur = prev + delta * torch.sign(_rand(1, 64, 32, seed=23))
    assert abs(ops.rel_l1(cur, prev) - delta / prev.abs().mean().item()) < 1e-6
    # not symmetric: the denominator is the PREVIOUS tensor
    assert abs(ops.rel_l1(prev, 1.25 * prev) - 0.2) < 1e-6


def test_rel_l1_bf16_rounding_points_and_sum_form():
    prev = (_rand(1, 128, 64, seed=24) * 2).bfloat16()
    cur = (prev.float() * 1.03 + 0.01 * _rand(1, 128, 64, seed=25)).bfloat16()
    r = ops.rel_l1(cur, prev)
    # result is a bf16 value (8 significant bits) and ~ the fp32 ratio within bf16 rounding
    assert torch.tensor(r).bfloat16().item() == r
    exact = ops.rel_l1(cur.float(), prev.float())
    assert abs(r - exact) / exact < 2e-2
    # same scalar from raw sums taken with a bf16-rounded difference
    sd = (cur - prev).abs().double().sum().item()
    sp = prev.abs().double().sum().item()
    assert ops.rel_l1_from_sums(sd, sp, cur.numel(), torch.bfloat16) == r


def test_poly_horner_matches_numpy():
    from oracle.teacache import COEFFICIENTS

    for name, c in COEFFICIENTS.items():
        p = np.poly1d(c)
        for x in (0.0, 0.013, 0.07, 0.31, 1.5):
            assert math.isclose(ops.poly_horner(c, x), float(p(x)), rel_tol=1e-12, abs_tol=1e-12), name


def test_timestep_embedding_layout():
    t = torch.tensor([0.0, 0.5, 1.0])
    e = ops.timestep_embedding(t)
    assert e.shape == (3, 256)
    # flip_sin_to_cos: first half cosines, second half sines; t = 0 -> cos = 1, sin = 0
    assert torch.allclose(e[0, :128], torch.ones(128)) and torch.allclose(e[0, 128:], torch.zeros(128))
    # channel 0 has frequency 1 at scale 1000: cos(1000 t), sin(1000 t)
    assert math.isclose(e[1, 0].item(), math.cos(500.0), abs_tol=1e-4)
    assert math.isclose(e[1, 128].item(), math.sin(500.0), abs_tol=1e-4)
    # last channel has frequency max_period^(-(127/128))
    f = math.exp(-math.log(10000) * 127 / 128)
    assert math.isclose(e[2, 127].item(), math.cos(1000.0 * f), abs_tol=1e-4)
    # integer timesteps (Wan passes them raw, scale 1) keep fractional frequencies
    ei = ops.timestep_embedding(torch.tensor([500]), scale=1.0)
    assert math.isclose(ei[0, 127].item(), math.cos(500.0 * f), abs_tol=1e-4)
    # 16-bit timesteps: frequencies stay fp32 unless the in-tree variant is asked for
    tb = torch.tensor([0.3]).bfloat16()
    e32 = ops.timestep_embedding(tb)
    assert math.isclose(e32[0, 127].item(), math.cos(1000.0 * f * float(tb[0])), abs_tol=1e-4)
    ecast = ops.timestep_embedding(tb, cast_freqs=True)
    fb = float(torch.tensor(f).bfloat16())
    assert math.isclose(ecast[0, 127].item(), math.cos(1000.0 * fb * float(tb[0])), abs_tol=1e-4)
