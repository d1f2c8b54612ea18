"""Pins of the oracle's conditioning embedders and output heads: ``ops.ada_layer_norm_continuous``,
``qwen_image.head``, ``flux.head``, ``flux.time_text_embed`` (+ the x1000 of ``flux.stem``),
``wan.condition_embedder`` and ``wan.head``.

Each function is checked on parameter settings that reduce it to ONE library routine or to a closed form
written here with numpy, chosen so that a swapped chunk, a dropped branch, a missing activation or a wrong
argument order changes the answer: a zero projection weight with a bias that fills only one chunk (pure
scale on ``F.layer_norm`` / pure shift), one-hot conditioning vectors (SiLU of a single known number), all
embedders but one zeroed, timestep 0 (the sinusoid is then exactly [1..1, 0..0]) and timestep 1/1000 (the
x1000 of the stem makes the argument of the sinusoid the bare frequency table).

What these pins cannot settle is the convention itself where it lives in a third-party class that is not in
the reference tree (diffusers ``AdaLayerNormContinuous`` returns ``scale, shift`` in that order;
``CombinedTimestepGuidanceTextProjEmbeddings`` adds the three embeddings); the tests state the convention
adopted in plain sight, so that a different reading of upstream shows up as ONE failing assertion here.
"""

import math

import numpy as np
import torch
import torch.nn.functional as F

from oracle import flux as ofx
from oracle import ops
from oracle import qwen_image as oq
from oracle import wan as ow


def _rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def _sinusoid_numpy(t, dim, max_period=10000.0):
    """[cos(t f_k) ..., sin(t f_k) ...], f_k = max_period ** (-k / (dim / 2)): diffusers ``Timesteps`` with
    flip_sin_to_cos=True and downscale_freq_shift=0, in float64."""
    half = dim // 2
    f = np.exp(-math.log(max_period) * np.arange(half, dtype=np.float64) / half)
    arg = np.asarray(t, dtype=np.float64)[:, None] * f[None, :]
    return np.concatenate([np.cos(arg), np.sin(arg)], axis=1)


# ------------------------------------------------------------------ AdaLayerNormContinuous
def test_ada_layer_norm_continuous_chunks_and_activation():
    B, S, C, E = 2, 5, 8, 6
    x, cond = _rand(B, S, C, seed=1, scale=3.0) + 2.0, _rand(B, E, seed=2)
    ln = F.layer_norm(x, (C,), None, None, 1e-6)
    zero_w = torch.zeros(2 * C, E, dtype=torch.float64)
    s = _rand(C, seed=3)
    # zero weight, bias fills the FIRST chunk only: the first chunk is the scale -> LN(x) * (1 + s), no shift
    got = ops.ada_layer_norm_continuous(x, cond, zero_w, torch.cat([s, torch.zeros(C, dtype=torch.float64)]), 1e-6)
    torch.testing.assert_close(got, ln * (1 + s), rtol=1e-12, atol=1e-12)
    # bias fills the SECOND chunk only: pure shift on the plain LayerNorm
    got = ops.ada_layer_norm_continuous(x, cond, zero_w, torch.cat([torch.zeros(C, dtype=torch.float64), s]), 1e-6)
    torch.testing.assert_close(got, ln + s, rtol=1e-12, atol=1e-12)
    # no bias at all and zero weight: the plain LayerNorm (the "1 +" is there, the affine is not)
    torch.testing.assert_close(ops.ada_layer_norm_continuous(x, cond, zero_w, None, 1e-6), ln, rtol=1e-12, atol=1e-12)
    # the projection sees SiLU(cond): a one-hot conditioning vector a * e_i gives column i times a * sigmoid(a),
    # for a negative a too (where SiLU differs most from the identity, GELU and ReLU)
    w = _rand(2 * C, E, seed=4)
    for a in (-1.5, 0.7):
        cond1 = torch.zeros(B, E, dtype=torch.float64)
        cond1[:, 2] = a
        act = a * torch.sigmoid(torch.tensor(a, dtype=torch.float64))
        want = ln * (1 + w[:C, 2] * act) + w[C:, 2] * act
        torch.testing.assert_close(ops.ada_layer_norm_continuous(x, cond1, w, None, 1e-6), want, rtol=1e-12, atol=1e-12)
    # each batch row is conditioned by its own vector
    got = ops.ada_layer_norm_continuous(x, cond, w, None, 1e-6)
    for b in range(B):
        alone = ops.ada_layer_norm_continuous(x[b:b + 1], cond[b:b + 1], w, None, 1e-6)
        torch.testing.assert_close(got[b:b + 1], alone, rtol=1e-12, atol=1e-12)
    # eps is the LayerNorm's: a constant row has zero variance and normalises to exactly 0 -> output = shift
    flat = torch.full((1, 1, C), 5.0, dtype=torch.float64)
    got = ops.ada_layer_norm_continuous(flat, cond[:1], zero_w, torch.cat([s, s + 1]), 1e-6)
    torch.testing.assert_close(got, (s + 1).view(1, 1, C), rtol=0, atol=1e-12)


def _head_case(module, cfg, inner, eps):
    """Shared by the Qwen-Image and Flux heads: norm_out (continuous adaLN, no affine) then proj_out."""
    w = {k: v.double() for k, v in module.init_params(cfg, seed=3, bias_std=0.02).items()} \
        if module is oq else {k: v.double() for k, v in module.init_params(cfg, seed=3).items()}
    B, S = 2, 7
    img, temb = _rand(B, S, inner, seed=5, scale=2.0), _rand(B, inner, seed=6)
    pw, pb = w["proj_out.weight"], w.get("proj_out.bias")
    ln = F.layer_norm(img, (inner,), None, None, eps)
    s = _rand(inner, seed=7)
    z = torch.zeros(inner, dtype=torch.float64)
    w0 = dict(w)
    w0["norm_out.linear.weight"] = torch.zeros_like(w["norm_out.linear.weight"])
    # (1) modulation switched off: the head is proj_out(LayerNorm(img))
    w0["norm_out.linear.bias"] = torch.cat([z, z])
    torch.testing.assert_close(module.head(w0, cfg, img, temb), F.linear(ln, pw, pb), rtol=1e-11, atol=1e-11)
    # (2) scale chunk only / (3) shift chunk only
    w0["norm_out.linear.bias"] = torch.cat([s, z])
    torch.testing.assert_close(module.head(w0, cfg, img, temb), F.linear(ln * (1 + s), pw, pb), rtol=1e-11, atol=1e-11)
    w0["norm_out.linear.bias"] = torch.cat([z, s])
    torch.testing.assert_close(module.head(w0, cfg, img, temb), F.linear(ln + s, pw, pb), rtol=1e-11, atol=1e-11)
    # (4) the real projection of SiLU(temb), stated with library calls only
    emb = F.linear(F.silu(temb), w["norm_out.linear.weight"], w.get("norm_out.linear.bias"))
    want = F.linear(ln * (1 + emb[:, None, :inner]) + emb[:, None, inner:], pw, pb)
    torch.testing.assert_close(module.head(w, cfg, img, temb), want, rtol=1e-11, atol=1e-11)
    # (5) the head is token-local: permuting tokens permutes outputs
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(8))
    torch.testing.assert_close(module.head(w, cfg, img[:, perm], temb), module.head(w, cfg, img, temb)[:, perm],
                               rtol=1e-11, atol=1e-11)


def test_qwen_head_is_continuous_adaln_then_projection():
    cfg = oq.tiny_config()
    _head_case(oq, cfg, cfg.num_heads * cfg.head_dim, cfg.eps)


def test_flux_head_is_continuous_adaln_then_projection():
    cfg = ofx.tiny_config()
    _head_case(ofx, cfg, cfg.num_heads * cfg.head_dim, 1e-6)


def test_qwen_transformer_forward_ends_in_the_pinned_head():
    """transformer_forward's last step is exactly the head pinned above, applied to the last block's image
    stream: rebuilt here from the collected block outputs with library calls."""
    cfg = oq.tiny_config()
    w = {k: v.double() for k, v in oq.init_params(cfg, seed=0, bias_std=0.02).items()}
    lat, txt, t = _rand(1, 16, cfg.in_channels, seed=1), _rand(1, 6, cfg.joint_attention_dim, seed=2), torch.tensor([0.4], dtype=torch.float64)
    out, blocks = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 4), collect_blocks=True)
    img = blocks[-1][0]
    _, _, temb = oq.stem(w, cfg, lat, txt, t)
    inner = cfg.num_heads * cfg.head_dim
    emb = F.linear(F.silu(temb), w["norm_out.linear.weight"], w["norm_out.linear.bias"])
    ln = F.layer_norm(img, (inner,), None, None, 1e-6)
    want = F.linear(ln * (1 + emb[:, None, :inner]) + emb[:, None, inner:], w["proj_out.weight"], w["proj_out.bias"])
    torch.testing.assert_close(out, want, rtol=1e-10, atol=1e-10)


# ------------------------------------------------------------------ Flux conditioning embedding
def _flux_weights():
    cfg = ofx.tiny_config()
    return cfg, {k: v.double() for k, v in ofx.init_params(cfg, seed=11).items()}


def _zero_embedder(w, name):
    out = dict(w)
    for k in w:
        if k.startswith(f"time_text_embed.{name}."):
            out[k] = torch.zeros_like(w[k])
    return out


def _mlp(w, pre, x):
    """Linear -> SiLU -> Linear with library calls (diffusers TimestepEmbedding / PixArtAlphaTextProjection(silu))."""
    h = F.linear(x, w[pre + ".linear_1.weight"], w[pre + ".linear_1.bias"])
    return F.linear(F.silu(h), w[pre + ".linear_2.weight"], w[pre + ".linear_2.bias"])


def test_flux_time_text_embed_one_branch_at_a_time():
    cfg, w = _flux_weights()
    B = 3
    t = torch.tensor([0.0, 1.0, 517.25], dtype=torch.float64)      # as the stem hands them over: already x1000
    g = torch.tensor([3500.0, 0.0, 1000.0], dtype=torch.float64)
    pooled = _rand(B, cfg.pooled_projection_dim, seed=12)
    sin_t = torch.from_numpy(_sinusoid_numpy(t.numpy(), 256))
    sin_g = torch.from_numpy(_sinusoid_numpy(g.numpy(), 256))
    only_t = _zero_embedder(_zero_embedder(w, "guidance_embedder"), "text_embedder")
    only_g = _zero_embedder(_zero_embedder(w, "timestep_embedder"), "text_embedder")
    only_p = _zero_embedder(_zero_embedder(w, "timestep_embedder"), "guidance_embedder")
    tol = dict(rtol=1e-4, atol=5e-6)   # the oracle's sinusoid is fp32: arguments of ~500 rad carry ~3e-5 rad of rounding
    torch.testing.assert_close(ofx.time_text_embed(only_t, cfg, t, g, pooled),
                               _mlp(w, "time_text_embed.timestep_embedder", sin_t), **tol)
    torch.testing.assert_close(ofx.time_text_embed(only_g, cfg, t, g, pooled),
                               _mlp(w, "time_text_embed.guidance_embedder", sin_g), **tol)
    torch.testing.assert_close(ofx.time_text_embed(only_p, cfg, t, g, pooled),
                               _mlp(w, "time_text_embed.text_embedder", pooled), rtol=1e-12, atol=1e-12)
    # the three embeddings are ADDED; without guidance the guidance embedder is not evaluated at all
    full = ofx.time_text_embed(w, cfg, t, g, pooled)
    parts = (_mlp(w, "time_text_embed.timestep_embedder", sin_t) + _mlp(w, "time_text_embed.guidance_embedder", sin_g)
             + _mlp(w, "time_text_embed.text_embedder", pooled))
    torch.testing.assert_close(full, parts, **tol)
    no_g = ofx.time_text_embed(w, cfg, t, None, pooled)
    torch.testing.assert_close(no_g, parts - _mlp(w, "time_text_embed.guidance_embedder", sin_g), **tol)
    # timestep 0: the sinusoid is exactly [1]*128 + [0]*128 (cosines first), so linear_1 reduces to the row sums of
    # its first 128 columns plus its bias
    w1, b1 = w["time_text_embed.timestep_embedder.linear_1.weight"], w["time_text_embed.timestep_embedder.linear_1.bias"]
    h0 = w1[:, :128].sum(dim=1) + b1
    want0 = F.linear(F.silu(h0), w["time_text_embed.timestep_embedder.linear_2.weight"],
                     w["time_text_embed.timestep_embedder.linear_2.bias"])
    torch.testing.assert_close(ofx.time_text_embed(only_t, cfg, t, g, pooled)[0], want0, rtol=1e-12, atol=1e-12)


def test_flux_stem_scales_timestep_and_guidance_by_1000():
    cfg, w = _flux_weights()
    lat = _rand(1, 4, cfg.in_channels, seed=13)
    text = _rand(1, 3, cfg.joint_attention_dim, seed=14)
    pooled = _rand(1, cfg.pooled_projection_dim, seed=15)
    t, g = torch.tensor([0.001], dtype=torch.float64), torch.tensor([0.002], dtype=torch.float64)
    img, txt, temb = ofx.stem(w, cfg, lat, text, pooled, t, g)
    # 0.001 * 1000 = 1 -> the argument of the sinusoid is the bare frequency table (2 for the guidance)
    want = (_mlp(w, "time_text_embed.timestep_embedder", torch.from_numpy(_sinusoid_numpy([1.0], 256)))
            + _mlp(w, "time_text_embed.guidance_embedder", torch.from_numpy(_sinusoid_numpy([2.0], 256)))
            + _mlp(w, "time_text_embed.text_embedder", pooled))
    torch.testing.assert_close(temb, want, rtol=1e-4, atol=5e-6)
    torch.testing.assert_close(img, F.linear(lat, w["x_embedder.weight"], w["x_embedder.bias"]), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(txt, F.linear(text, w["context_embedder.weight"], w["context_embedder.bias"]),
                               rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ Wan condition embedder and head
def _wan_weights():
    cfg = ow.tiny_config()
    return cfg, {k: v.double() for k, v in ow.init_params(cfg, seed=21).items()}


def test_wan_condition_embedder_branches():
    cfg, w = _wan_weights()
    pre = "condition_embedder."
    B, L = 2, 5
    text = _rand(B, L, w[pre + "text_embedder.linear_1.weight"].shape[1], seed=22)
    t = torch.tensor([0.0, 873.5], dtype=torch.float64)
    temb, tproj, ctx = ow.condition_embedder(w, cfg, t, text)
    C = temb.shape[-1]
    assert temb.shape == (B, C) and tproj.shape == (B, 6 * C) and ctx.shape == (B, L, C)
    # time branch with library calls: sinusoid (timesteps are NOT rescaled here) -> Linear -> SiLU -> Linear
    sin = torch.from_numpy(_sinusoid_numpy(t.numpy(), cfg.freq_dim))
    want_temb = _mlp(w, pre + "time_embedder", sin)
    torch.testing.assert_close(temb, want_temb, rtol=1e-4, atol=5e-6)
    # timestep 0 -> [1..1, 0..0]: the first linear reduces to row sums of its first half of columns
    w1, b1 = w[pre + "time_embedder.linear_1.weight"], w[pre + "time_embedder.linear_1.bias"]
    h0 = w1[:, : cfg.freq_dim // 2].sum(dim=1) + b1
    want0 = F.linear(F.silu(h0), w[pre + "time_embedder.linear_2.weight"], w[pre + "time_embedder.linear_2.bias"])
    torch.testing.assert_close(temb[0], want0, rtol=1e-12, atol=1e-12)
    # the six modulation rows come from SiLU(temb), not from temb and not from the sinusoid: make temb a known
    # constant vector (zero last weight, bias b) and compare with Linear(SiLU(b))
    b = _rand(C, seed=23)
    wz = dict(w)
    wz[pre + "time_embedder.linear_2.weight"] = torch.zeros_like(w[pre + "time_embedder.linear_2.weight"])
    wz[pre + "time_embedder.linear_2.bias"] = b
    temb_b, tproj_b, _ = ow.condition_embedder(wz, cfg, t, text)
    torch.testing.assert_close(temb_b, b.expand(B, C), rtol=0, atol=0)
    torch.testing.assert_close(tproj_b, F.linear(F.silu(b), w[pre + "time_proj.weight"], w[pre + "time_proj.bias"]).expand(B, 6 * C),
                               rtol=1e-12, atol=1e-12)
    # text branch: Linear -> GELU(tanh) -> Linear, token-local and independent of the timestep; the activation
    # is the tanh form written out here, which differs from the erf form by up to 5e-4
    h = F.linear(text, w[pre + "text_embedder.linear_1.weight"], w[pre + "text_embedder.linear_1.bias"])
    act = 0.5 * h * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (h + 0.044715 * h ** 3)))
    want_ctx = F.linear(act, w[pre + "text_embedder.linear_2.weight"], w[pre + "text_embedder.linear_2.bias"])
    torch.testing.assert_close(ctx, want_ctx, rtol=1e-12, atol=1e-12)
    assert (F.gelu(h * 30) - 0.5 * (h * 30) * (1 + torch.tanh(math.sqrt(2 / math.pi) * (h * 30 + 0.044715 * (h * 30) ** 3)))).abs().max() > 1e-5
    _, _, ctx2 = ow.condition_embedder(w, cfg, t + 5.0, text)
    assert torch.equal(ctx, ctx2)
    # per-token timesteps [B*S] with timestep_seq_len: the same embedding per token, reshaped to [B,S,...]
    S = 3
    tt = torch.tensor([0.0, 10.0, 20.0, 30.0, 40.0, 873.5], dtype=torch.float64)
    temb_s, tproj_s, _ = ow.condition_embedder(w, cfg, tt, text, timestep_seq_len=S)
    assert temb_s.shape == (B, S, C) and tproj_s.shape == (B, S, 6 * C)
    torch.testing.assert_close(temb_s[0, 0], temb[0], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(temb_s[1, 2], temb[1], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(tproj_s[1, 2], tproj[1], rtol=1e-12, atol=1e-12)


def test_wan_head_shift_then_scale_of_table_plus_temb():
    cfg, w = _wan_weights()
    B, grid = 2, (2, 2, 3)
    S = grid[0] * grid[1] * grid[2]
    C = w["output_scale_shift_prepare.scale_shift_table"].shape[-1]
    x, temb = _rand(B, S, C, seed=24, scale=2.0), _rand(B, C, seed=25)
    table = w["output_scale_shift_prepare.scale_shift_table"].reshape(2, C)
    ln = F.layer_norm(x, (C,), None, None, cfg.eps)
    pw, pb = w["proj_out.weight"], w["proj_out.bias"]

    def tokens(out):  # undo the unpatchify: [B, C_out, F, H, W] -> [B, S, p_t*p_h*p_w*C_out] in proj_out's layout
        p_t, p_h, p_w = cfg.patch_size
        f, h, ww = grid
        o = out.reshape(B, -1, f, p_t, h, p_h, ww, p_w).permute(0, 2, 4, 6, 3, 5, 7, 1)
        return o.reshape(B, S, -1)

    # row 0 of the table (+ temb) is the SHIFT, row 1 the SCALE: zero one of them at a time, temb = 0
    z = torch.zeros(B, C, dtype=torch.float64)
    w_shift = dict(w)
    w_shift["output_scale_shift_prepare.scale_shift_table"] = torch.stack([table[0], torch.zeros(C, dtype=torch.float64)]).reshape_as(
        w["output_scale_shift_prepare.scale_shift_table"])
    torch.testing.assert_close(tokens(ow.head(w_shift, cfg, x, z, grid, B)), F.linear(ln + table[0], pw, pb), rtol=1e-6, atol=1e-7)
    w_scale = dict(w)
    w_scale["output_scale_shift_prepare.scale_shift_table"] = torch.stack([torch.zeros(C, dtype=torch.float64), table[1]]).reshape_as(
        w["output_scale_shift_prepare.scale_shift_table"])
    torch.testing.assert_close(tokens(ow.head(w_scale, cfg, x, z, grid, B)), F.linear(ln * (1 + table[1]), pw, pb), rtol=1e-6, atol=1e-7)
    # temb is added to BOTH rows
    want = F.linear(ln * (1 + table[1] + temb[:, None]) + table[0] + temb[:, None], pw, pb)
    torch.testing.assert_close(tokens(ow.head(w, cfg, x, temb, grid, B)), want, rtol=1e-6, atol=1e-7)
    # per-token temb [B,S,C] with every token equal reduces to the per-batch form
    torch.testing.assert_close(ow.head(w, cfg, x, temb[:, None].expand(B, S, C).contiguous(), grid, B),
                               ow.head(w, cfg, x, temb, grid, B), rtol=1e-12, atol=1e-12)


def test_rms_norm_head_cast_order_is_the_one_the_reference_tree_writes_out():
    """vLLM's RMSNorm is absent from the reference tree, but the tree writes the same layer out for another
    model (model_executor/models/qwen3_tts/modeling_qwen3_tts.py:590-598): normalise in float32, cast to the
    input dtype, THEN multiply by the weight. Wan's DistributedRMSNorm (wan2_2_transformer.py:70-89) multiplies
    in float32 and casts last; on bf16 inputs the two orders round differently, and the per-head norm must be
    the first, the whole-row norm the second."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 7, 128, generator=g).to(torch.bfloat16)
    w = (1 + 0.3 * torch.randn(128, generator=g)).to(torch.bfloat16)
    normed = x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)
    cast_then_weight = w * normed.to(torch.bfloat16)
    weight_then_cast = (normed * w.float()).to(torch.bfloat16)
    assert not torch.equal(cast_then_weight, weight_then_cast), "the input does not tell the two orders apart"
    assert torch.equal(ops.rms_norm_head(x, w), cast_then_weight)
    assert torch.equal(ops.rms_norm_row_fp32(x, w.float()).to(torch.bfloat16), weight_then_cast)
