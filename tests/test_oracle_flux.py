"""Pins for the Flux oracle that do not retype its formulas: library routines, invariances that the
architecture implies (token-permutation equivariance with ids carried along, zero gates = identity,
translation of the image grid), fp32-vs-fp64 agreement, and linearity of the split projection the
product uses in place of the channel concatenation."""

import numpy as np
import torch

from oracle import flux as ofx
from oracle import ops


def _setup(seed=0, B=1, grid=(4, 5), n_txt=6, dtype=torch.float64, bias_std=0.05):
    cfg = ofx.tiny_config()
    w = ofx.init_params(cfg, seed=seed, dtype=dtype, bias_std=bias_std, std=0.05)
    g = torch.Generator().manual_seed(seed + 1)
    lat = torch.randn(B, grid[0] * grid[1], cfg.in_channels, generator=g, dtype=dtype)
    txt = torch.randn(B, n_txt, cfg.joint_attention_dim, generator=g, dtype=dtype)
    pooled = torch.randn(B, cfg.pooled_projection_dim, generator=g, dtype=dtype)
    t = torch.rand(B, generator=g, dtype=dtype)
    gd = torch.full((B,), 3.5, dtype=dtype)
    return cfg, w, lat, txt, pooled, t, gd, ofx.latent_image_ids(*grid), torch.zeros(n_txt, 3)


def test_pos_embed_against_numpy_and_identity_on_text_rows():
    cfg = ofx.tiny_config()
    ids = torch.cat([torch.zeros(5, 3), ofx.latent_image_ids(3, 4)], dim=0)
    cos, sin = ofx.flux_pos_embed(cfg, ids)
    assert cos.dtype == torch.float64 and cos.shape == (17, sum(cfg.axes_dims_rope) // 2)
    assert torch.all(cos[:5] == 1) and torch.all(sin[:5] == 0)
    # independent statement: complex exponentials per axis with numpy
    col = 0
    for a, d in enumerate(cfg.axes_dims_rope):
        inv = 1.0 / np.power(float(cfg.theta), np.arange(0, d, 2, dtype=np.float64) / d)
        z = np.exp(1j * np.outer(ids[:, a].numpy().astype(np.float64), inv))
        np.testing.assert_allclose(cos[:, col:col + d // 2].numpy(), z.real, atol=1e-14)
        np.testing.assert_allclose(sin[:, col:col + d // 2].numpy(), z.imag, atol=1e-14)
        col += d // 2
    # ids are (0, y, x): row-major over the grid
    assert ofx.latent_image_ids(3, 4)[1 * 4 + 2].tolist() == [0.0, 1.0, 2.0]


def test_rotary_scores_depend_on_grid_offsets_only():
    """<rope(q, p), rope(k, p')> depends on p - p' only, so translating the whole image grid changes
    no image-image score."""
    cfg = ofx.tiny_config()
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, 12, 1, cfg.head_dim, generator=g, dtype=torch.float64)
    k = torch.randn(1, 12, 1, cfg.head_dim, generator=g, dtype=torch.float64)
    ids = ofx.latent_image_ids(3, 4)
    c0, s0 = ofx.flux_pos_embed(cfg, ids)
    c1, s1 = ofx.flux_pos_embed(cfg, ids + torch.tensor([0.0, 7.0, 3.0]))
    sc0 = torch.einsum("bqhd,bkhd->bqk", ops.apply_rotary(q, c0, s0), ops.apply_rotary(k, c0, s0))
    sc1 = torch.einsum("bqhd,bkhd->bqk", ops.apply_rotary(q, c1, s1), ops.apply_rotary(k, c1, s1))
    torch.testing.assert_close(sc0, sc1, atol=1e-10, rtol=0)


def test_token_permutation_equivariance():
    """Permuting image tokens together with their ids permutes the image outputs; permuting text
    tokens (all ids zero) leaves the image outputs unchanged. A mix-up of the two streams in the joint
    sequence, of the id order, or of the split after attention breaks this."""
    cfg, w, lat, txt, pooled, t, gd, img_ids, txt_ids = _setup()
    base = ofx.transformer_forward(w, cfg, lat, txt, pooled, t, img_ids, txt_ids, guidance=gd)
    g = torch.Generator().manual_seed(9)
    pi = torch.randperm(lat.shape[1], generator=g)
    pt = torch.randperm(txt.shape[1], generator=g)
    out_i = ofx.transformer_forward(w, cfg, lat[:, pi], txt, pooled, t, img_ids[pi], txt_ids, guidance=gd)
    torch.testing.assert_close(out_i, base[:, pi], atol=2e-6, rtol=0)  # softmax and RMS statistics are fp32
    out_t = ofx.transformer_forward(w, cfg, lat, txt[:, pt], pooled, t, img_ids, txt_ids, guidance=gd)
    torch.testing.assert_close(out_t, base, atol=2e-6, rtol=0)
    # ...but permuting image tokens WITHOUT their ids is a different input
    out_bad = ofx.transformer_forward(w, cfg, lat[:, pi], txt, pooled, t, img_ids, txt_ids, guidance=gd)
    assert (out_bad - base[:, pi]).abs().max() > 1e-3


def test_zero_modulation_projections_make_every_block_the_identity():
    """With the AdaLayerNormZero(-Single) projections zeroed, every gate is 0: both streams pass
    through all blocks unchanged whatever the other weights are."""
    cfg, w, lat, txt, pooled, t, gd, img_ids, txt_ids = _setup(seed=2)
    w = dict(w)
    for k in list(w):
        if ".norm1.linear." in k or ".norm1_context.linear." in k or ".norm.linear." in k:
            w[k] = torch.zeros_like(w[k])
    img, enc, temb = ofx.stem(w, cfg, lat, txt, pooled, t, gd)
    cos, sin = ofx.flux_pos_embed(cfg, torch.cat((txt_ids, img_ids), dim=0))
    e, h = ofx.dual_block_forward(w, 0, cfg, img, enc, temb, cos, sin)
    assert torch.equal(h, img) and torch.equal(e, enc)
    e, h = ofx.single_block_forward(w, 0, cfg, img, enc, temb, cos, sin)
    assert torch.equal(h, img) and torch.equal(e, enc)


def test_gate_chunks_select_the_right_branch():
    """Bias-only modulation (weights zero): opening ONLY gate_msa (3rd of 6 chunks) must give
    img + attention output, opening ONLY gate_mlp (6th) img + feed-forward of LN(img)."""
    cfg, w, lat, txt, pooled, t, gd, img_ids, txt_ids = _setup(seed=4)
    C = cfg.dim
    img, enc, temb = ofx.stem(w, cfg, lat, txt, pooled, t, gd)
    cos, sin = ofx.flux_pos_embed(cfg, torch.cat((txt_ids, img_ids), dim=0))

    def run(open_chunk):
        ww = dict(w)
        for name in ("norm1", "norm1_context"):
            ww[f"transformer_blocks.0.{name}.linear.weight"] = torch.zeros(6 * C, C, dtype=img.dtype)
            b = torch.zeros(6 * C, dtype=img.dtype)
            if name == "norm1":
                b[open_chunk * C:(open_chunk + 1) * C] = 1.0
            ww[f"transformer_blocks.0.{name}.linear.bias"] = b
        return ofx.dual_block_forward(ww, 0, cfg, img, enc, temb, cos, sin)

    ln = torch.nn.functional.layer_norm
    e, h = run(2)
    a_img, _ = ofx.attention_forward(w, "transformer_blocks.0.attn.", cfg, ln(img, (C,), eps=1e-6),
                                     ln(enc, (C,), eps=1e-6), cos, sin)
    torch.testing.assert_close(h, img + a_img, atol=2e-6, rtol=0)
    assert torch.equal(e, enc)
    e, h = run(5)
    torch.testing.assert_close(h, img + ofx.feed_forward(w, "transformer_blocks.0.ff.", ln(img, (C,), eps=1e-6)),
                               atol=1e-10, rtol=0)
    assert torch.equal(e, enc)


def test_fp32_agrees_with_fp64():
    cfg, w, lat, txt, pooled, t, gd, img_ids, txt_ids = _setup(seed=6, B=2)
    want = ofx.transformer_forward(w, cfg, lat, txt, pooled, t, img_ids, txt_ids, guidance=gd)
    w32 = {k: v.float() for k, v in w.items()}
    got = ofx.transformer_forward(w32, cfg, lat.float(), txt.float(), pooled.float(), t.float(), img_ids, txt_ids,
                                  guidance=gd.float())
    torch.testing.assert_close(got.double(), want, atol=2e-4, rtol=1e-3)


def test_split_projection_equals_projection_of_concatenation():
    """proj_out(cat([a, m], -1)) == a Wa^T + m Wm^T + b with Wa, Wm the column ranges of the weight."""
    g = torch.Generator().manual_seed(1)
    a = torch.randn(3, 7, 16, generator=g, dtype=torch.float64)
    m = torch.randn(3, 7, 64, generator=g, dtype=torch.float64)
    W = torch.randn(16, 80, generator=g, dtype=torch.float64)
    b = torch.randn(16, generator=g, dtype=torch.float64)
    want = torch.nn.functional.linear(torch.cat([a, m], dim=-1), W, b)
    got = torch.nn.functional.linear(m, W[:, 16:], b) + a @ W[:, :16].t()
    torch.testing.assert_close(got, want, atol=1e-12, rtol=0)


def test_shift_and_scale_chunks_sit_where_the_reference_tree_writes_them():
    """The remaining four of AdaLayerNormZero's six chunks. The reference tree writes the layer out at
    model_executor/models/qwen3_tts/tokenizer_25hz/modeling_qwen3_tts_tokenizer_v1.py:473-488:
    chunk(6) = shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp with
    x = LN(x) * (1 + scale_msa) + shift_msa. Bias-only modulation, one chunk at a time:
    chunk 0 must SHIFT the attention input (seen in the TeaCache decision tensor), chunk 1 must SCALE it;
    with gate_mlp open, chunk 3 must shift and chunk 4 scale the feed-forward input."""
    cfg, w, lat, txt, pooled, t, gd, img_ids, txt_ids = _setup(seed=6)
    C = cfg.dim
    img, enc, temb = ofx.stem(w, cfg, lat, txt, pooled, t, gd)
    cos, sin = ofx.flux_pos_embed(cfg, torch.cat((txt_ids, img_ids), dim=0))
    ln = torch.nn.functional.layer_norm(img, (C,), eps=1e-6)
    val = torch.linspace(0.25, 0.75, C, dtype=img.dtype)

    def weights(chunks: dict):
        ww = dict(w)
        for name in ("norm1", "norm1_context"):
            ww[f"transformer_blocks.0.{name}.linear.weight"] = torch.zeros(6 * C, C, dtype=img.dtype)
            b = torch.zeros(6 * C, dtype=img.dtype)
            if name == "norm1":
                for ch, v in chunks.items():
                    b[ch * C:(ch + 1) * C] = v
            ww[f"transformer_blocks.0.{name}.linear.bias"] = b
        return ww

    torch.testing.assert_close(ofx.modulated_input(weights({0: val}), cfg, img, temb), ln + val, atol=1e-12, rtol=0)
    torch.testing.assert_close(ofx.modulated_input(weights({1: val}), cfg, img, temb), ln * (1 + val), atol=1e-12, rtol=0)
    ff = lambda x: ofx.feed_forward(w, "transformer_blocks.0.ff.", x)  # noqa: E731
    _, h = ofx.dual_block_forward(weights({5: 1.0, 3: val}), 0, cfg, img, enc, temb, cos, sin)
    torch.testing.assert_close(h, img + ff(ln + val), atol=1e-10, rtol=0)
    _, h = ofx.dual_block_forward(weights({5: 1.0, 4: val}), 0, cfg, img, enc, temb, cos, sin)
    torch.testing.assert_close(h, img + ff(ln * (1 + val)), atol=1e-10, rtol=0)
