"""Pins for the Wan oracle that do not retype its formulas: a library routine for the patch embedding
and its inverse, invariances of the architecture (token permutation with the rotary tables carried
along, text-token permutation, zero gates), the relative-position property of the 3D rotary tables,
and fp32-vs-fp64 agreement."""

import torch

from oracle import ops
from oracle import wan as ow


def _setup(seed=0, B=1, fhw=(2, 4, 6), n_txt=5, dtype=torch.float64):
    cfg = ow.tiny_config()
    w = {k: v.to(dtype) for k, v in ow.init_params(cfg, seed=seed, std=0.05, bias_std=0.05, norm_jitter=0.1).items()}
    g = torch.Generator().manual_seed(seed + 1)
    video = torch.randn(B, cfg.in_channels, *fhw, generator=g, dtype=dtype)
    text = torch.randn(B, n_txt, cfg.text_dim, generator=g, dtype=dtype)
    t = torch.tensor([417.0, 902.0][:B], dtype=dtype)
    return cfg, w, video, text, t


def test_rope_table_layout_and_relative_position():
    cfg = ow.tiny_config()
    D = cfg.head_dim
    cos, sin = ow.wan_rope_tables(cfg, 3, 4, 5)
    assert cos.shape == (1, 60, 1, D) and cos.dtype == torch.float32
    # each value appears twice along D; widths per axis are (D - 4*(D//6), 2*(D//6), 2*(D//6))
    assert torch.equal(cos[..., 0::2], cos[..., 1::2]) and torch.equal(sin[..., 0::2], sin[..., 1::2])
    wt = D - 4 * (D // 6)
    tok = lambda f, h, w: (f * 4 + h) * 5 + w  # noqa: E731
    # the frame slice depends on f only, the height slice on h only, the width slice on w only
    assert torch.equal(cos[0, tok(1, 0, 0), 0, :wt], cos[0, tok(1, 3, 4), 0, :wt])
    assert torch.equal(cos[0, tok(0, 2, 0), 0, wt:wt + 2 * (D // 6)], cos[0, tok(2, 2, 3), 0, wt:wt + 2 * (D // 6)])
    assert torch.equal(cos[0, tok(0, 0, 3), 0, wt + 2 * (D // 6):], cos[0, tok(2, 1, 3), 0, wt + 2 * (D // 6):])
    assert torch.all(cos[0, 0] == 1) and torch.all(sin[0, 0] == 0)
    # scores depend on grid offsets only: compare pairs with equal (df, dh, dw)
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 1, D, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 1, D, generator=g, dtype=torch.float64)

    def score(a, b):
        qa = ops.apply_rotary_wan(q, cos[:, a:a + 1].double(), sin[:, a:a + 1].double())
        kb = ops.apply_rotary_wan(k, cos[:, b:b + 1].double(), sin[:, b:b + 1].double())
        return (qa * kb).sum()

    torch.testing.assert_close(score(tok(0, 1, 1), tok(1, 3, 2)), score(tok(1, 0, 2), tok(2, 2, 3)), atol=1e-6, rtol=0)
    assert abs(score(tok(0, 1, 1), tok(1, 3, 2)) - score(tok(0, 1, 1), tok(1, 3, 3))) > 1e-4


def test_patch_embedding_is_a_linear_over_patches():
    """The stem's Conv3d (library routine) equals gathering each (C_in, 1, 2, 2) patch into a row and
    multiplying by the flattened kernel — the form the product uses."""
    cfg, w, video, text, t = _setup(B=2)
    x, _, _, _ = ow.stem(w, cfg, video, t, text)
    B, Cin, nf, hh, ww = video.shape
    rows = video.view(B, Cin, nf, 1, hh // 2, 2, ww // 2, 2).permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(B, -1, Cin * 4)
    want = rows @ w["patch_embedding.weight"].view(cfg.dim, -1).t() + w["patch_embedding.bias"]
    torch.testing.assert_close(x, want, atol=1e-12, rtol=0)


def test_unpatchify_inverts_patchify_layout():
    """head() with an identity-like projection puts token (f,h,w)'s (p_t,p_h,p_w,c) block back at
    video[c, f*p_t.., h*p_h.., w*p_w..]."""
    cfg = ow.tiny_config()
    grid, B = (2, 3, 4), 1
    n_out = cfg.out_channels * 4
    w = {"output_scale_shift_prepare.scale_shift_table": torch.zeros(1, 2, cfg.dim, dtype=torch.float64),
         "proj_out.weight": torch.zeros(n_out, cfg.dim, dtype=torch.float64),
         "proj_out.bias": torch.zeros(n_out, dtype=torch.float64)}
    w["proj_out.weight"][:, :n_out] = torch.eye(n_out, dtype=torch.float64)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(B, 24, cfg.dim, generator=g, dtype=torch.float64)
    out = ow.head(w, cfg, x, torch.zeros(B, cfg.dim, dtype=torch.float64), grid, B)
    assert out.shape == (B, cfg.out_channels, 2, 6, 8)
    xn = torch.nn.functional.layer_norm(x, (cfg.dim,), eps=cfg.eps)
    f, h, ww_, ph, pw, c = 1, 2, 3, 1, 0, 5
    tok = (f * 3 + h) * 4 + ww_
    # projection output channel order is (p_t, p_h, p_w, c)
    assert torch.isclose(out[0, c, f, h * 2 + ph, ww_ * 2 + pw], xn[0, tok, (ph * 2 + pw) * cfg.out_channels + c])


def test_token_permutation_equivariance_of_a_block():
    cfg, w, video, text, t = _setup(seed=3)
    x, temb, temb6, ctx = ow.stem(w, cfg, video, t, text)
    cos, sin = ow.wan_rope_tables(cfg, 2, 2, 3)
    base = ow.block_forward(w, 0, cfg, x, ctx, temb6, cos, sin)
    g = torch.Generator().manual_seed(5)
    p = torch.randperm(x.shape[1], generator=g)
    pt = torch.randperm(ctx.shape[1], generator=g)
    out = ow.block_forward(w, 0, cfg, x[:, p], ctx, temb6, cos[:, p], sin[:, p])
    torch.testing.assert_close(out, base[:, p], atol=2e-6, rtol=0)
    out_t = ow.block_forward(w, 0, cfg, x, ctx[:, pt], temb6, cos, sin)
    torch.testing.assert_close(out_t, base, atol=2e-6, rtol=0)
    out_bad = ow.block_forward(w, 0, cfg, x[:, p], ctx, temb6, cos, sin)
    assert (out_bad - base[:, p]).abs().max() > 1e-3


def test_gates_and_plain_cross_attention_residual():
    """table + temb = 0 closes both gates: what is left is exactly x + cross_attention(norm2(x)) —
    the cross-attention residual carries no gate."""
    cfg, w, video, text, t = _setup(seed=4)
    x, temb, temb6, ctx = ow.stem(w, cfg, video, t, text)
    cos, sin = ow.wan_rope_tables(cfg, 2, 2, 3)
    w = dict(w)
    w["blocks.0.scale_shift_table"] = -temb6[:1].clone()
    out = ow.block_forward(w, 0, cfg, x, ctx, temb6[:1], cos, sin)
    n = torch.nn.functional.layer_norm(x, (cfg.dim,), w["blocks.0.norm2.weight"], w["blocks.0.norm2.bias"], cfg.eps)
    want = x + ow.cross_attention(w, "blocks.0.attn2.", cfg, n, ctx)
    torch.testing.assert_close(out, want, atol=2e-6, rtol=0)  # the block's LayerNorms are fp32
    # opening only the self-attention gate (3rd of the 6 rows) adds attn1 of the unmodulated LayerNorm
    tbl = -temb6[:1].clone()
    tbl[:, 2] += 1.0
    w["blocks.0.scale_shift_table"] = tbl
    out = ow.block_forward(w, 0, cfg, x, ctx, temb6[:1], cos, sin)
    x1 = x + ow.self_attention(w, "blocks.0.attn1.", cfg, torch.nn.functional.layer_norm(x, (cfg.dim,), eps=cfg.eps),
                               cos, sin)
    n = torch.nn.functional.layer_norm(x1, (cfg.dim,), w["blocks.0.norm2.weight"], w["blocks.0.norm2.bias"], cfg.eps)
    torch.testing.assert_close(out, x1 + ow.cross_attention(w, "blocks.0.attn2.", cfg, n, ctx), atol=2e-6, rtol=0)


def test_fp32_agrees_with_fp64():
    cfg, w, video, text, t = _setup(seed=6, B=2)
    want = ow.transformer_forward(w, cfg, video, t, text)
    w32 = {k: v.float() for k, v in w.items()}
    got = ow.transformer_forward(w32, cfg, video.float(), t.float(), text.float())
    assert got.shape == video.shape
    torch.testing.assert_close(got.double(), want, atol=5e-4, rtol=1e-3)


# ---------------------------------------------------------------------- per-token timesteps (TI2V)
def test_per_token_timesteps_all_equal_reduce_to_the_scalar_form():
    cfg, w, video, text, t = _setup(B=2)
    S = 2 * 2 * 3
    want = ow.transformer_forward(w, cfg, video, t, text)
    got = ow.transformer_forward(w, cfg, video, t[:, None].expand(2, S).contiguous(), text)
    torch.testing.assert_close(got, want, atol=1e-12, rtol=0)


def test_per_token_timesteps_are_token_local_when_attention_is_cut():
    """Self- and cross-attention output projections zeroed: every token is processed on its own, so with
    two timestep values spread over the tokens each token must come out as in the scalar-timestep run
    with its own value - through both modulations, both gates and the head."""
    cfg, w, video, text, _ = _setup(B=1)
    w = dict(w)
    for i in range(cfg.num_layers):
        for a in ("attn1", "attn2"):
            for kind in ("weight", "bias"):
                w[f"blocks.{i}.{a}.to_out.{kind}"] = torch.zeros_like(w[f"blocks.{i}.{a}.to_out.{kind}"])
    S = 12
    ta, tb = 130.0, 860.0
    pick = torch.tensor([0, 1, 1, 0, 0, 0, 1, 0, 1, 1, 0, 1], dtype=torch.bool)
    ts = torch.where(pick, torch.tensor(tb), torch.tensor(ta)).to(video.dtype)[None]
    mixed = ow.transformer_forward(w, cfg, video, ts, text)
    out_a = ow.transformer_forward(w, cfg, video, torch.tensor([ta], dtype=video.dtype), text)
    out_b = ow.transformer_forward(w, cfg, video, torch.tensor([tb], dtype=video.dtype), text)
    # token (f, h, w) of the 2x2x3 patch grid owns output pixels [:, :, f, 2h:2h+2, 2w:2w+2]
    for tok in range(S):
        f, h, x = tok // 6, (tok % 6) // 3, tok % 3
        sl = (slice(None), slice(None), slice(f, f + 1), slice(2 * h, 2 * h + 2), slice(2 * x, 2 * x + 2))
        torch.testing.assert_close(mixed[sl], (out_b if pick[tok] else out_a)[sl], atol=1e-12, rtol=0)
    assert (out_a - out_b).abs().max().item() > 1e-3


# ---------------------------------------------------------------------- image conditioning (I2V)
def _i2v_setup(seed=0, B=1, n_img=7, n_txt=5, pos=False):
    import dataclasses

    cfg = dataclasses.replace(ow.tiny_config(), image_dim=48, added_kv_proj_dim=256, text_context_len=n_txt,
                              pos_embed_seq_len=2 * n_img if pos else None)
    w = {k: v.double() for k, v in ow.init_params(cfg, seed=seed, std=0.05, bias_std=0.05, norm_jitter=0.1).items()}
    g = torch.Generator().manual_seed(seed + 1)
    video = torch.randn(B, cfg.in_channels, 2, 4, 6, generator=g, dtype=torch.float64)
    text = torch.randn(B, n_txt, cfg.text_dim, generator=g, dtype=torch.float64)
    feats = torch.randn(2 * B if pos else B, n_img, cfg.image_dim, generator=g, dtype=torch.float64)
    t = torch.tensor([417.0, 902.0][:B], dtype=torch.float64)
    return cfg, w, video, text, feats, t


def test_image_embedder_against_library_modules():
    cfg, w, _, _, feats, _ = _i2v_setup()
    p = "condition_embedder.image_embedder."
    n1, n2 = torch.nn.LayerNorm(48).double(), torch.nn.LayerNorm(256).double()
    l1, l2 = torch.nn.Linear(48, 48).double(), torch.nn.Linear(48, 256).double()
    with torch.no_grad():
        for m, name in ((n1, "norm1"), (n2, "norm2"), (l1, "ff.net.0.proj"), (l2, "ff.net.2")):
            m.weight.copy_(w[p + name + ".weight"])
            m.bias.copy_(w[p + name + ".bias"])
        want = n2(l2(torch.nn.GELU()(l1(n1(feats)))))
    torch.testing.assert_close(ow.image_embedder(w, cfg, feats), want, atol=1e-6, rtol=0)  # norms run in fp32
    # learned positions: rows of two consecutive entries are joined before the positions are added
    cfg2, w2, _, _, feats2, _ = _i2v_setup(pos=True)
    joined = ow.image_embedder(w2, cfg2, feats2)
    assert joined.shape == (1, 14, 256)
    w3 = dict(w2)
    pe = w3.pop(p + "pos_embed")
    shifted = torch.cat([feats2[0], feats2[1]], dim=0)[None] + pe
    torch.testing.assert_close(joined, ow.image_embedder(w3, cfg2, shifted), atol=1e-12, rtol=0)


def test_image_branch_is_a_second_softmax_added_to_the_text_attention():
    """A dead image value projection must give the text-only model (pins the split point of the context
    and that the two attentions are added, not merged into one softmax); permuting the image tokens must
    change nothing; and doubling the image branch's contribution by duplicating every image token must
    change nothing either (a separate softmax is invariant to key duplication, a plain sum is not)."""
    cfg, w, video, text, feats, t = _i2v_setup()
    import dataclasses

    base = ow.transformer_forward(w, cfg, video, t, text, image_feats=feats)
    dead = dict(w)
    for i in range(cfg.num_layers):
        for kind in ("weight", "bias"):
            dead[f"blocks.{i}.attn2.add_v_proj.{kind}"] = torch.zeros_like(w[f"blocks.{i}.attn2.add_v_proj.{kind}"])
    text_only_cfg = dataclasses.replace(cfg, image_dim=None, added_kv_proj_dim=None)
    torch.testing.assert_close(ow.transformer_forward(dead, cfg, video, t, text, image_feats=feats),
                               ow.transformer_forward(w, text_only_cfg, video, t, text), atol=1e-12, rtol=0)
    assert (base - ow.transformer_forward(w, text_only_cfg, video, t, text)).abs().max().item() > 1e-4
    perm = torch.randperm(feats.shape[1], generator=torch.Generator().manual_seed(3))
    torch.testing.assert_close(ow.transformer_forward(w, cfg, video, t, text, image_feats=feats[:, perm]), base,
                               atol=2e-6, rtol=0)  # softmax and RMS statistics are fp32 inside the oracle
    twice = torch.cat([feats, feats], dim=1)
    torch.testing.assert_close(ow.transformer_forward(w, cfg, video, t, text, image_feats=twice), base,
                               atol=2e-6, rtol=0)
    # a text token moved into the image slice would break the count: the context is [image; text]
    x, temb, temb6, ctx = ow.stem(w, cfg, video, t, text, feats)
    assert ctx.shape[1] == feats.shape[1] + text.shape[1]
    torch.testing.assert_close(ctx[:, :feats.shape[1]], ow.image_embedder(w, cfg, feats), atol=0, rtol=0)
