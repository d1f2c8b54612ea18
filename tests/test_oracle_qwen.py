"""Pins for the Qwen-Image oracle that do not retype its formulas: rotary tables against numpy complex
exponentials at independently stated positions, invariances the architecture implies (masked text keys =
deleted text keys, batch rows independent, closed gates = identity, one open gate = that branch only),
fp32-vs-fp64 agreement, and for the editing variant (``zero_cond_t``) the cases that reduce to the plain
model plus the token-locality of the per-token conditioning."""

import numpy as np
import torch
import torch.nn.functional as F

from oracle import ops
from oracle import qwen_image as oq


def _setup(seed=0, B=2, grid=(1, 4, 6), n_txt=7, dtype=torch.float64, bias_std=0.05, std=0.05):
    cfg = oq.tiny_config()
    w = oq.init_params(cfg, seed=seed, dtype=dtype, bias_std=bias_std, std=std)
    g = torch.Generator().manual_seed(seed + 1)
    n = grid[0] * grid[1] * grid[2]
    lat = torch.randn(B, n, cfg.in_channels, generator=g, dtype=dtype)
    txt = torch.randn(B, n_txt, cfg.joint_attention_dim, generator=g, dtype=dtype)
    t = torch.rand(B, generator=g, dtype=dtype)
    return cfg, w, lat, txt, t


def _expected_tables(cfg, shapes, txt_len, layer3d=False):
    """Positions stated directly: image idx has frames idx.., rows y - ceil(h/2), columns x - ceil(w/2);
    text token j sits at max over images of max(h//2, w//2), plus j, on all three axes. Layered variant:
    the last image sits at frame -1 and the text start is at least the number of layers."""
    rows = []
    for idx, (f, h, w) in enumerate(shapes):
        first = -1 if layer3d and idx == len(shapes) - 1 else idx
        for t in range(f):
            for y in range(h):
                for x in range(w):
                    rows.append((first + t, y - (h + 1) // 2, x - (w + 1) // 2))
    start = max(max(h // 2, w // 2) for _, h, w in shapes)
    if layer3d:
        start = max(start, len(shapes) - 1)
    txt_rows = [(start + j,) * 3 for j in range(txt_len)]

    def table(pos_rows):
        cols = []
        for a, d in enumerate(cfg.axes_dims_rope):
            inv = 1.0 / np.power(float(cfg.theta), np.arange(0, d, 2, dtype=np.float64) / d)
            cols.append(np.exp(1j * np.outer(np.array([r[a] for r in pos_rows], dtype=np.float64), inv)))
        return np.concatenate(cols, axis=1)

    return table(rows), table(txt_rows)


def test_rotary_tables_against_numpy_positions():
    cfg = oq.tiny_config()
    for shapes in ([(1, 4, 6)], [(1, 5, 3)], [(1, 4, 4), (1, 6, 2), (2, 3, 5)]):
        vid, txt = oq.qwen_rope_freqs_images(cfg, shapes, txt_len=5)
        want_v, want_t = _expected_tables(cfg, shapes, 5)
        assert vid.shape == want_v.shape and txt.shape == want_t.shape and vid.dtype == torch.complex64
        # fp32 angles up to ~6 rad: 1e-5 absolute covers the rounding of the table, not a wrong position
        np.testing.assert_allclose(vid.numpy(), want_v, atol=1e-5)
        np.testing.assert_allclose(txt.numpy(), want_t, atol=1e-5)
    one = oq.qwen_rope_freqs(cfg, 1, 4, 6, txt_len=5)
    many = oq.qwen_rope_freqs_images(cfg, [(1, 4, 6)], txt_len=5)
    assert torch.equal(one[0], many[0]) and torch.equal(one[1], many[1])


def test_layered_rotary_tables_against_numpy_positions():
    cfg = oq.tiny_config()
    for shapes in ([(1, 4, 6), (1, 4, 6), (1, 4, 6)], [(1, 2, 2)] * 5 + [(1, 2, 3)], [(1, 3, 3)]):
        vid, txt = oq.qwen_rope_freqs_images(cfg, shapes, txt_len=4, layer3d=True)
        want_v, want_t = _expected_tables(cfg, shapes, 4, layer3d=True)
        np.testing.assert_allclose(vid.numpy(), want_v, atol=1e-5)
        np.testing.assert_allclose(txt.numpy(), want_t, atol=1e-5)
    # five 2x2 layers: the half-extents are 1, so the layer count (5) decides where the text starts
    _, txt = oq.qwen_rope_freqs_images(cfg, [(1, 2, 2)] * 5 + [(1, 2, 3)], txt_len=1, layer3d=True)
    _, txt_plain = oq.qwen_rope_freqs_images(cfg, [(1, 2, 2)] * 5 + [(1, 2, 3)], txt_len=6)
    assert torch.equal(txt[0], txt_plain[4])  # plain start is 1: its row 4 is position 5


def test_additional_t_cond_adds_the_picked_table_row():
    cfg, w, lat, txt, t = _setup()
    w = dict(w)
    table = torch.randn(2, cfg.dim, generator=torch.Generator().manual_seed(9), dtype=torch.float64)
    base = oq.time_text_embed(w, t, torch.float64)
    w["time_text_embed.addition_t_embedding.weight"] = table
    got = oq.time_text_embed(w, t, torch.float64, torch.tensor([1, 0]))
    torch.testing.assert_close(got - base, table[[1, 0]], atol=1e-12, rtol=0)
    import pytest
    with pytest.raises(ValueError):
        oq.time_text_embed(w, t, torch.float64)
    # a zero table leaves the whole forward unchanged
    w["time_text_embed.addition_t_embedding.weight"] = torch.zeros_like(table)
    plain = {k: v for k, v in w.items() if "addition_t" not in k}
    torch.testing.assert_close(
        oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6), addition_t_cond=torch.tensor([1, 1])),
        oq.transformer_forward(plain, cfg, lat, txt, t, (1, 4, 6)), atol=0, rtol=0)


def test_modulate_index_layout():
    idx = oq.modulate_index([[(1, 2, 3), (1, 2, 2), (1, 1, 1)], [(1, 2, 3), (1, 1, 5)]])
    assert idx.dtype == torch.int32
    assert idx.tolist() == [[0] * 6 + [1] * 5, [0] * 6 + [1] * 5]
    assert oq.modulate_index([[(1, 2, 2)]]).tolist() == [[0, 0, 0, 0]]


def test_masked_text_keys_equal_deleted_text_keys():
    """Text positions start at a fixed offset and grow with the token number, so cutting the text tail
    leaves every remaining position unchanged: masking the last text tokens as keys must give the image
    output of the shorter prompt. A wrong joint order ([img; txt] instead of [txt; img]) or a mask
    applied to the wrong rows breaks this."""
    cfg, w, lat, txt, t = _setup(n_txt=9)
    keep = 6
    S_img = lat.shape[1]
    mask = torch.ones(2, 9 + S_img, dtype=torch.bool)
    mask[:, keep:9] = False
    masked = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6), key_mask=mask)
    short = oq.transformer_forward(w, cfg, lat, txt[:, :keep], t, (1, 4, 6))
    torch.testing.assert_close(masked, short, atol=2e-6, rtol=0)


def test_batch_rows_are_independent():
    cfg, w, lat, txt, t = _setup(B=2)
    both = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6))
    for b in range(2):
        one = oq.transformer_forward(w, cfg, lat[b:b + 1], txt[b:b + 1], t[b:b + 1], (1, 4, 6))
        torch.testing.assert_close(both[b:b + 1], one, atol=2e-6, rtol=0)


def _gate_only(w, cfg, which):
    """Modulation that is zero except for gate = 1 on the named (stream, branch) pairs: weights of the
    modulation projections zero, biases zero except the gate chunks. Chunk order per stream is
    (shift1, scale1, gate1, shift2, scale2, gate2)."""
    C = cfg.dim
    w = dict(w)
    for i in range(cfg.num_layers):
        for s in ("img", "txt"):
            w[f"transformer_blocks.{i}.{s}_mod.1.weight"] = torch.zeros_like(w[f"transformer_blocks.{i}.{s}_mod.1.weight"])
            b = torch.zeros_like(w[f"transformer_blocks.{i}.{s}_mod.1.bias"])
            if (s, "attn") in which:
                b[2 * C:3 * C] = 1
            if (s, "mlp") in which:
                b[5 * C:6 * C] = 1
            w[f"transformer_blocks.{i}.{s}_mod.1.bias"] = b
    return w


def test_closed_gates_make_the_blocks_an_identity():
    cfg, w, lat, txt, t = _setup()
    w0 = _gate_only(w, cfg, set())
    out, per_block = oq.transformer_forward(w0, cfg, lat, txt, t, (1, 4, 6), collect_blocks=True)
    img0, txt0, temb = oq.stem(w0, cfg, lat, txt, t)
    for img_b, txt_b in per_block:
        assert torch.equal(img_b, img0) and torch.equal(txt_b, txt0)
    torch.testing.assert_close(out, oq.head(w0, cfg, img0, temb), atol=0, rtol=0)


def test_one_open_gate_adds_that_branch_only():
    """Image MLP gate open, everything else closed, one block: img = img0 + MLP(LayerNorm(img0)) stated
    with library routines; text untouched. Pins the gate chunk positions and that shift/scale of zero
    leave the normalised rows alone."""
    cfg, w, lat, txt, t = _setup()
    w1 = _gate_only(w, cfg, {("img", "mlp")})
    img0, txt0, temb = oq.stem(w1, cfg, lat, txt, t)
    vf, tf = oq.qwen_rope_freqs(cfg, 1, 4, 6, txt_len=txt.shape[1])
    txt1, img1 = oq.block_forward(w1, 0, cfg, img0, txt0, temb, vf, tf)
    assert torch.equal(txt1, txt0)
    p = "transformer_blocks.0.img_mlp."
    h = F.layer_norm(img0, (cfg.dim,), eps=cfg.eps)
    h = F.gelu(F.linear(h, w1[p + "net.0.proj.weight"], w1[p + "net.0.proj.bias"]), approximate="tanh")
    want = img0 + F.linear(h, w1[p + "net.2.weight"], w1[p + "net.2.bias"])
    torch.testing.assert_close(img1, want, atol=1e-9, rtol=0)
    # text attention gate open instead: text changes, image does not
    w2 = _gate_only(w, cfg, {("txt", "attn")})
    txt2, img2 = oq.block_forward(w2, 0, cfg, img0, txt0, temb, vf, tf)
    assert torch.equal(img2, img0) and not torch.equal(txt2, txt0)


def test_attention_of_a_block_against_library_routine():
    """Both attention gates open, MLP gates closed, no rotation (a 1x1x1 image sits at position 0 on
    every axis... only for that token), so use the library attention on explicitly rotated q/k instead:
    the block's image delta must equal to_out(SDPA(...)) built from library calls and the oracle's own
    pinned per-op functions."""
    cfg, w, lat, txt, t = _setup(B=1, grid=(1, 2, 3), n_txt=4)
    w1 = _gate_only(w, cfg, {("img", "attn"), ("txt", "attn")})
    img0, txt0, temb = oq.stem(w1, cfg, lat, txt, t)
    vf, tf = oq.qwen_rope_freqs(cfg, 1, 2, 3, txt_len=4)
    txt1, img1 = oq.block_forward(w1, 0, cfg, img0, txt0, temb, vf, tf)
    p = "transformer_blocks.0.attn."
    H, D = cfg.num_heads, cfg.head_dim

    def qkv(x, name):
        y = F.linear(F.layer_norm(x, (cfg.dim,), eps=cfg.eps), w1[p + name + ".weight"], w1[p + name + ".bias"])
        return [c.unflatten(-1, (H, D)) for c in y.chunk(3, dim=-1)]

    def rot(x, fr):  # complex product on consecutive pairs
        xc = torch.view_as_complex(x.reshape(*x.shape[:-1], -1, 2).contiguous())
        return torch.view_as_real(xc * fr.to(xc.dtype)[None, :, None, :]).flatten(-2)

    iq, ik, iv = qkv(img0, "to_qkv")
    tq, tk, tv = qkv(txt0, "add_kv_proj")
    rms = lambda x, wt: F.rms_norm(x, (D,), wt, eps=cfg.eps)  # noqa: E731
    q = torch.cat([rot(rms(tq, w1[p + "norm_added_q.weight"]), tf), rot(rms(iq, w1[p + "norm_q.weight"]), vf)], dim=1)
    k = torch.cat([rot(rms(tk, w1[p + "norm_added_k.weight"]), tf), rot(rms(ik, w1[p + "norm_k.weight"]), vf)], dim=1)
    v = torch.cat([tv, iv], dim=1)
    o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    o = o.flatten(2, 3)
    want_img = img0 + F.linear(o[:, 4:], w1[p + "to_out.weight"], w1[p + "to_out.bias"])
    want_txt = txt0 + F.linear(o[:, :4], w1[p + "to_add_out.weight"], w1[p + "to_add_out.bias"])
    torch.testing.assert_close(img1, want_img, atol=2e-6, rtol=0)
    torch.testing.assert_close(txt1, want_txt, atol=2e-6, rtol=0)


def test_fp32_agrees_with_fp64():
    cfg, w, lat, txt, t = _setup()
    want = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6))
    w32 = {k: v.float() for k, v in w.items()}
    got = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), (1, 4, 6))
    assert (got.double() - want).abs().max().item() <= 2e-4 * want.abs().max().item() + 1e-5


def test_modulated_input_is_block0_norm1_of_the_stem_output():
    cfg, w, lat, txt, t = _setup()
    img0, _, temb = oq.stem(w, cfg, lat, txt, t)
    got = oq.modulated_input(w, cfg, img0, temb)
    mod = F.linear(F.silu(temb), w["transformer_blocks.0.img_mod.1.weight"], w["transformer_blocks.0.img_mod.1.bias"])
    C = cfg.dim
    want = F.layer_norm(img0, (C,), eps=cfg.eps) * (1 + mod[:, None, C:2 * C]) + mod[:, None, :C]
    torch.testing.assert_close(got, want, atol=1e-9, rtol=0)


# ------------------------------------------------------------------------------- editing variant
def test_zero_cond_t_single_image_equals_plain_model():
    """One image per sample: every token has index 0 = the real-timestep rows, the text stream and the
    head use the first half of temb, so the doubled-timestep path must reproduce the plain forward."""
    cfg, w, lat, txt, t = _setup()
    plain = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6))
    edit = oq.transformer_forward(w, cfg, lat, txt, t, (1, 4, 6), zero_cond_t=True)
    torch.testing.assert_close(edit, plain, atol=1e-12, rtol=0)


def test_zero_cond_t_at_timestep_zero_equals_plain_model():
    """t = 0 makes both halves of the doubled timestep equal, so the per-token choice is void."""
    cfg, w, lat, txt, t = _setup(grid=(1, 4, 6))
    shapes = [(1, 2, 6), (1, 2, 3), (1, 3, 2)]  # 12 + 6 + 6 = 24 tokens
    t0 = torch.zeros_like(t)
    plain = oq.transformer_forward(w, cfg, lat, txt, t0, shapes)
    edit = oq.transformer_forward(w, cfg, lat, txt, t0, shapes, zero_cond_t=True)
    torch.testing.assert_close(edit, plain, atol=1e-12, rtol=0)
    # and at t != 0 the variant does differ once target tokens exist
    assert not torch.allclose(oq.transformer_forward(w, cfg, lat, txt, t, shapes),
                              oq.transformer_forward(w, cfg, lat, txt, t, shapes, zero_cond_t=True), atol=1e-6)


def test_zero_cond_t_target_tokens_ignore_the_timestep_when_attention_is_cut():
    """With both attention output projections zeroed every token is processed on its own. Tokens of the
    later images (index 1) are modulated by the timestep-zero rows in norm1 AND norm2 and gated by the
    same rows, so their block output cannot depend on t; tokens of the first image must."""
    cfg, w, lat, txt, t = _setup(B=2)
    w = dict(w)
    for n in ("to_out", "to_add_out"):
        for kind in ("weight", "bias"):
            key = f"transformer_blocks.0.attn.{n}.{kind}"
            w[key] = torch.zeros_like(w[key])
    shapes = [(1, 2, 6), (1, 3, 4)]  # 12 source tokens, 12 target tokens
    index = oq.modulate_index([shapes] * 2)
    vf, tf = oq.qwen_rope_freqs_images(cfg, shapes, txt_len=txt.shape[1])
    outs = []
    for tt in (t, (t + 0.37) % 1.0):
        img0, txt0, temb = oq.stem(w, cfg, lat, txt, torch.cat([tt, tt * 0]))
        outs.append(oq.block_forward(w, 0, cfg, img0, txt0, temb, vf, tf, modulate_index=index, zero_cond_t=True))
    (txt_a, img_a), (txt_b, img_b) = outs
    torch.testing.assert_close(img_a[:, 12:], img_b[:, 12:], atol=1e-12, rtol=0)
    assert (img_a[:, :12] - img_b[:, :12]).abs().max().item() > 1e-4
    assert (txt_a - txt_b).abs().max().item() > 1e-4  # text follows the real timestep


def test_ops_used_by_the_variant_accept_its_shapes():
    # gate per token [B,S,C] in the gated residual: equals the broadcast form row by row
    g = torch.Generator().manual_seed(5)
    h, y = torch.randn(2, 5, 8, generator=g), torch.randn(2, 5, 8, generator=g)
    gate = torch.randn(2, 5, 8, generator=g)
    got = ops.gated_residual(h, y, gate)
    for s in range(5):
        torch.testing.assert_close(got[:, s:s + 1], ops.gated_residual(h[:, s:s + 1], y[:, s:s + 1], gate[:, s:s + 1]))
