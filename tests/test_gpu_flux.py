"""Flux blocks on the GPU: a tiny dual+single-stream MMDiT (2 + 2 blocks, hidden 256, 4 heads x 64,
64 image + 16 text tokens, and a ragged 8x11 grid) built from the HIP kernels in bf16 against the fp32
CPU oracle, per block (max-abs <= 2e-2, cosine >= 0.9995); the joint-sequence fast path of the single
blocks against their two-stream reference signature; TeaCache decisions with the Flux polynomial
against the oracle's state machine."""

import pytest
import torch

from oracle import denoise as odn
from oracle import flux as ofx
from oracle import teacache as otc

pytestmark = pytest.mark.gpu


def _cosine(a, b):
    a, b = a.float().flatten().cpu(), b.float().flatten().cpu()
    return float(torch.dot(a, b) / (a.norm() * b.norm()))


def _build(gpu, dtype=torch.bfloat16, seed=0, bias_std=0.02, ref_rounding=False, guidance=True):
    from vllm_omni_amd.attention.selector import get_attn_backend
    from vllm_omni_amd.blocks.flux import FluxTransformer2DModel

    get_attn_backend.cache_clear()
    cfg = ofx.tiny_config()
    if not guidance:
        cfg = ofx.FluxConfig(**{**cfg.__dict__, "guidance_embeds": False})
    w32 = ofx.init_params(cfg, seed=seed, dtype=torch.float32, bias_std=bias_std)
    w_lp = {k: v.to(dtype) for k, v in w32.items()}
    model = FluxTransformer2DModel(
        in_channels=cfg.in_channels, out_channels=cfg.out_channels, num_layers=cfg.num_layers,
        num_single_layers=cfg.num_single_layers, attention_head_dim=cfg.head_dim,
        num_attention_heads=cfg.num_heads, joint_attention_dim=cfg.joint_attention_dim,
        pooled_projection_dim=cfg.pooled_projection_dim, guidance_embeds=cfg.guidance_embeds,
        axes_dims_rope=cfg.axes_dims_rope, ref_rounding=ref_rounding).to(gpu).to(dtype)
    model.load_flat_state(w_lp)
    return cfg, w_lp, model


def _inputs(cfg, B, grid=(8, 8), n_txt=16, seed=1, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    lat = torch.randn(B, grid[0] * grid[1], cfg.in_channels, generator=g).to(dtype)
    txt = torch.randn(B, n_txt, cfg.joint_attention_dim, generator=g).to(dtype)
    pooled = torch.randn(B, cfg.pooled_projection_dim, generator=g).to(dtype)
    t = torch.rand(B, generator=g).to(dtype)
    guidance = torch.full((B,), 3.5)
    return lat, txt, pooled, t, guidance, ofx.latent_image_ids(*grid), torch.zeros(n_txt, 3)


@pytest.mark.parametrize("fuse_min_rows", [0, 1024])
@pytest.mark.parametrize("grid,n_txt,B", [((8, 8), 16, 2), ((8, 11), 13, 1)])
def test_tiny_flux_per_block_parity(gpu, monkeypatch, grid, n_txt, B, fuse_min_rows):
    from vllm_omni_amd.blocks import qwen_image

    monkeypatch.setattr(qwen_image, "FUSE_MIN_ROWS", fuse_min_rows)  # 0: gated epilogues also at this size
    cfg, w, model = _build(gpu)
    lat, txt, pooled, t, gd, img_ids, txt_ids = _inputs(cfg, B, grid, n_txt)
    w32 = {k: v.float() for k, v in w.items()}
    want, per_block = ofx.transformer_forward(w32, cfg, lat.float(), txt.float(), pooled.float(), t.float(),
                                              img_ids, txt_ids, guidance=gd, collect_blocks=True)
    with torch.inference_mode():
        img, enc, temb, rot = model.prepare(lat.to(gpu), txt.to(gpu), pooled.to(gpu), t.to(gpu), img_ids.to(gpu),
                                            txt_ids.to(gpu), gd.to(gpu))
        blocks = list(model.transformer_blocks) + list(model.single_transformer_blocks)
        for i, block in enumerate(blocks):
            enc, img = block(hidden_states=img, encoder_hidden_states=enc, temb=temb, image_rotary_emb=rot)
            ref_img, ref_txt = per_block[i]
            for name, got, ref in (("img", img, ref_img), ("txt", enc, ref_txt)):
                err = (got.float().cpu() - ref).abs().max().item()
                cos = _cosine(got, ref)
                print(f"flux block {i} {name}: max-abs {err:.4f} cosine {cos:.6f}", flush=True)
                assert err <= 2e-2 and cos >= 0.9995, (i, name, err, cos)
        out = model.finish(img, temb, return_dict=False)[0]
    assert (out.float().cpu() - want).abs().max().item() <= 2e-2 and _cosine(out, want) >= 0.9995
    # forward() keeps one joint tensor through the single blocks: same result as block-by-block calls
    with torch.inference_mode():
        out2 = model(lat.to(gpu), txt.to(gpu), pooled.to(gpu), t.to(gpu), img_ids.to(gpu), txt_ids.to(gpu),
                     gd.to(gpu)).sample
    assert torch.equal(out2, out)


def test_flux_without_guidance_embedding_and_fused_modulation(gpu):
    cfg, w, model = _build(gpu, guidance=False)
    lat, txt, pooled, t, _, img_ids, txt_ids = _inputs(cfg, 2, seed=4)
    w32 = {k: v.float() for k, v in w.items()}
    want = ofx.transformer_forward(w32, cfg, lat.float(), txt.float(), pooled.float(), t.float(), img_ids, txt_ids)
    args = (lat.to(gpu), txt.to(gpu), pooled.to(gpu), t.to(gpu), img_ids.to(gpu), txt_ids.to(gpu))
    with torch.inference_mode():
        before = model(*args).sample
        model.fuse_modulation()
        for name, p in model.named_parameters():
            assert torch.equal(p.cpu(), w[name]), name
        after = model(*args).sample
    assert (before.float().cpu() - want).abs().max().item() <= 2e-2 and _cosine(before, want) >= 0.9995
    assert (after.float() - before.float()).abs().max().item() <= 2e-2 and _cosine(after, before) >= 0.9999


def test_flux_text_rows_are_not_rotated(gpu):
    """Text ids are zeros: the joint table is the identity on text rows (cos 1, sin 0), so shifting
    the image grid's ids must leave nothing but the image/text relative geometry changed — and a
    table built from all-zero ids must equal running with no rotary table at all."""
    cfg, w, model = _build(gpu)
    lat, txt, pooled, t, gd, img_ids, txt_ids = _inputs(cfg, 1, seed=8)
    blk = model.transformer_blocks[0]
    with torch.inference_mode():
        img, enc, temb, _ = model.prepare(lat.to(gpu), txt.to(gpu), pooled.to(gpu), t.to(gpu), img_ids.to(gpu),
                                          txt_ids.to(gpu), gd.to(gpu))
        zero_rot = model.pos_embed(torch.zeros(txt_ids.shape[0] + img_ids.shape[0], 3, device=gpu))
        assert torch.all(zero_rot[0] == 1) and torch.all(zero_rot[1] == 0)
        e0, h0 = blk(hidden_states=img, encoder_hidden_states=enc, temb=temb, image_rotary_emb=zero_rot)
        e1, h1 = blk(hidden_states=img, encoder_hidden_states=enc, temb=temb, image_rotary_emb=None)
    assert torch.equal(h0, h1) and torch.equal(e0, e1)


def _oracle_teacache_run(cfg, w, lat0, txt, pooled, gd, img_ids, txt_ids, steps, thresh):
    tc = otc.TeaCacheOracle(otc.COEFFICIENTS["FluxTransformer2DModel"], thresh, do_true_cfg=False)
    cos, sin = ofx.flux_pos_embed(cfg, torch.cat((txt_ids, img_ids), dim=0))

    def predict(latents, text, t):
        img, enc, temb = ofx.stem(w, cfg, latents, text, pooled, t, gd)
        mod = ofx.modulated_input(w, cfg, img, temb)

        def run():
            h, e = img, enc
            for i in range(cfg.num_layers):
                e, h = ofx.dual_block_forward(w, i, cfg, h, e, temb, cos, sin)
            for i in range(cfg.num_single_layers):
                e, h = ofx.single_block_forward(w, i, cfg, h, e, temb, cos, sin)
            return (h, e)

        return tc(mod, img, enc, run, lambda h: ofx.head(w, cfg, h, temb))

    return odn.diffuse(predict, lat0, txt, None, steps), tc.log


def test_flux_teacache_decisions_match_oracle(gpu):
    """28 steps, threshold 0.25, the reference's Flux coefficients, bf16 on both sides: identical
    skip/compute sequence, and the skip rate is reported."""
    from vllm_omni_amd.cache.teacache import TeaCacheBackend
    from vllm_omni_amd.denoise import diffuse_flux

    steps, thresh = 28, 0.25
    cfg, w, model = _build(gpu, ref_rounding=True)
    lat0, txt, pooled, _, gd, img_ids, txt_ids = _inputs(cfg, 1, seed=21)
    want_lat, log = _oracle_teacache_run(cfg, w, lat0, txt, pooled, gd, img_ids, txt_ids, steps, thresh)

    class Pipe:
        transformer = model

    backend = TeaCacheBackend({"rel_l1_thresh": thresh})
    backend.enable(Pipe)
    backend.refresh(Pipe, steps)
    with torch.inference_mode():
        got_lat = diffuse_flux(model, lat0.to(gpu), txt.to(gpu), pooled.to(gpu), img_ids.to(gpu), txt_ids.to(gpu),
                               steps, guidance_scale=3.5)
    hook = TeaCacheBackend.hook_of(Pipe)
    got = [d["compute"] for d in hook.decisions]
    ref = [d["compute"] for d in log]
    margins = [abs(d["acc"] - thresh) for d in log if d["rel"] is not None and d["acc"] > 0]
    print("oracle decisions:", ref, flush=True)
    print("rel (oracle | hip):", [(a["rel"], b["rel"]) for a, b in zip(log, hook.decisions)], flush=True)
    print("min |acc - thresh| margin:", min(margins) if margins else None, flush=True)
    print(f"skip rate: {ref.count(False)}/{len(ref)}", flush=True)
    assert got == ref
    assert 0 < ref.count(False) < len(ref), "trajectory should exercise both skip and compute"
    err = (got_lat.float().cpu() - want_lat.float()).abs().max().item()
    print(f"final latents max-abs diff vs bf16 oracle: {err:.4f}", flush=True)
    assert err < 0.25


def test_flux_width_blocks_against_oracle(gpu):
    """One dual and one single block at the Flux width and sequence (hidden 3072 = 24 heads x 128, 512 text +
    4096 image tokens, batch 1) against the fp32 oracle: the launches of the Flux-shape benchmark (fused
    epilogues, the two accumulating GEMMs of the single block's proj_out, attention on 4608 keys)."""
    from vllm_omni_amd.attention.selector import get_attn_backend
    from vllm_omni_amd.blocks.flux import FluxSingleTransformerBlock, FluxTransformerBlock

    get_attn_backend.cache_clear()
    cfg = ofx.FluxConfig(num_layers=1, num_single_layers=1)
    g = torch.Generator().manual_seed(23)

    def params(shapes, prefix):
        out = {}
        for n, shape in shapes.items():
            if n.endswith(("norm_q.weight", "norm_k.weight", "norm_added_q.weight", "norm_added_k.weight")):
                t = 1 + 0.1 * torch.randn(shape, generator=g)
            else:
                t = 0.02 * torch.randn(shape, generator=g)
            out[prefix + n] = t.bfloat16()
        return out

    w = {**params(ofx.dual_block_param_shapes(cfg), "transformer_blocks.0."),
         **params(ofx.single_block_param_shapes(cfg), "single_transformer_blocks.0.")}
    dual = FluxTransformerBlock(cfg.dim, cfg.num_heads, cfg.head_dim).to(gpu).bfloat16()
    single = FluxSingleTransformerBlock(cfg.dim, cfg.num_heads, cfg.head_dim).to(gpu).bfloat16()
    with torch.no_grad():
        for blk, prefix in ((dual, "transformer_blocks.0."), (single, "single_transformer_blocks.0.")):
            for k, p in blk.named_parameters():
                p.copy_(w[prefix + k].to(gpu))
    S_img, S_txt = 4096, 512
    img = torch.randn(1, S_img, cfg.dim, generator=g).bfloat16()
    txt = torch.randn(1, S_txt, cfg.dim, generator=g).bfloat16()
    temb = (0.5 * torch.randn(1, cfg.dim, generator=g)).bfloat16()
    cos, sin = ofx.flux_pos_embed(cfg, torch.cat([torch.zeros(S_txt, 3), ofx.latent_image_ids(64, 64)], dim=0))
    wf = {k: v.float() for k, v in w.items()}
    t1, i1 = ofx.dual_block_forward(wf, 0, cfg, img.float(), txt.float(), temb.float(), cos, sin)
    t2, i2 = ofx.single_block_forward(wf, 0, cfg, i1, t1, temb.float(), cos, sin)
    rot = (cos.to(gpu), sin.to(gpu))
    with torch.inference_mode():
        gt1, gi1 = dual(hidden_states=img.to(gpu), encoder_hidden_states=txt.to(gpu), temb=temb.to(gpu),
                        image_rotary_emb=rot)
        # the single block is checked on the oracle's (rounded) input so that the two errors do not add
        gt2, gi2 = single(hidden_states=i1.bfloat16().to(gpu), encoder_hidden_states=t1.bfloat16().to(gpu),
                          temb=temb.to(gpu), image_rotary_emb=rot)
    t2r, i2r = ofx.single_block_forward(wf, 0, cfg, i1.bfloat16().float(), t1.bfloat16().float(), temb.float(), cos, sin)
    for name, got, want in (("dual img", gi1, i1), ("dual txt", gt1, t1), ("single img", gi2, i2r), ("single txt", gt2, t2r)):
        a, b = got.flatten().cpu().double(), want.flatten().double()
        err, mag = (a - b).abs().max().item(), b.abs().max().item()
        cos_ab = float(torch.dot(a, b) / (a.norm() * b.norm()))
        print(f"flux-width {name}: max-abs {err:.4f} cosine {cos_ab:.6f} (|x| max {mag:.2f})", flush=True)
        assert err <= 2e-2 * max(1.0, mag / 2) and cos_ab >= 0.9995


def test_flux_teacache_decisions_on_the_fused_path(gpu):
    """The default (fused-epilogue) Flux model under the hook against the oracle and against the reference-rounding
    build: same 28 decisions; per-step rel / accumulated distance / distance to the threshold logged."""
    from vllm_omni_amd.cache.teacache import TeaCacheBackend
    from vllm_omni_amd.denoise import diffuse_flux

    steps, thresh = 28, 0.25
    runs = {}
    for name, kw in (("fused", {}), ("ref_rounding", {"ref_rounding": True})):
        cfg, w, model = _build(gpu, **kw)
        if name == "fused":
            model.fuse_modulation()   # as bench.py runs it
        lat0, txt, pooled, _, gd, img_ids, txt_ids = _inputs(cfg, 1, seed=21)

        class Pipe:
            transformer = model

        backend = TeaCacheBackend({"rel_l1_thresh": thresh})
        backend.enable(Pipe)
        backend.refresh(Pipe, steps)
        with torch.inference_mode():
            lat = diffuse_flux(model, lat0.to(gpu), txt.to(gpu), pooled.to(gpu), img_ids.to(gpu), txt_ids.to(gpu),
                               steps, guidance_scale=3.5)
        runs[name] = (list(TeaCacheBackend.hook_of(Pipe).decisions), lat.float().cpu())
    _, log = _oracle_teacache_run(cfg, w, lat0, txt, pooled, gd, img_ids, txt_ids, steps, thresh)
    fused, rr = runs["fused"][0], runs["ref_rounding"][0]
    print("step rel(fused)  rel(ref)   rel(oracle) acc(fused) |acc-thresh| compute", flush=True)
    for i, (a, b, o) in enumerate(zip(fused, rr, log)):
        if a["rel"] is not None:
            print(f"{i:4d} {a['rel']:.6f}  {b['rel']:.6f}  {o['rel']:.6f}  {a['acc']:.6f}  "
                  f"{abs(a['acc'] - thresh) if a['acc'] > 0 else float('nan'):.6f}   {a['compute']}", flush=True)
    assert [d["compute"] for d in fused] == [d["compute"] for d in rr] == [d["compute"] for d in log]
    n_skip = sum(1 for d in fused if not d["compute"])
    print(f"skip rate on the fused path: {n_skip}/{len(fused)}", flush=True)
    assert 0 < n_skip < len(fused)
    assert (runs["fused"][1] - runs["ref_rounding"][1]).abs().max().item() < 0.25

