"""Block- and model-level parity on the GPU: the tiny dual-stream MMDiT (2 blocks, hidden 256,
4 heads x 64, 256 image + 64 text tokens) built from the HIP kernels in bf16 against the fp32 CPU
oracle, per block (max-abs <= 2e-2, cosine >= 0.9995); TeaCache decisions against the oracle's
sequential-CFG state machine; CFG-batched against sequential calls."""

import numpy as np
import pytest
import torch

from oracle import denoise as odn
from oracle import qwen_image as oq
from oracle import teacache as otc

pytestmark = pytest.mark.gpu

IMG_SHAPE = (1, 16, 16)   # 32x32 latent patchified 2x2
S_IMG, S_TXT = 256, 64


def _cosine(a, b):
    a, b = a.flatten().cpu().double(), b.flatten().cpu().double()
    return float(torch.dot(a, b) / (a.norm() * b.norm()))


def _build(gpu, dtype=torch.bfloat16, seed=0, bias_std=0.02, ref_rounding=False, load=True, **model_kwargs):
    from vllm_omni_amd.attention.selector import get_attn_backend
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformer2DModel

    get_attn_backend.cache_clear()
    cfg = oq.tiny_config()
    w32 = oq.init_params(cfg, seed=seed, dtype=torch.float32, bias_std=bias_std)
    w_lp = {k: v.to(dtype) for k, v in w32.items()}           # the 16-bit weights both sides use
    model = QwenImageTransformer2DModel(
        in_channels=cfg.in_channels, out_channels=cfg.out_channels, num_layers=cfg.num_layers,
        attention_head_dim=cfg.head_dim, num_attention_heads=cfg.num_heads,
        joint_attention_dim=cfg.joint_attention_dim, axes_dims_rope=cfg.axes_dims_rope,
        ref_rounding=ref_rounding, **model_kwargs).to(gpu).to(dtype)
    if load:
        model.load_flat_state(w_lp)
    return cfg, w_lp, model


def _inputs(B, seed=1, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    lat = torch.randn(B, S_IMG, 64, generator=g).to(dtype)
    txt = torch.randn(B, S_TXT, 256, generator=g).to(dtype)
    t = torch.rand(B, generator=g).to(dtype)
    return lat, txt, t


@pytest.mark.parametrize("fuse_min_rows", [0, 1024])
def test_tiny_model_per_block_parity(gpu, monkeypatch, fuse_min_rows):
    """``fuse_min_rows`` = 0: every gated projection is one GEMM per batch entry with the gate and the
    residual in its epilogue; 1024: at this size all of them run as one GEMM plus the gated-residual kernel."""
    from vllm_omni_amd.blocks import qwen_image

    monkeypatch.setattr(qwen_image, "FUSE_MIN_ROWS", fuse_min_rows)
    cfg, w, model = _build(gpu)
    lat, txt, t = _inputs(2)
    w32 = {k: v.float() for k, v in w.items()}
    want, per_block = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), IMG_SHAPE,
                                             collect_blocks=True)
    with torch.inference_mode():
        img, enc, temb, rot = model.prepare(lat.to(gpu), txt.to(gpu), t.to(gpu), [IMG_SHAPE], [S_TXT])
        for i, block in enumerate(model.transformer_blocks):
            enc, img = block(hidden_states=img, encoder_hidden_states=enc, encoder_hidden_states_mask=None,
                             temb=temb, image_rotary_emb=rot)
            ref_img, ref_txt = per_block[i]
            for name, got, ref in (("img", img, ref_img), ("txt", enc, ref_txt)):
                err = (got.float().cpu() - ref).abs().max().item()
                cos = _cosine(got, ref)
                print(f"block {i} {name}: max-abs {err:.4f} cosine {cos:.6f}", flush=True)
                assert err <= 2e-2 and cos >= 0.9995, (i, name, err, cos)
        out = model.finish(img, temb, return_dict=False)[0]
    assert (out.float().cpu() - want).abs().max().item() <= 2e-2
    assert _cosine(out, want) >= 0.9995
    # whole forward through forward() gives the same tensor as the staged calls
    with torch.inference_mode():
        out2 = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [IMG_SHAPE], [S_TXT]).sample
    assert torch.equal(out2, out)


@pytest.mark.parametrize("B,grid,n_txt", [(2, (1, 12, 20), 37), (1, (1, 7, 9), 128), (3, (1, 16, 16), 5)])
def test_tiny_model_ragged_shapes(gpu, B, grid, n_txt):
    """Non-square grids, odd token counts, a text length that is not a multiple of the 64-key tile (the
    values are then copied into the joint buffer instead of being read in place), batch 3."""
    cfg, w, model = _build(gpu)
    model.fuse_modulation()
    g = torch.Generator().manual_seed(61)
    n_img = grid[0] * grid[1] * grid[2]
    lat = torch.randn(B, n_img, 64, generator=g).bfloat16()
    txt = torch.randn(B, n_txt, 256, generator=g).bfloat16()
    t = torch.rand(B, generator=g).bfloat16()
    w32 = {k: v.float() for k, v in w.items()}
    want = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), grid)
    with torch.inference_mode():
        got = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [grid], [n_txt]).sample
    err = (got.float().cpu() - want).abs().max().item()
    print(f"B={B} grid={grid} text={n_txt}: max-abs {err:.4f} cosine {_cosine(got, want):.6f}", flush=True)
    assert err <= 2e-2 and _cosine(got, want) >= 0.9995


def test_headline_shape_block_against_oracle(gpu):
    """One block at the width and sequence the metric is quoted on (hidden 3072 = 24 heads x 128, MLP 12288,
    batch 2, 4096 image + 256 text tokens, 64x64 rotary grid) against the fp32 oracle of the same block: the
    launches are the benchmark's own (fused GEMM epilogues, key-split last round of the attention, 16-byte
    vector paths everywhere), which the tiny model does not reach."""
    from vllm_omni_amd.attention.selector import get_attn_backend
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformerBlock, RotaryTables

    get_attn_backend.cache_clear()
    cfg = oq.QwenConfig(num_layers=1)
    g = torch.Generator().manual_seed(17)
    w = {}
    for n, shape in oq.block_param_shapes(cfg).items():
        if n.endswith(("norm_q.weight", "norm_k.weight")):
            t = 1 + 0.1 * torch.randn(shape, generator=g)
        else:
            t = 0.02 * torch.randn(shape, generator=g)
        w["transformer_blocks.0." + n] = t.bfloat16()
    blk = QwenImageTransformerBlock(cfg.dim, cfg.num_heads, cfg.head_dim).to(gpu).bfloat16()
    with torch.no_grad():
        for k, p in blk.named_parameters():
            p.copy_(w["transformer_blocks.0." + k].to(gpu))
    B, S_img, S_txt = 2, 4096, 256
    img = torch.randn(B, S_img, cfg.dim, generator=g).bfloat16()
    txt = torch.randn(B, S_txt, cfg.dim, generator=g).bfloat16()
    temb = (0.5 * torch.randn(B, cfg.dim, generator=g)).bfloat16()
    vf, tf = oq.qwen_rope_freqs(cfg, 1, 64, 64, txt_len=S_txt)
    want_txt, want_img = oq.block_forward({k: v.float() for k, v in w.items()}, 0, cfg, img.float(), txt.float(),
                                          temb.float(), vf, tf)
    with torch.inference_mode():
        got_txt, got_img = blk(hidden_states=img.to(gpu), encoder_hidden_states=txt.to(gpu),
                               encoder_hidden_states_mask=None, temb=temb.to(gpu),
                               image_rotary_emb=RotaryTables(vf.to(gpu), tf.to(gpu)))
    for name, got, want in (("img", got_img, want_img), ("txt", got_txt, want_txt)):
        err = (got.float().cpu() - want).abs().max().item()
        mag = want.abs().max().item()
        print(f"headline-shape block {name}: max-abs {err:.4f} cosine {_cosine(got, want):.6f} (|x| max {mag:.2f})", flush=True)
        # a bf16 ulp at |x| in [4, 8) is 3e-2: the absolute bound scales with the magnitude reached
        assert err <= 2e-2 * max(1.0, mag / 2) and _cosine(got, want) >= 0.9995
        assert (want - (img if name == "img" else txt).float()).abs().max().item() > 20 * err  # the block did something


def test_forward_under_hip_graph_capture(gpu):
    """The whole forward can be recorded in a HIP graph (no host synchronisation, no allocation outside
    torch's capture pool, no memset nodes on the path): several replays on new inputs, with eager work
    and synchronisations in between, each give the eager result bit for bit."""
    cfg, w, model = _build(gpu)
    model.fuse_modulation()
    lat, txt, t = _inputs(2, seed=41)
    lat_g, txt_g, t_g = lat.to(gpu), txt.to(gpu), t.to(gpu)

    def fwd():
        return model(lat_g, txt_g, None, t_g, [IMG_SHAPE], [S_TXT]).sample

    with torch.inference_mode():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):     # warm-up on the side stream: workspaces and plans exist before capture
            for _ in range(2):
                fwd()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = fwd()
        for seed in (42, 43, 44):
            new_lat, _, new_t = _inputs(2, seed=seed)
            lat_g.copy_(new_lat.to(gpu))
            t_g.copy_(new_t.to(gpu))
            graph.replay()
            torch.cuda.synchronize()
            got = out.clone()
            want = fwd()
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"replay with seed {seed} differs from eager"


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 4e-3), (torch.float32, 2e-4)])
def test_tiny_model_fp16_and_fp32(gpu, dtype, tol):
    """fp16 runs the same kernels as bf16 (with the +-65504 clip of qit.py:809-812 live); fp32 activations
    bypass the flash backend for torch SDPA like the reference's Attention layer does
    (attention/layer.py:127-132) and use the fp32 instantiations of the other kernels."""
    cfg, w, model = _build(gpu, dtype=dtype)
    model.fuse_modulation()
    lat, txt, t = _inputs(2, seed=31, dtype=dtype)
    w32 = {k: v.float() for k, v in w.items()}
    want = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), IMG_SHAPE)
    with torch.inference_mode():
        got = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [IMG_SHAPE], [S_TXT]).sample
    assert got.dtype == dtype
    err = (got.float().cpu() - want).abs().max().item()
    print(f"{dtype}: max-abs {err:.2e} cosine {_cosine(got, want):.7f}", flush=True)
    assert err <= tol and _cosine(got, want) >= 0.99999


@pytest.mark.parametrize("fuse", [False, True])
def test_editing_variant_per_token_conditioning(gpu, fuse):
    """zero_cond_t: doubled timestep, per-token choice between the two conditioning rows in both norms
    and both gates of the image stream, text stream and head on the real-timestep rows. Source image
    8x16, two target images 4x16 each (256 tokens)."""
    cfg, w, model = _build(gpu, zero_cond_t=True)
    # N(0, 0.02) weights make the timestep almost irrelevant: strengthen the conditioning path so that a
    # dropped or swapped index moves the output far beyond the bf16 tolerance
    w = {k: (v * 8 if "img_mod.1.weight" in k or "timestep_embedder.linear_2.weight" in k else v) for k, v in w.items()}
    model.load_flat_state(w)
    if fuse:
        model.fuse_modulation()
    shapes = [(1, 8, 16), (1, 4, 16), (1, 4, 16)]
    lat, txt, t = _inputs(2, seed=21)
    w32 = {k: v.float() for k, v in w.items()}
    want = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), shapes, zero_cond_t=True)
    plain = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), shapes)
    with torch.inference_mode():
        index = model.modulate_index([shapes, shapes], gpu)
        assert index.dtype == torch.int32 and index.cpu().tolist() == [[0] * 128 + [1] * 128] * 2
        got = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [shapes, shapes], [S_TXT]).sample
    err = (got.float().cpu() - want).abs().max().item()
    print(f"editing variant (fused modulation {fuse}): max-abs {err:.4f} cosine {_cosine(got, want):.6f}", flush=True)
    assert err <= 2e-2 and _cosine(got, want) >= 0.9995
    # the test would not notice a dropped index if the two models agreed anyway: they do not
    assert (plain - want).abs().max().item() > 10 * err


def test_layered_variant_rope_and_additional_t_cond(gpu):
    """use_layer3d_rope (condition image at frame -1, text start at least the layer count) and
    use_additional_t_cond (a 2-entry learned embedding added to the timestep embedding)."""
    cfg, w, model = _build(gpu, use_layer3d_rope=True, use_additional_t_cond=True, load=False)
    g = torch.Generator().manual_seed(51)
    w = dict(w)
    w["time_text_embed.addition_t_embedding.weight"] = torch.randn(2, cfg.dim, generator=g).bfloat16()
    # sharper attention (q/k norm weights 3 -> logits x9): with N(0, 0.02) projections the attention is close
    # to uniform and positions would hardly matter
    w = {k: (v * 3 if k.endswith(("norm_q.weight", "norm_k.weight")) else v) for k, v in w.items()}
    model.load_flat_state(w)
    shapes = [(1, 8, 8), (1, 8, 8), (1, 8, 8), (1, 8, 8)]   # three layers + the condition image, 256 tokens
    lat, txt, t = _inputs(2, seed=52)
    cond = torch.tensor([1, 0])
    w32 = {k: v.float() for k, v in w.items()}
    want = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), shapes, layer3d_rope=True,
                                  addition_t_cond=cond)
    other = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), shapes, addition_t_cond=cond)
    with torch.inference_mode():
        got = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [shapes, shapes], [S_TXT],
                    additional_t_cond=cond.to(gpu)).sample
        with pytest.raises(ValueError, match="addition_t_cond"):
            model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [shapes, shapes], [S_TXT])
    err = (got.float().cpu() - want).abs().max().item()
    print(f"layered variant: max-abs {err:.4f} cosine {_cosine(got, want):.6f}", flush=True)
    assert err <= 2e-2 and _cosine(got, want) >= 0.9995
    assert (other - want).abs().max().item() > 5 * err   # the frame position of the last image matters


def test_teacache_refuses_the_editing_variant(gpu):
    from vllm_omni_amd.cache.teacache.extractors import extract_qwen_context

    cfg, w, model = _build(gpu, zero_cond_t=True)
    lat, txt, t = _inputs(1)
    with pytest.raises(NotImplementedError):
        extract_qwen_context(model, lat.to(gpu), txt.to(gpu), None, t.to(gpu), [[IMG_SHAPE]], [S_TXT])


def test_block_with_text_padding_mask(gpu):
    cfg, w, model = _build(gpu)
    lat, txt, t = _inputs(2, seed=3)
    mask = torch.ones(2, S_TXT, dtype=torch.bool)
    mask[1, 40:] = False
    joint = torch.cat([mask, torch.ones(2, S_IMG, dtype=torch.bool)], dim=1)
    w32 = {k: v.float() for k, v in w.items()}
    want = oq.transformer_forward(w32, cfg, lat.float(), txt.float(), t.float(), IMG_SHAPE, key_mask=joint)
    with torch.inference_mode():
        got = model(lat.to(gpu), txt.to(gpu), mask.to(gpu), t.to(gpu), [IMG_SHAPE], [S_TXT]).sample
    assert (got.float().cpu() - want).abs().max().item() <= 2e-2 and _cosine(got, want) >= 0.9995


def _oracle_teacache_run(cfg, w, lat0, pos, neg, steps, thresh, dtype):
    """Sequential-CFG denoise loop with the oracle's TeaCache, all in `dtype` on the CPU."""
    tc = otc.TeaCacheOracle(otc.COEFFICIENTS["QwenImageTransformer2DModel"], thresh, do_true_cfg=True)

    def predict(latents, text, t):
        img, txt, temb = oq.stem(w, cfg, latents, text, t)
        vf, tf = oq.qwen_rope_freqs(cfg, *IMG_SHAPE, txt_len=text.shape[1])
        mod = oq.modulated_input(w, cfg, img, temb)

        def run():
            h, e = img, txt
            for i in range(cfg.num_layers):
                e, h = oq.block_forward(w, i, cfg, h, e, temb, vf, tf)
            return (h, e)

        return tc(mod, img, txt, run, lambda h: oq.head(w, cfg, h, temb))

    out = odn.diffuse(predict, lat0, pos, neg, steps, cfg_scale=4.0, normalize=True)
    return out, tc.log


def test_teacache_decisions_match_oracle_batched_cfg(gpu):
    """Same seeded inputs, bf16 on both sides: the CFG-batched HIP path must take exactly the
    oracle's (sequential-CFG) skip/compute decisions, branch by branch, step by step."""
    from vllm_omni_amd.cache.teacache import TeaCacheBackend
    from vllm_omni_amd.denoise import DenoiseInputs, diffuse

    steps, thresh = 12, 0.25
    cfg, w, model = _build(gpu, ref_rounding=True)
    g = torch.Generator().manual_seed(11)
    lat0 = torch.randn(1, S_IMG, 64, generator=g).bfloat16()
    pos = torch.randn(1, S_TXT, 256, generator=g).bfloat16()
    neg = torch.randn(1, S_TXT, 256, generator=g).bfloat16()
    want_lat, log = _oracle_teacache_run(cfg, w, lat0, pos, neg, steps, thresh, torch.bfloat16)

    class Pipe:
        transformer = model

    backend = TeaCacheBackend({"rel_l1_thresh": thresh})
    backend.enable(Pipe)
    backend.refresh(Pipe, steps)
    with torch.inference_mode():
        got_lat = diffuse(model, DenoiseInputs(lat0.to(gpu), pos.to(gpu), neg.to(gpu), IMG_SHAPE), steps,
                          true_cfg_scale=4.0, cfg_normalize=True)
    hook = TeaCacheBackend.hook_of(Pipe)
    got = [(d["branch"], d["compute"]) for d in hook.decisions]
    ref = [("teacache_" + d["branch"], d["compute"]) for d in log]
    margins = [abs(d["acc"] - thresh) for d in log if d["rel"] is not None and d["acc"] > 0]
    print("oracle decisions:", ref, flush=True)
    print("rel (oracle | hip):", [(a["rel"], b["rel"]) for a, b in zip(log, hook.decisions)], flush=True)
    print("min |acc - thresh| margin:", min(margins) if margins else None, flush=True)
    assert got == ref
    n_skip = sum(1 for _, c in got if not c)
    assert 0 < n_skip < len(got), "trajectory should exercise both skip and compute"
    err = (got_lat.float().cpu() - want_lat.float()).abs().max().item()
    print(f"final latents max-abs diff vs bf16 oracle: {err:.4f}", flush=True)
    assert err < 0.25  # bf16-vs-bf16 drift over 12 steps; decisions above are the exact check


def test_teacache_decisions_on_the_fused_path(gpu):
    """The model as bench.py builds it (fused GEMM epilogues, prescaled gate rows, values read in place) under the
    hook: its decisions must equal the oracle's and those of the reference-rounding build on the same seeds. The
    extractor rounds the decision tensor like the reference whatever the blocks do, so the only difference between
    the two builds is the drift of the latents; rel, the accumulated distance and its distance to the threshold
    are logged per step for both."""
    from vllm_omni_amd.cache.teacache import TeaCacheBackend
    from vllm_omni_amd.denoise import DenoiseInputs, diffuse

    steps, thresh = 12, 0.25
    g = torch.Generator().manual_seed(11)
    lat0 = torch.randn(1, S_IMG, 64, generator=g).bfloat16()
    pos = torch.randn(1, S_TXT, 256, generator=g).bfloat16()
    neg = torch.randn(1, S_TXT, 256, generator=g).bfloat16()
    runs = {}
    for name, kw in (("fused", {}), ("ref_rounding", {"ref_rounding": True})):
        cfg, w, model = _build(gpu, **kw)
        if name == "fused":
            model.fuse_modulation()   # as bench.py runs it: all modulation projections of a step in one GEMM

        class Pipe:
            transformer = model

        backend = TeaCacheBackend({"rel_l1_thresh": thresh})
        backend.enable(Pipe)
        backend.refresh(Pipe, steps)
        with torch.inference_mode():
            lat = diffuse(model, DenoiseInputs(lat0.to(gpu), pos.to(gpu), neg.to(gpu), IMG_SHAPE), steps,
                          true_cfg_scale=4.0, cfg_normalize=True)
        runs[name] = (list(TeaCacheBackend.hook_of(Pipe).decisions), lat.float().cpu())
    _, log = _oracle_teacache_run(cfg, w, lat0, pos, neg, steps, thresh, torch.bfloat16)
    fused, rr = runs["fused"][0], runs["ref_rounding"][0]
    print("step branch            rel(fused)  rel(ref)    acc(fused)  acc(ref)   |acc-thresh| compute", flush=True)
    for i, (a, b) in enumerate(zip(fused, rr)):
        if a["rel"] is not None:
            print(f"{i // 2:4d} {a['branch']:18s} {a['rel']:.6f}  {b['rel']:.6f}  {a['acc']:.6f}  {b['acc']:.6f}  "
                  f"{abs(a['acc'] - thresh) if a['acc'] > 0 else float('nan'):.6f}   {a['compute']}", flush=True)
    assert [(d["branch"], d["compute"]) for d in fused] == [(d["branch"], d["compute"]) for d in rr]
    assert [(d["branch"], d["compute"]) for d in fused] == [("teacache_" + d["branch"], d["compute"]) for d in log]
    n_skip = sum(1 for d in fused if not d["compute"])
    assert 0 < n_skip < len(fused)
    drift = (runs["fused"][1] - runs["ref_rounding"][1]).abs().max().item()
    print(f"fused vs reference-rounding latents after {steps} steps: max-abs {drift:.4f}; skipped {n_skip}/{len(fused)}",
          flush=True)
    assert drift < 0.25


def test_fused_modulation_is_bit_identical(gpu):
    """Stacking the 2L modulation projections changes the schedule, not one output bit of a block
    stack fed with the same temb (per-row GEMV results do not depend on how many rows are stacked...
    up to the GEMM library's tiling, so compare at tolerance and the parameters for equality)."""
    cfg, w, model = _build(gpu)
    lat, txt, t = _inputs(2, seed=9)
    with torch.inference_mode():
        before = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [IMG_SHAPE], [S_TXT]).sample
        model.fuse_modulation()
        for name, p in model.named_parameters():
            assert torch.equal(p.cpu(), w[name]), name
        after = model(lat.to(gpu), txt.to(gpu), None, t.to(gpu), [IMG_SHAPE], [S_TXT]).sample
    assert (after.float() - before.float()).abs().max().item() <= 2e-2 and _cosine(after, before) >= 0.9999


def test_weights_loaded_after_fusing_are_used(gpu):
    """fuse_modulation() stacks weights and the model caches float32 copies of the gated projections' biases;
    loading another state afterwards must be picked up by both."""
    cfg, w, model = _build(gpu, seed=0)
    lat, txt, t = _inputs(2, seed=12)
    args = (lat.to(gpu), txt.to(gpu), None, t.to(gpu), [IMG_SHAPE], [S_TXT])
    model.fuse_modulation()
    with torch.inference_mode():
        model(*args)                                   # populates the caches with the seed-0 biases
    w2 = {k: v.bfloat16() for k, v in oq.init_params(cfg, seed=5, bias_std=0.05).items()}
    model.load_flat_state(w2)
    _, _, fresh = _build(gpu, seed=5, bias_std=0.05)
    with torch.inference_mode():
        got = model(*args).sample
        want = fresh(*args).sample
    assert (got.float() - want.float()).abs().max().item() <= 2e-2 and _cosine(got, want) >= 0.9999


def test_cfg_batched_equals_sequential(gpu):
    cfg, w, model = _build(gpu)
    lat, _, _ = _inputs(1, seed=5)
    with pytest.raises(TypeError, match="guidance"):   # as in the reference, whose time embedding takes none
        model(lat.to(gpu), torch.zeros(1, S_TXT, 256, device=gpu).bfloat16(), None, torch.ones(1, device=gpu),
              [IMG_SHAPE], [S_TXT], guidance=torch.ones(1, device=gpu))
    g = torch.Generator().manual_seed(6)
    text = torch.randn(2, S_TXT, 256, generator=g).bfloat16().to(gpu)
    t = torch.tensor([0.7, 0.7]).bfloat16().to(gpu)
    with torch.inference_mode():
        both = model(lat.to(gpu).expand(2, -1, -1), text, None, t, [IMG_SHAPE], [S_TXT, S_TXT]).sample
        one = [model(lat.to(gpu), text[i:i + 1], None, t[i:i + 1], [IMG_SHAPE], [S_TXT]).sample for i in range(2)]
    for i in range(2):
        d = (both[i:i + 1].float() - one[i].float()).abs().max().item()
        assert d <= 2e-2, d   # GEMM tiling may differ with M; everything else is row-independent


def test_cfg_mixin_diffuse_one_call_against_two(gpu):
    """The reference's step loop (QwenImageCFGParallelMixin.diffuse) around the HIP transformer, prompts of
    different lengths: the one-call schedule (negative prompt padded and masked) against the reference's two
    sequential calls, and, for equal lengths, against this package's own loop."""
    from vllm_omni_amd import denoise

    cfg, w, model = _build(gpu)
    steps = 4
    g = torch.Generator().manual_seed(21)
    lat0 = torch.randn(1, S_IMG, 64, generator=g).bfloat16().to(gpu)
    pos = torch.randn(1, S_TXT, 256, generator=g).bfloat16().to(gpu)
    neg = torch.randn(1, S_TXT, 256, generator=g).bfloat16().to(gpu)

    class Pipe(denoise.QwenImageCFGParallelMixin):
        transformer = model

    def run(batched, negative):
        pipe = Pipe()
        pipe.batch_cfg_branches = batched
        pipe.scheduler = denoise.FlowMatchEulerScheduler()
        pipe.scheduler.set_timesteps(sigmas=np.linspace(1.0, 1.0 / steps, steps), device=gpu,
                                     mu=denoise.calculate_shift(S_IMG))
        with torch.inference_mode():
            return pipe.diffuse(pos, None, negative, None, lat0, [[IMG_SHAPE]], [S_TXT], [negative.shape[1]],
                                pipe.scheduler.timesteps, True, None, 4.0, cfg_normalize=True,
                                additional_transformer_kwargs={"return_dict": False})

    short = neg[:, :40]
    one_call, two_calls = run(True, short), run(False, short)
    assert model.cfg_batched_branches is None          # the last run made two calls per step
    d = (one_call.float() - two_calls.float()).abs().max().item()
    print(f"ragged prompts, {steps} steps: one call vs two, max-abs {d:.4f}", flush=True)
    assert d <= 5e-2 and _cosine(one_call, two_calls) >= 0.9995
    # the padding must not leak: other padding values, same answer
    same_len = run(True, neg)
    with torch.inference_mode():
        own = denoise.diffuse(model, denoise.DenoiseInputs(lat0, pos, neg, IMG_SHAPE), steps, 4.0, True)
    assert torch.equal(same_len, own)
    assert (same_len.float() - one_call.float()).abs().max().item() > 1e-2   # 24 more negative tokens matter
