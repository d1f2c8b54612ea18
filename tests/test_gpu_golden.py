"""HIP kernels against the committed vectors (tests/golden/oracle_vectors.npz), through the C ABI: the
same inputs the file holds, fp32 where the kernel takes it (bit-level tolerance), bf16 with the
tolerances of the parity tests otherwise."""

import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

V = {k: torch.from_numpy(a) for k, a in
     np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_vectors.npz")).items()}


def test_elementwise_kernels_fp32_against_vectors(gpu):
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD

    x = V["rms.x"].to(gpu)                      # [2,5,3,16]
    out = torch.empty_like(x)
    kernels.qknorm_rope(x, None, None, out, None, None, V["rms.w"].to(gpu), None, None, None, eps=1e-6,
                        norm_mode=ODIT_NORM_HEAD)
    torch.testing.assert_close(out.cpu(), V["rms.head"], atol=2e-6, rtol=2e-6)
    cos, sin = V["rope.cos"].to(gpu), V["rope.sin"].to(gpu)
    for neox, key in ((False, "rope.interleaved"), (True, "rope.neox")):
        from vllm_omni_amd._lib import ODIT_NORM_NONE
        kernels.qknorm_rope(x, None, None, out, None, None, None, None, cos, sin, norm_mode=ODIT_NORM_NONE, neox=neox)
        torch.testing.assert_close(out.cpu(), V[key], atol=2e-6, rtol=2e-6)
    h, mod = V["adaln.x"].to(gpu), V["adaln.mod"].to(gpu)
    shift, scale, gate = mod.chunk(3, dim=-1)
    got = kernels.adaln_modulate(h, shift, scale, eps=1e-6)
    torch.testing.assert_close(got.cpu(), V["adaln.out"], atol=5e-6, rtol=5e-6)
    got = kernels.adaln_modulate(h[:1], shift, scale, eps=1e-6, index=V["adaln.index"].to(gpu))
    torch.testing.assert_close(got.cpu(), V["adaln.out_indexed"], atol=5e-6, rtol=5e-6)
    sums = kernels.rel_l1_sums(V["rel_l1.cur"].to(gpu), V["rel_l1.prev"].to(gpu), ref_rounding=False).cpu()
    rel = (sums[:, 0] / 64) / (sums[:, 1] / 64 + 1e-8)
    torch.testing.assert_close(rel, V["rel_l1.value"], atol=1e-6, rtol=1e-6)


def test_attention_bf16_against_vectors(gpu):
    from vllm_omni_amd import kernels

    # D = 16 is below the kernel's head sizes: embed the vectors' heads in D = 64 with zero padding, which
    # changes neither the scores nor the first 16 output columns
    def pad(t):
        return torch.nn.functional.pad(t, (0, 48)).bfloat16().to(gpu)

    q, k, v = pad(V["attn.q"]), pad(V["attn.k"]), pad(V["attn.v"])
    got = kernels.attn_fwd(q, k, v, 0.25)[..., :16].float().cpu()
    torch.testing.assert_close(got, V["attn.out"], atol=2e-2, rtol=2e-2)
    got = kernels.attn_fwd(q, k, v, 0.25, key_mask=V["attn.mask"].to(gpu))[..., :16].float().cpu()
    torch.testing.assert_close(got, V["attn.out_masked"], atol=2e-2, rtol=2e-2)


def _cos(a, b):
    a, b = a.float().flatten().cpu(), b.float().flatten().cpu()
    return float(torch.dot(a, b) / (a.norm() * b.norm()))


def test_tiny_models_bf16_against_vectors(gpu):
    from oracle import flux as ofx
    from oracle import qwen_image as oq
    from oracle import wan as ow
    from vllm_omni_amd.attention.selector import get_attn_backend
    from vllm_omni_amd.blocks.flux import FluxTransformer2DModel
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformer2DModel
    from vllm_omni_amd.blocks.wan import WanTransformer3DModel

    get_attn_backend.cache_clear()
    bf = torch.bfloat16
    cfg = oq.tiny_config()
    m = QwenImageTransformer2DModel(in_channels=cfg.in_channels, out_channels=cfg.out_channels,
                                    num_layers=cfg.num_layers, attention_head_dim=cfg.head_dim,
                                    num_attention_heads=cfg.num_heads, joint_attention_dim=cfg.joint_attention_dim,
                                    axes_dims_rope=cfg.axes_dims_rope).to(gpu).to(bf)
    m.load_flat_state(oq.init_params(cfg, seed=11, bias_std=0.02))
    with torch.inference_mode():
        out = m(V["qwen.latents"].to(gpu, bf), V["qwen.text"].to(gpu, bf), None, V["qwen.timestep"].to(gpu, bf),
                [(1, 4, 4)], [6]).sample
    assert (out.float().cpu() - V["qwen.out"]).abs().max() <= 2e-2 and _cos(out, V["qwen.out"]) >= 0.9995

    fcfg = ofx.tiny_config()
    fm = FluxTransformer2DModel(in_channels=fcfg.in_channels, out_channels=fcfg.out_channels,
                                num_layers=fcfg.num_layers, num_single_layers=fcfg.num_single_layers,
                                attention_head_dim=fcfg.head_dim, num_attention_heads=fcfg.num_heads,
                                joint_attention_dim=fcfg.joint_attention_dim,
                                pooled_projection_dim=fcfg.pooled_projection_dim,
                                axes_dims_rope=fcfg.axes_dims_rope).to(gpu).to(bf)
    fm.load_flat_state(ofx.init_params(fcfg, seed=12, bias_std=0.02))
    with torch.inference_mode():
        out = fm(V["flux.latents"].to(gpu, bf), V["flux.text"].to(gpu, bf), V["flux.pooled"].to(gpu, bf),
                 torch.tensor([0.4], device=gpu, dtype=bf), ofx.latent_image_ids(3, 4).to(gpu),
                 torch.zeros(5, 3, device=gpu), torch.tensor([3.5], device=gpu)).sample
    assert (out.float().cpu() - V["flux.out"]).abs().max() <= 2e-2 and _cos(out, V["flux.out"]) >= 0.9995

    wcfg = ow.tiny_config()
    wm = WanTransformer3DModel(patch_size=wcfg.patch_size, num_attention_heads=wcfg.num_heads,
                               attention_head_dim=wcfg.head_dim, in_channels=wcfg.in_channels,
                               out_channels=wcfg.out_channels, text_dim=wcfg.text_dim, ffn_dim=wcfg.ffn_dim,
                               num_layers=wcfg.num_layers, rope_max_seq_len=wcfg.rope_max_seq_len).to(gpu).to(bf)
    wm.load_flat_state(ow.init_params(wcfg, seed=13, bias_std=0.02, norm_jitter=0.1))
    with torch.inference_mode():
        out = wm(V["wan.video"].to(gpu, bf), torch.tensor([650.0], device=gpu), V["wan.text"].to(gpu, bf)).sample
    assert (out.float().cpu() - V["wan.out"]).abs().max() <= 2e-2 and _cos(out, V["wan.out"]) >= 0.9995
