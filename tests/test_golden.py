"""The oracle against its committed vectors (tests/golden/oracle_vectors.npz, written by
tests/golden/make_golden.py): every stored output must be reproduced from the stored inputs (and, for
the tiny models, from weights regenerated from their seeds). These vectors come from the oracle itself,
not from the reference (which cannot be imported here); they catch unintended changes of the oracle."""

import os

import numpy as np
import torch

from oracle import flux as ofx
from oracle import ops
from oracle import qwen_image as oq
from oracle import wan as ow

V = {k: torch.from_numpy(a) for k, a in
     np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_vectors.npz")).items()}
TOL = dict(atol=1e-6, rtol=1e-6)


def test_ops_reproduce_their_vectors():
    torch.testing.assert_close(ops.sdpa(V["attn.q"], V["attn.k"], V["attn.v"], 0.25), V["attn.out"], **TOL)
    torch.testing.assert_close(ops.sdpa(V["attn.q"], V["attn.k"], V["attn.v"], 0.25, key_mask=V["attn.mask"]),
                               V["attn.out_masked"], **TOL)
    torch.testing.assert_close(ops.rms_norm_head(V["rms.x"], V["rms.w"], 1e-6), V["rms.head"], **TOL)
    torch.testing.assert_close(ops.apply_rotary(V["rms.x"], V["rope.cos"], V["rope.sin"], interleaved=True),
                               V["rope.interleaved"], **TOL)
    torch.testing.assert_close(ops.apply_rotary(V["rms.x"], V["rope.cos"], V["rope.sin"], interleaved=False),
                               V["rope.neox"], **TOL)
    out, gate = ops.ada_layer_norm(V["adaln.x"], V["adaln.mod"], None, 1e-6)
    torch.testing.assert_close(out, V["adaln.out"], **TOL)
    torch.testing.assert_close(gate, V["adaln.gate"], **TOL)
    torch.testing.assert_close(ops.ada_layer_norm(V["adaln.x"][:1], V["adaln.mod"], V["adaln.index"], 1e-6)[0],
                               V["adaln.out_indexed"], **TOL)
    for i in range(3):
        assert abs(ops.rel_l1(V["rel_l1.cur"][i], V["rel_l1.prev"][i]) - V["rel_l1.value"][i].item()) < 1e-7
        assert ops.rel_l1(V["rel_l1.cur"][i].bfloat16(), V["rel_l1.prev"][i].bfloat16()) == V["rel_l1.value_bf16"][i].item()
    torch.testing.assert_close(ops.timestep_embedding(V["temb.t"]), V["temb.scale1000"], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(ops.timestep_embedding(V["temb.t"] * 1000, scale=1.0), V["temb.scale1"], atol=1e-5, rtol=1e-5)


def test_tiny_models_reproduce_their_vectors():
    cfg = oq.tiny_config()
    w = oq.init_params(cfg, seed=11, bias_std=0.02)
    out = oq.transformer_forward(w, cfg, V["qwen.latents"], V["qwen.text"], V["qwen.timestep"], (1, 4, 4))
    torch.testing.assert_close(out, V["qwen.out"], atol=1e-5, rtol=1e-5)
    fcfg = ofx.tiny_config()
    wf = ofx.init_params(fcfg, seed=12, bias_std=0.02)
    out = ofx.transformer_forward(wf, fcfg, V["flux.latents"], V["flux.text"], V["flux.pooled"], torch.tensor([0.4]),
                                  ofx.latent_image_ids(3, 4), torch.zeros(5, 3), guidance=torch.tensor([3.5]))
    torch.testing.assert_close(out, V["flux.out"], atol=1e-5, rtol=1e-5)
    wcfg = ow.tiny_config()
    ww = ow.init_params(wcfg, seed=13, bias_std=0.02, norm_jitter=0.1)
    out = ow.transformer_forward(ww, wcfg, V["wan.video"], torch.tensor([650.0]), V["wan.text"])
    torch.testing.assert_close(out, V["wan.out"], atol=1e-5, rtol=1e-5)
