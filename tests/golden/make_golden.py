"""Writes tests/golden/oracle_vectors.npz: small input/output vectors of the CPU oracle.

What these are: regression anchors for the oracle and a second, file-based target for the GPU parity
tests. What they are not: vectors produced by the reference — its modules import vllm and diffusers at
module top and cannot be imported where this runs, and its own tests hold no vectors for this path. The
oracle is pinned against library routines, closed forms and invariants in tests/test_oracle_*.py; this
file freezes its outputs so that a later edit of the oracle that changes a result is caught.

    python tests/golden/make_golden.py        # rewrites the .npz next to this script
"""

from __future__ import annotations

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import flux as ofx  # noqa: E402
from oracle import ops  # noqa: E402
from oracle import qwen_image as oq  # noqa: E402
from oracle import wan as ow  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_vectors.npz")


def build() -> dict[str, np.ndarray]:
    g = torch.Generator().manual_seed(2024)
    v: dict[str, torch.Tensor] = {}

    def rnd(*shape, scale=1.0):
        return torch.randn(*shape, generator=g) * scale

    # ---- per-op vectors (fp32) ----
    q, k, val = rnd(1, 10, 2, 16), rnd(1, 12, 2, 16), rnd(1, 12, 2, 16)
    mask = torch.tensor([[1, 1, 0, 1, 1, 1, 0, 0, 1, 1, 1, 1]], dtype=torch.bool)
    v["attn.q"], v["attn.k"], v["attn.v"], v["attn.mask"] = q, k, val, mask
    v["attn.out"] = ops.sdpa(q, k, val, 0.25)
    v["attn.out_masked"] = ops.sdpa(q, k, val, 0.25, key_mask=mask)
    x = rnd(2, 5, 3, 16)
    w = 1 + 0.1 * rnd(16)
    v["rms.x"], v["rms.w"] = x, w
    v["rms.head"] = ops.rms_norm_head(x, w, 1e-6)
    v["rms.row"] = ops.rms_norm_row_fp32(x.flatten(2), 1 + 0.1 * rnd(48), 1e-6)
    ang = rnd(5, 8)
    v["rope.cos"], v["rope.sin"] = torch.cos(ang), torch.sin(ang)
    v["rope.interleaved"] = ops.apply_rotary(x, torch.cos(ang), torch.sin(ang), interleaved=True)
    v["rope.neox"] = ops.apply_rotary(x, torch.cos(ang), torch.sin(ang), interleaved=False)
    h = rnd(2, 5, 48)
    mod = rnd(2, 3 * 48, scale=0.3)
    v["adaln.x"], v["adaln.mod"] = h, mod
    out, gate = ops.ada_layer_norm(h, mod, None, 1e-6)
    v["adaln.out"], v["adaln.gate"] = out, gate
    idx = torch.tensor([[0, 1, 1, 0, 1]])
    v["adaln.index"] = idx
    v["adaln.out_indexed"] = ops.ada_layer_norm(h[:1], mod, idx, 1e-6)[0]
    v["gated.out"] = ops.gated_residual(h, rnd(2, 5, 48), gate)
    cur, prev = rnd(3, 64), rnd(3, 64)
    v["rel_l1.cur"], v["rel_l1.prev"] = cur, prev
    v["rel_l1.value"] = torch.tensor([ops.rel_l1(cur[i], prev[i]) for i in range(3)], dtype=torch.float64)
    v["rel_l1.value_bf16"] = torch.tensor([ops.rel_l1(cur[i].bfloat16(), prev[i].bfloat16()) for i in range(3)],
                                          dtype=torch.float64)
    t = torch.tensor([0.0, 0.25, 1.0])
    v["temb.t"] = t
    v["temb.scale1000"] = ops.timestep_embedding(t)
    v["temb.scale1"] = ops.timestep_embedding(t * 1000, scale=1.0)

    # ---- tiny models, fp32, seeded weights (regenerated from the seed by the tests) ----
    cfg = oq.tiny_config()
    wq = oq.init_params(cfg, seed=11, bias_std=0.02)
    lat, txt, ts = rnd(1, 16, cfg.in_channels), rnd(1, 6, cfg.joint_attention_dim), torch.tensor([0.6])
    v["qwen.latents"], v["qwen.text"], v["qwen.timestep"] = lat, txt, ts
    v["qwen.out"] = oq.transformer_forward(wq, cfg, lat, txt, ts, (1, 4, 4))

    fcfg = ofx.tiny_config()
    wf = ofx.init_params(fcfg, seed=12, bias_std=0.02)
    flat, ftxt, fpool = rnd(1, 12, fcfg.in_channels), rnd(1, 5, fcfg.joint_attention_dim), rnd(1, fcfg.pooled_projection_dim)
    v["flux.latents"], v["flux.text"], v["flux.pooled"] = flat, ftxt, fpool
    v["flux.out"] = ofx.transformer_forward(wf, fcfg, flat, ftxt, fpool, torch.tensor([0.4]), ofx.latent_image_ids(3, 4),
                                            torch.zeros(5, 3), guidance=torch.tensor([3.5]))

    wcfg = ow.tiny_config()
    ww = ow.init_params(wcfg, seed=13, bias_std=0.02, norm_jitter=0.1)
    vid, wtxt = rnd(1, wcfg.in_channels, 2, 4, 6), rnd(1, 7, wcfg.text_dim)
    v["wan.video"], v["wan.text"] = vid, wtxt
    v["wan.out"] = ow.transformer_forward(ww, wcfg, vid, torch.tensor([650.0]), wtxt)
    return {k_: t_.numpy() for k_, t_ in v.items()}


if __name__ == "__main__":
    vecs = build()
    np.savez_compressed(OUT, **vecs)
    print(f"wrote {OUT}: {len(vecs)} arrays, {os.path.getsize(OUT)} bytes")
