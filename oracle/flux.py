"""Oracle restatement of the Flux dual-stream + single-stream MMDiT forward (test infrastructure only).

Functional, like ``oracle/qwen_image.py``: weights are a flat ``dict[str, Tensor]`` keyed with the
reference's parameter names. Reference file: ``vllm_omni/diffusion/models/flux/flux_transformer.py``
(cited below as ``flux.py``).

Third-party arithmetic on this path (diffusers>=0.36.0, absent from the reference tree — **parity
unpinned** at that boundary, upstream conventions adopted):
  * ``AdaLayerNormZero``        emb = Linear(SiLU(temb)); chunk(6) = shift_msa, scale_msa, gate_msa,
                                shift_mlp, scale_mlp, gate_mlp; x = LN(x)(1 + scale_msa) + shift_msa
  * ``AdaLayerNormZeroSingle``  emb = Linear(SiLU(temb)); chunk(3) = shift, scale, gate
  * ``AdaLayerNormContinuous``  chunk(2) = scale, shift
  * ``CombinedTimestep(Guidance)TextProjEmbeddings``  sinusoid(256, cos first) -> MLP for timestep and
                                guidance, PixArtAlphaTextProjection (Linear, SiLU, Linear) for the pooled
                                text vector; the three are summed
  * ``get_1d_rotary_pos_embed(use_real=False, freqs_dtype=float64)``  exp(i * pos * theta^(-2j/dim))
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import ops


@dataclass(frozen=True)
class FluxConfig:
    """Defaults = FLUX.1 (flux.py:440-453)."""

    num_layers: int = 19
    num_single_layers: int = 38
    num_heads: int = 24
    head_dim: int = 128
    in_channels: int = 64
    out_channels: int = 64
    patch_size: int = 1
    joint_attention_dim: int = 4096
    pooled_projection_dim: int = 768
    guidance_embeds: bool = True
    axes_dims_rope: tuple[int, int, int] = (16, 56, 56)
    theta: int = 10000
    mlp_ratio: int = 4
    eps: float = 1e-6

    @property
    def dim(self) -> int:
        return self.num_heads * self.head_dim


def tiny_config() -> FluxConfig:
    """CPU-runnable case: 2 dual + 2 single blocks, hidden 256 = 4 heads x 64."""
    return FluxConfig(num_layers=2, num_single_layers=2, num_heads=4, head_dim=64, in_channels=64,
                      out_channels=64, joint_attention_dim=128, pooled_projection_dim=96,
                      axes_dims_rope=(8, 28, 28))


# ------------------------------------------------------------------------------------- weights
def dual_block_param_shapes(cfg: FluxConfig) -> dict[str, tuple[int, ...]]:
    C, D, F_ = cfg.dim, cfg.head_dim, cfg.dim * cfg.mlp_ratio
    return {
        "norm1.linear.weight": (6 * C, C), "norm1.linear.bias": (6 * C,),
        "norm1_context.linear.weight": (6 * C, C), "norm1_context.linear.bias": (6 * C,),
        "attn.to_qkv.weight": (3 * C, C), "attn.to_qkv.bias": (3 * C,),
        "attn.add_kv_proj.weight": (3 * C, C), "attn.add_kv_proj.bias": (3 * C,),
        "attn.norm_q.weight": (D,), "attn.norm_k.weight": (D,),
        "attn.norm_added_q.weight": (D,), "attn.norm_added_k.weight": (D,),
        "attn.to_out.0.weight": (C, C), "attn.to_out.0.bias": (C,),
        "attn.to_add_out.weight": (C, C), "attn.to_add_out.bias": (C,),
        "ff.net.0.proj.weight": (F_, C), "ff.net.0.proj.bias": (F_,),
        "ff.net.2.weight": (C, F_), "ff.net.2.bias": (C,),
        "ff_context.net.0.proj.weight": (F_, C), "ff_context.net.0.proj.bias": (F_,),
        "ff_context.net.2.weight": (C, F_), "ff_context.net.2.bias": (C,),
    }


def single_block_param_shapes(cfg: FluxConfig) -> dict[str, tuple[int, ...]]:
    C, D, F_ = cfg.dim, cfg.head_dim, cfg.dim * cfg.mlp_ratio
    return {
        "norm.linear.weight": (3 * C, C), "norm.linear.bias": (3 * C,),
        "proj_mlp.weight": (F_, C), "proj_mlp.bias": (F_,),
        "proj_out.weight": (C, C + F_), "proj_out.bias": (C,),
        "attn.to_qkv.weight": (3 * C, C), "attn.to_qkv.bias": (3 * C,),
        "attn.norm_q.weight": (D,), "attn.norm_k.weight": (D,),
    }


def stem_param_shapes(cfg: FluxConfig) -> dict[str, tuple[int, ...]]:
    C = cfg.dim
    out = {
        "x_embedder.weight": (C, cfg.in_channels), "x_embedder.bias": (C,),
        "context_embedder.weight": (C, cfg.joint_attention_dim), "context_embedder.bias": (C,),
        "time_text_embed.timestep_embedder.linear_1.weight": (C, 256),
        "time_text_embed.timestep_embedder.linear_1.bias": (C,),
        "time_text_embed.timestep_embedder.linear_2.weight": (C, C),
        "time_text_embed.timestep_embedder.linear_2.bias": (C,),
        "time_text_embed.text_embedder.linear_1.weight": (C, cfg.pooled_projection_dim),
        "time_text_embed.text_embedder.linear_1.bias": (C,),
        "time_text_embed.text_embedder.linear_2.weight": (C, C),
        "time_text_embed.text_embedder.linear_2.bias": (C,),
        "norm_out.linear.weight": (2 * C, C), "norm_out.linear.bias": (2 * C,),
        "proj_out.weight": (cfg.patch_size ** 2 * cfg.out_channels, C),
        "proj_out.bias": (cfg.patch_size ** 2 * cfg.out_channels,),
    }
    if cfg.guidance_embeds:
        out.update({
            "time_text_embed.guidance_embedder.linear_1.weight": (C, 256),
            "time_text_embed.guidance_embedder.linear_1.bias": (C,),
            "time_text_embed.guidance_embedder.linear_2.weight": (C, C),
            "time_text_embed.guidance_embedder.linear_2.bias": (C,),
        })
    return out


def init_params(cfg: FluxConfig, seed: int = 0, dtype: torch.dtype = torch.float32, std: float = 0.02,
                bias_std: float = 0.0, device: str = "cpu") -> dict[str, torch.Tensor]:
    """Synthetic weights: matrices N(0, std), RMSNorm weights 1, biases N(0, bias_std) (0 by default)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    out: dict[str, torch.Tensor] = {}

    def make(name: str, shape: tuple[int, ...]):
        if name.endswith(("norm_q.weight", "norm_k.weight")):
            t = torch.ones(shape)
        elif name.endswith(".bias"):
            t = torch.randn(shape, generator=g) * bias_std if bias_std > 0 else torch.zeros(shape)
        else:
            t = torch.randn(shape, generator=g) * std
        out[name] = t.to(dtype).to(device)

    for n, s in stem_param_shapes(cfg).items():
        make(n, s)
    for i in range(cfg.num_layers):
        for n, s in dual_block_param_shapes(cfg).items():
            make(f"transformer_blocks.{i}.{n}", s)
    for i in range(cfg.num_single_layers):
        for n, s in single_block_param_shapes(cfg).items():
            make(f"single_transformer_blocks.{i}.{n}", s)
    return out


# ------------------------------------------------------------------------------------- rope tables
def latent_image_ids(height: int, width: int) -> torch.Tensor:
    """[H*W, 3] ids (0, y, x) of the packed latent grid. models/flux/pipeline_flux.py:386-394
    (text ids are zeros: pipeline_flux.py:386)."""
    ids = torch.zeros(height, width, 3)
    ids[..., 1] = ids[..., 1] + torch.arange(height)[:, None]
    ids[..., 2] = ids[..., 2] + torch.arange(width)[None, :]
    return ids.reshape(height * width, 3)


def flux_pos_embed(cfg: FluxConfig, ids: torch.Tensor):
    """FluxPosEmbed.forward, flux.py:369-396: per axis exp(i * pos * theta^(-2j/d)) evaluated in
    float64, real and imaginary parts concatenated over the axes -> (cos, sin) [S, D/2] float64."""
    pos = ids.float()
    cos_out, sin_out = [], []
    for i, d in enumerate(cfg.axes_dims_rope):
        inv = 1.0 / (cfg.theta ** (torch.arange(0, d, 2, dtype=torch.float64)[: d // 2] / d))
        ang = torch.outer(pos[:, i].to(torch.float64), inv)
        cos_out.append(torch.cos(ang))
        sin_out.append(torch.sin(ang))
    return torch.cat(cos_out, dim=-1), torch.cat(sin_out, dim=-1)


# ------------------------------------------------------------------------------------- forward
def _lin(w, prefix, x):
    return F.linear(x, w[prefix + ".weight"], w.get(prefix + ".bias"))


def _ln(x, eps):
    return F.layer_norm(x, (x.shape[-1],), None, None, eps)


def attention_forward(w, pre, cfg: FluxConfig, x, ctx, cos, sin):
    """FluxAttention.forward, flux.py:165-231: per-head RMSNorm of q,k on each stream BEFORE the
    [txt;img] concatenation, interleaved rotary on the joint sequence with cos/sin cast to the
    activation dtype, attention, split and output projections (dual) or the raw joint output (single)."""
    H, D = cfg.num_heads, cfg.head_dim
    q, k, v = (t.unflatten(-1, (H, D)) for t in _lin(w, pre + "to_qkv", x).chunk(3, dim=-1))
    q = ops.rms_norm_head(q, w[pre + "norm_q.weight"], cfg.eps)
    k = ops.rms_norm_head(k, w[pre + "norm_k.weight"], cfg.eps)
    if ctx is not None:
        cq, ck, cv = (t.unflatten(-1, (H, D)) for t in _lin(w, pre + "add_kv_proj", ctx).chunk(3, dim=-1))
        cq = ops.rms_norm_head(cq, w[pre + "norm_added_q.weight"], cfg.eps)
        ck = ops.rms_norm_head(ck, w[pre + "norm_added_k.weight"], cfg.eps)
        q, k, v = torch.cat([cq, q], dim=1), torch.cat([ck, k], dim=1), torch.cat([cv, v], dim=1)
    c, s = cos.to(q.dtype), sin.to(q.dtype)
    q, k = ops.apply_rotary(q, c, s), ops.apply_rotary(k, c, s)
    o = ops.sdpa(q, k, v, 1.0 / (D ** 0.5)).flatten(2, 3).to(q.dtype)
    if ctx is None:
        return o
    n = ctx.shape[1]
    return _lin(w, pre + "to_out.0", o[:, n:]), _lin(w, pre + "to_add_out", o[:, :n])


def feed_forward(w, pre, x):
    """Linear -> GELU(tanh) -> Linear. flux.py:30-82."""
    return _lin(w, pre + "net.2", ops.gelu_tanh(_lin(w, pre + "net.0.proj", x)))


def dual_block_forward(w, i: int, cfg: FluxConfig, img, txt, temb, cos, sin):
    """FluxTransformerBlock.forward, flux.py:260-314. Returns (txt, img) like the reference."""
    pre = f"transformer_blocks.{i}."
    sh, sc, g_msa, sh_mlp, sc_mlp, g_mlp = _lin(w, pre + "norm1.linear", F.silu(temb)).chunk(6, dim=1)
    csh, csc, cg_msa, csh_mlp, csc_mlp, cg_mlp = _lin(w, pre + "norm1_context.linear", F.silu(temb)).chunk(6, dim=1)
    n_img = _ln(img, cfg.eps) * (1 + sc[:, None]) + sh[:, None]
    n_txt = _ln(txt, cfg.eps) * (1 + csc[:, None]) + csh[:, None]
    a_img, a_txt = attention_forward(w, pre + "attn.", cfg, n_img, n_txt, cos, sin)
    img = img + g_msa.unsqueeze(1) * a_img
    n2 = _ln(img, 1e-6) * (1 + sc_mlp[:, None]) + sh_mlp[:, None]
    img = img + g_mlp.unsqueeze(1) * feed_forward(w, pre + "ff.", n2)
    txt = txt + cg_msa.unsqueeze(1) * a_txt
    c2 = _ln(txt, 1e-6) * (1 + csc_mlp[:, None]) + csh_mlp[:, None]
    txt = txt + cg_mlp.unsqueeze(1) * feed_forward(w, pre + "ff_context.", c2)
    return txt, img


def single_block_forward(w, i: int, cfg: FluxConfig, img, txt, temb, cos, sin):
    """FluxSingleTransformerBlock.forward, flux.py:337-366: over the joint [txt;img] sequence,
    attention and the MLP branch run on the same modulated input; their outputs are concatenated on
    the channel axis, projected, gated and added back."""
    pre = f"single_transformer_blocks.{i}."
    n_txt = txt.shape[1]
    x = torch.cat([txt, img], dim=1)
    sh, sc, gate = _lin(w, pre + "norm.linear", F.silu(temb)).chunk(3, dim=1)
    n = _ln(x, 1e-6) * (1 + sc[:, None]) + sh[:, None]
    mlp = ops.gelu_tanh(_lin(w, pre + "proj_mlp", n))
    att = attention_forward(w, pre + "attn.", cfg, n, None, cos, sin)
    x = x + gate.unsqueeze(1) * _lin(w, pre + "proj_out", torch.cat([att, mlp], dim=2))
    return x[:, :n_txt], x[:, n_txt:]


def _mlp2(w, pre, x):
    return _lin(w, pre + ".linear_2", F.silu(_lin(w, pre + ".linear_1", x)))


def time_text_embed(w, cfg: FluxConfig, timestep, guidance, pooled):
    """CombinedTimestep(Guidance)TextProjEmbeddings (diffusers; call site flux.py:462-466, 537-541)."""
    t_emb = _mlp2(w, "time_text_embed.timestep_embedder",
                  ops.timestep_embedding(timestep, scale=1.0).to(pooled.dtype))
    if guidance is not None:
        t_emb = t_emb + _mlp2(w, "time_text_embed.guidance_embedder",
                              ops.timestep_embedding(guidance, scale=1.0).to(pooled.dtype))
    return t_emb + _mlp2(w, "time_text_embed.text_embedder", pooled)


def stem(w, cfg: FluxConfig, latents, text, pooled, timestep, guidance):
    """x_embedder, timestep (and guidance) x 1000 in the activation dtype, conditioning embedding,
    context_embedder. flux.py:531-542."""
    img = _lin(w, "x_embedder", latents)
    timestep = timestep.to(dtype=img.dtype) * 1000
    if guidance is not None:
        guidance = guidance.to(dtype=img.dtype) * 1000
    temb = time_text_embed(w, cfg, timestep, guidance, pooled)
    txt = _lin(w, "context_embedder", text)
    return img, txt, temb


def head(w, cfg: FluxConfig, img, temb):
    """norm_out (AdaLayerNormContinuous) + proj_out. flux.py:579-580."""
    x = ops.ada_layer_norm_continuous(img, temb, w["norm_out.linear.weight"], w.get("norm_out.linear.bias"), 1e-6)
    return _lin(w, "proj_out", x)


def modulated_input(w, cfg: FluxConfig, img, temb):
    """TeaCache's decision tensor for Flux: block 0's norm1 applied to the x_embedder output (the
    recipe sketched at cache/teacache/extractors.py:597-613)."""
    sh, sc = _lin(w, "transformer_blocks.0.norm1.linear", F.silu(temb)).chunk(6, dim=1)[:2]
    return _ln(img, cfg.eps) * (1 + sc[:, None]) + sh[:, None]


def transformer_forward(w, cfg: FluxConfig, latents, text, pooled, timestep, img_ids, txt_ids, guidance=None,
                        collect_blocks: bool = False):
    """FluxTransformer2DModel.forward, flux.py:496-586. latents [B,S_img,in], text [B,S_txt,J],
    pooled [B,P], timestep/guidance [B] (timestep in [0,1]), ids [S,3]."""
    img, txt, temb = stem(w, cfg, latents, text, pooled, timestep, guidance)
    cos, sin = flux_pos_embed(cfg, torch.cat((txt_ids, img_ids), dim=0))
    per_block = []
    for i in range(cfg.num_layers):
        txt, img = dual_block_forward(w, i, cfg, img, txt, temb, cos, sin)
        if collect_blocks:
            per_block.append((img, txt))
    for i in range(cfg.num_single_layers):
        txt, img = single_block_forward(w, i, cfg, img, txt, temb, cos, sin)
        if collect_blocks:
            per_block.append((img, txt))
    out = head(w, cfg, img, temb)
    return (out, per_block) if collect_blocks else out
