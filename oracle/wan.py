"""Oracle restatement of the Wan video DiT forward (test infrastructure only).

Functional: weights are a flat ``dict[str, Tensor]`` keyed with the reference's parameter names.
Reference file: ``vllm_omni/diffusion/models/wan2_2/wan2_2_transformer.py`` (``wan.py`` below).
Covered: the T2V path (``temb`` [B, 6, C]), the per-token-timestep TI2V form (``timestep`` [B, S],
``temb`` [B, S, 6, C], wan.py:641-652, 864-876) and the I2V image branch (image embedder wan.py:224-248,
second cross-attention over the image context wan.py:541-575).

Third-party arithmetic on this path (diffusers>=0.36.0, absent from the reference tree — **parity
unpinned** at that boundary, upstream conventions adopted): ``FP32LayerNorm`` (layer_norm evaluated
in fp32, cast back to the input dtype; an ``nn.LayerNorm`` subclass, so eps 1e-5 and an affine pair
where the reference passes no arguments), ``Timesteps`` / ``TimestepEmbedding``,
``PixArtAlphaTextProjection(act_fn="gelu_tanh")`` (Linear, GELU-tanh, Linear),
``FeedForward(mult=1, activation_fn="gelu")`` of the image embedder (Linear, exact GELU, Linear; parameter
names ``net.0.proj`` / ``net.2``).
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import ops


@dataclass(frozen=True)
class WanConfig:
    """Defaults = Wan2.1-14B (wan.py:753-770)."""

    patch_size: tuple[int, int, int] = (1, 2, 2)
    num_heads: int = 40
    head_dim: int = 128
    in_channels: int = 16
    out_channels: int = 16
    text_dim: int = 4096
    freq_dim: int = 256
    ffn_dim: int = 13824
    num_layers: int = 40
    cross_attn_norm: bool = True
    eps: float = 1e-6
    rope_max_seq_len: int = 1024
    theta: float = 10000.0
    image_dim: int | None = None            # I2V: width of the image-encoder features
    added_kv_proj_dim: int | None = None    # I2V: width of the embedded image context (= dim in the checkpoints)
    pos_embed_seq_len: int | None = None    # first+last-frame variant: learned positions over 2 x 257 tokens
    text_context_len: int = 512             # the reference hardcodes 512 text tokens (wan.py:540-543)

    @property
    def dim(self) -> int:
        return self.num_heads * self.head_dim


def tiny_config() -> WanConfig:
    """CPU-runnable case: 2 blocks, hidden 256 = 4 heads x 64, FFN 640, 96-wide text features."""
    return WanConfig(num_heads=4, head_dim=64, in_channels=8, out_channels=8, text_dim=96, ffn_dim=640,
                     num_layers=2, rope_max_seq_len=64)


# ------------------------------------------------------------------------------------- weights
def block_param_shapes(cfg: WanConfig) -> dict[str, tuple[int, ...]]:
    C, F_ = cfg.dim, cfg.ffn_dim
    out = {
        "scale_shift_table": (1, 6, C),
        "attn1.to_qkv.weight": (3 * C, C), "attn1.to_qkv.bias": (3 * C,),
        "attn1.norm_q.weight": (C,), "attn1.norm_k.weight": (C,),
        "attn1.to_out.weight": (C, C), "attn1.to_out.bias": (C,),
        "attn2.to_q.weight": (C, C), "attn2.to_q.bias": (C,),
        "attn2.to_k.weight": (C, C), "attn2.to_k.bias": (C,),
        "attn2.to_v.weight": (C, C), "attn2.to_v.bias": (C,),
        "attn2.norm_q.weight": (C,), "attn2.norm_k.weight": (C,),
        "attn2.to_out.weight": (C, C), "attn2.to_out.bias": (C,),
        "ffn.net_0.proj.weight": (F_, C), "ffn.net_0.proj.bias": (F_,),
        "ffn.net_2.weight": (C, F_), "ffn.net_2.bias": (C,),
    }
    if cfg.cross_attn_norm:
        out.update({"norm2.weight": (C,), "norm2.bias": (C,)})
    if cfg.added_kv_proj_dim is not None:
        A = cfg.added_kv_proj_dim
        out.update({"attn2.add_k_proj.weight": (C, A), "attn2.add_k_proj.bias": (C,),
                    "attn2.add_v_proj.weight": (C, A), "attn2.add_v_proj.bias": (C,),
                    "attn2.norm_added_k.weight": (C,)})
    return out


def stem_param_shapes(cfg: WanConfig) -> dict[str, tuple[int, ...]]:
    C = cfg.dim
    img = {}
    if cfg.image_dim is not None:
        I, p = cfg.image_dim, "condition_embedder.image_embedder."
        img = {p + "norm1.weight": (I,), p + "norm1.bias": (I,),
               p + "ff.net.0.proj.weight": (I, I), p + "ff.net.0.proj.bias": (I,),
               p + "ff.net.2.weight": (C, I), p + "ff.net.2.bias": (C,),
               p + "norm2.weight": (C,), p + "norm2.bias": (C,)}
        if cfg.pos_embed_seq_len is not None:
            img[p + "pos_embed"] = (1, cfg.pos_embed_seq_len, I)
    return {
        **img,
        "patch_embedding.weight": (C, cfg.in_channels, *cfg.patch_size), "patch_embedding.bias": (C,),
        "condition_embedder.time_embedder.linear_1.weight": (C, cfg.freq_dim),
        "condition_embedder.time_embedder.linear_1.bias": (C,),
        "condition_embedder.time_embedder.linear_2.weight": (C, C),
        "condition_embedder.time_embedder.linear_2.bias": (C,),
        "condition_embedder.time_proj.weight": (6 * C, C), "condition_embedder.time_proj.bias": (6 * C,),
        "condition_embedder.text_embedder.linear_1.weight": (C, cfg.text_dim),
        "condition_embedder.text_embedder.linear_1.bias": (C,),
        "condition_embedder.text_embedder.linear_2.weight": (C, C),
        "condition_embedder.text_embedder.linear_2.bias": (C,),
        "output_scale_shift_prepare.scale_shift_table": (1, 2, C),
        "proj_out.weight": (cfg.out_channels * math.prod(cfg.patch_size), C),
        "proj_out.bias": (cfg.out_channels * math.prod(cfg.patch_size),),
    }


def init_params(cfg: WanConfig, seed: int = 0, dtype: torch.dtype = torch.float32, std: float = 0.02,
                bias_std: float = 0.0, norm_jitter: float = 0.0) -> dict[str, torch.Tensor]:
    """Matrices N(0, std); scale_shift tables N(0,1)/sqrt(C) as the reference initialises them
    (wan.py:631, 330); RMSNorm / LayerNorm weights 1 (+ N(0, norm_jitter)); biases N(0, bias_std)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    out: dict[str, torch.Tensor] = {}

    def make(name: str, shape: tuple[int, ...]):
        if name.endswith("scale_shift_table"):
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name.endswith(("norm_q.weight", "norm_k.weight", "norm_added_k.weight", "norm1.weight", "norm2.weight")):
            t = torch.ones(shape) + (torch.randn(shape, generator=g) * norm_jitter if norm_jitter > 0 else 0)
        elif name.endswith(".bias"):
            t = torch.randn(shape, generator=g) * bias_std if bias_std > 0 else torch.zeros(shape)
        else:
            t = torch.randn(shape, generator=g) * std
        out[name] = t.to(dtype)

    for n, s in stem_param_shapes(cfg).items():
        make(n, s)
    for i in range(cfg.num_layers):
        for n, s in block_param_shapes(cfg).items():
            make(f"blocks.{i}.{n}", s)
    return out


# ------------------------------------------------------------------------------------- rope
def wan_rope_tables(cfg: WanConfig, frames: int, height: int, width: int):
    """WanRotaryPosEmbed, wan.py:147-222. Per axis (t, h, w) of widths (D - 4*(D//6), 2*(D//6),
    2*(D//6)): angle = pos * theta^(-2j/dim) in float64, cos/sin cast to float32 and each repeated
    twice along the last axis; the three axes are concatenated per token of the (frames, height,
    width) patch grid. Returns (cos, sin) of shape [1, F*H*W, 1, D]."""
    D = cfg.head_dim
    h_dim = w_dim = 2 * (D // 6)
    t_dim = D - h_dim - w_dim
    cos_ax, sin_ax = [], []
    for dim in (t_dim, h_dim, w_dim):
        inv = 1.0 / (cfg.theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
        ang = torch.outer(torch.arange(cfg.rope_max_seq_len, dtype=torch.float64), inv)
        cos_ax.append(ang.cos().float().repeat_interleave(2, dim=-1))
        sin_ax.append(ang.sin().float().repeat_interleave(2, dim=-1))

    def grid(ax):
        f = ax[0][:frames].view(frames, 1, 1, -1).expand(frames, height, width, -1)
        h = ax[1][:height].view(1, height, 1, -1).expand(frames, height, width, -1)
        w = ax[2][:width].view(1, 1, width, -1).expand(frames, height, width, -1)
        return torch.cat([f, h, w], dim=-1).reshape(1, frames * height * width, 1, -1)

    return grid(cos_ax), grid(sin_ax)


# ------------------------------------------------------------------------------------- forward
def _lin(w, prefix, x):
    return F.linear(x, w[prefix + ".weight"], w.get(prefix + ".bias"))


def fp32_layer_norm(x, weight, bias, eps):
    """diffusers FP32LayerNorm: layer_norm in fp32, result cast back to x.dtype."""
    return F.layer_norm(x.float(), (x.shape[-1],), None if weight is None else weight.float(),
                        None if bias is None else bias.float(), eps).to(x.dtype)


def self_attention(w, pre, cfg: WanConfig, x, cos, sin):
    """WanSelfAttention.forward, wan.py:394-430: fused QKV, whole-row fp32 RMSNorm of q and k, 3D
    rotary, attention, output projection."""
    H, D = cfg.num_heads, cfg.head_dim
    q, k, v = _lin(w, pre + "to_qkv", x).chunk(3, dim=-1)
    q = ops.rms_norm_row_fp32(q, w[pre + "norm_q.weight"], cfg.eps).unflatten(2, (H, D))
    k = ops.rms_norm_row_fp32(k, w[pre + "norm_k.weight"], cfg.eps).unflatten(2, (H, D))
    v = v.unflatten(2, (H, D))
    q, k = ops.apply_rotary_wan(q, cos, sin), ops.apply_rotary_wan(k, cos, sin)
    o = ops.sdpa(q, k, v, 1.0 / (D ** 0.5)).flatten(2, 3).type_as(q)
    return _lin(w, pre + "to_out", o)


def cross_attention(w, pre, cfg: WanConfig, x, ctx):
    """WanCrossAttention.forward, wan.py:532-586: q from the video tokens, k/v from the text tokens,
    whole-row RMSNorm on q and k, no rotary. With the image branch (``added_kv_proj_dim``) the context is
    [image tokens; 512 text tokens]: a second, separate softmax attention of the same q over the image
    tokens (own k/v projections, own k norm) is added to the text attention before the output projection."""
    H, D = cfg.num_heads, cfg.head_dim
    ctx_img = None
    if cfg.added_kv_proj_dim is not None:
        n_img = ctx.shape[1] - cfg.text_context_len
        ctx_img, ctx = ctx[:, :n_img], ctx[:, n_img:]
    q = ops.rms_norm_row_fp32(_lin(w, pre + "to_q", x), w[pre + "norm_q.weight"], cfg.eps).unflatten(2, (H, D))
    k = ops.rms_norm_row_fp32(_lin(w, pre + "to_k", ctx), w[pre + "norm_k.weight"], cfg.eps).unflatten(2, (H, D))
    v = _lin(w, pre + "to_v", ctx).unflatten(2, (H, D))
    o = ops.sdpa(q, k, v, 1.0 / (D ** 0.5)).flatten(2, 3).type_as(q)
    if ctx_img is not None:
        ki = ops.rms_norm_row_fp32(_lin(w, pre + "add_k_proj", ctx_img), w[pre + "norm_added_k.weight"], cfg.eps)
        vi = _lin(w, pre + "add_v_proj", ctx_img)
        oi = ops.sdpa(q, ki.unflatten(2, (H, D)), vi.unflatten(2, (H, D)), 1.0 / (D ** 0.5))
        o = o + oi.flatten(2, 3).type_as(q)
    return _lin(w, pre + "to_out", o)


def block_forward(w, i: int, cfg: WanConfig, x, ctx, temb6, cos, sin):
    """WanTransformerBlock.forward, wan.py:634-675. temb6 [B, 6, C], or [B, S, 6, C] with per-token
    timesteps; modulation and the gated residuals are evaluated in fp32 and cast back."""
    pre = f"blocks.{i}."
    if temb6.ndim == 4:
        mods = (w[pre + "scale_shift_table"].unsqueeze(0) + temb6.float()).chunk(6, dim=2)
        sh, sc, g, csh, csc, cg = (m.squeeze(2) for m in mods)
    else:
        sh, sc, g, csh, csc, cg = (w[pre + "scale_shift_table"] + temb6.float()).chunk(6, dim=1)
    n = (fp32_layer_norm(x.float(), None, None, cfg.eps) * (1 + sc) + sh).type_as(x)
    a = self_attention(w, pre + "attn1.", cfg, n, cos, sin)
    x = (x.float() + a * g).type_as(x)
    if cfg.cross_attn_norm:
        n = fp32_layer_norm(x.float(), w[pre + "norm2.weight"], w[pre + "norm2.bias"], cfg.eps).type_as(x)
    else:
        n = x
    x = x + cross_attention(w, pre + "attn2.", cfg, n, ctx)
    n = (fp32_layer_norm(x.float(), None, None, cfg.eps) * (1 + csc) + csh).type_as(x)
    ff = _lin(w, pre + "ffn.net_2", ops.gelu_tanh(_lin(w, pre + "ffn.net_0.proj", n)))
    return (x.float() + ff.float() * cg).type_as(x)


def image_embedder(w, cfg: WanConfig, image_feats):
    """WanImageEmbedding.forward, wan.py:239-248: (optional learned positions over the first+last frame
    pair, rows of two consecutive batch entries joined) -> FP32LayerNorm -> Linear, GELU, Linear ->
    FP32LayerNorm. The two norms are built without arguments: eps 1e-5, affine."""
    pre = "condition_embedder.image_embedder."
    x = image_feats
    if pre + "pos_embed" in w:
        _, n, e = x.shape
        x = x.view(-1, 2 * n, e) + w[pre + "pos_embed"]
    x = fp32_layer_norm(x, w[pre + "norm1.weight"], w[pre + "norm1.bias"], 1e-5)
    x = _lin(w, pre + "ff.net.2", F.gelu(_lin(w, pre + "ff.net.0.proj", x)))
    return fp32_layer_norm(x, w[pre + "norm2.weight"], w[pre + "norm2.bias"], 1e-5)


def condition_embedder(w, cfg: WanConfig, timestep, text, timestep_seq_len: int | None = None):
    """WanTimeTextImageEmbedding.forward, wan.py:275-296 -> (temb [B,C], timestep_proj [B,6C], text);
    with ``timestep_seq_len`` the flattened [B*S] timesteps give temb [B,S,C] and timestep_proj [B,S,6C]."""
    pre = "condition_embedder."
    t = ops.timestep_embedding(timestep, dim=cfg.freq_dim, scale=1.0)
    if timestep_seq_len is not None:
        t = t.unflatten(0, (-1, timestep_seq_len))
    t = t.to(w[pre + "time_embedder.linear_1.weight"].dtype)
    temb = _lin(w, pre + "time_embedder.linear_2", F.silu(_lin(w, pre + "time_embedder.linear_1", t))).type_as(text)
    tproj = _lin(w, pre + "time_proj", F.silu(temb))
    ctx = _lin(w, pre + "text_embedder.linear_2", ops.gelu_tanh(_lin(w, pre + "text_embedder.linear_1", text)))
    return temb, tproj, ctx


def stem(w, cfg: WanConfig, video, timestep, text, image_feats=None):
    """Patch embedding (Conv3d with kernel = stride = patch), flatten to tokens, condition embeddings.
    wan.py:852-881. video [B, C_in, F, H, W]; timestep [B] or, per token, [B, S]; with ``image_feats``
    the embedded image tokens are put in front of the text tokens (wan.py:878-879)."""
    x = F.conv3d(video, w["patch_embedding.weight"], w["patch_embedding.bias"], stride=cfg.patch_size)
    x = x.flatten(2).transpose(1, 2)
    ts_len = None
    if timestep.ndim == 2:
        ts_len, timestep = timestep.shape[1], timestep.flatten()
    temb, tproj, ctx = condition_embedder(w, cfg, timestep, text, ts_len)
    if image_feats is not None:
        ctx = torch.cat([image_embedder(w, cfg, image_feats), ctx], dim=1)
    return x, temb, tproj.unflatten(tproj.ndim - 1, (6, -1)), ctx


def head(w, cfg: WanConfig, x, temb, grid, batch):
    """Output modulation (shift, scale = table + temb), fp32 LayerNorm, projection, unpatchify.
    wan.py:887-905; per-token temb [B,S,C] gives per-token shift and scale (wan.py:324-331)."""
    table = w["output_scale_shift_prepare.scale_shift_table"]
    if temb.ndim == 3:
        shift, scale = ((table.unsqueeze(0) + temb.unsqueeze(2)).chunk(2, dim=2))
        shift, scale = shift.squeeze(2), scale.squeeze(2)
        x = (fp32_layer_norm(x.float(), None, None, cfg.eps) * (1 + scale) + shift).type_as(x)
        return _unpatchify(cfg, _lin(w, "proj_out", x), grid, batch)
    shift, scale = (table + temb.unsqueeze(1)).chunk(2, dim=1)
    x = (fp32_layer_norm(x.float(), None, None, cfg.eps) * (1 + scale) + shift).type_as(x)
    return _unpatchify(cfg, _lin(w, "proj_out", x), grid, batch)


def _unpatchify(cfg: WanConfig, x, grid, batch):
    p_t, p_h, p_w = cfg.patch_size
    x = x.reshape(batch, *grid, p_t, p_h, p_w, -1).permute(0, 7, 1, 4, 2, 5, 3, 6)
    return x.flatten(6, 7).flatten(4, 5).flatten(2, 3)


def transformer_forward(w, cfg: WanConfig, video, timestep, text, collect_blocks: bool = False,
                        image_feats=None):
    """WanTransformer3DModel.forward, wan.py:838-910."""
    B, _, nf, hh, ww = video.shape
    p_t, p_h, p_w = cfg.patch_size
    grid = (nf // p_t, hh // p_h, ww // p_w)
    cos, sin = wan_rope_tables(cfg, *grid)
    x, temb, temb6, ctx = stem(w, cfg, video, timestep, text, image_feats)
    per_block = []
    for i in range(cfg.num_layers):
        x = block_forward(w, i, cfg, x, ctx, temb6, cos, sin)
        if collect_blocks:
            per_block.append(x)
    out = head(w, cfg, x, temb, grid, B)
    return (out, per_block) if collect_blocks else out
