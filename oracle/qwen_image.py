"""Oracle restatement of the Qwen-Image dual-stream MMDiT forward (test infrastructure only).

Functional: weights live in a flat ``dict[str, Tensor]`` keyed with the reference's parameter names
(``transformer_blocks.3.attn.to_qkv.weight`` ...), so the same dict can be loaded into the product
modules. Reference file: ``vllm_omni/diffusion/models/qwen_image/qwen_image_transformer.py`` (cited
below as ``qit.py``).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import ops


@dataclass(frozen=True)
class QwenConfig:
    """Shape of the model. Defaults = Qwen-Image (qit.py:885-899)."""

    num_layers: int = 60
    num_heads: int = 24
    head_dim: int = 128
    in_channels: int = 64
    out_channels: int = 16
    patch_size: int = 2
    joint_attention_dim: int = 3584
    mlp_ratio: int = 4
    axes_dims_rope: tuple[int, int, int] = (16, 56, 56)
    theta: int = 10000
    eps: float = 1e-6

    @property
    def dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def proj_out_dim(self) -> int:
        return self.patch_size * self.patch_size * self.out_channels


def tiny_config() -> QwenConfig:
    """The CPU-runnable case: 2 blocks, hidden 256 = 4 heads x 64, MLP 4x, 2x2 patches of a 16-channel
    latent (64 input features), 256-wide text features."""
    return QwenConfig(num_layers=2, num_heads=4, head_dim=64, in_channels=64, out_channels=16,
                      joint_attention_dim=256, axes_dims_rope=(8, 28, 28))


# ------------------------------------------------------------------------------------- weights
def block_param_shapes(cfg: QwenConfig) -> dict[str, tuple[int, ...]]:
    C, D, F_ = cfg.dim, cfg.head_dim, cfg.dim * cfg.mlp_ratio
    return {
        "img_mod.1.weight": (6 * C, C), "img_mod.1.bias": (6 * C,),
        "txt_mod.1.weight": (6 * C, C), "txt_mod.1.bias": (6 * C,),
        "attn.to_qkv.weight": (3 * C, C), "attn.to_qkv.bias": (3 * C,),
        "attn.add_kv_proj.weight": (3 * C, C), "attn.add_kv_proj.bias": (3 * C,),
        "attn.norm_q.weight": (D,), "attn.norm_k.weight": (D,),
        "attn.norm_added_q.weight": (D,), "attn.norm_added_k.weight": (D,),
        "attn.to_out.weight": (C, C), "attn.to_out.bias": (C,),
        "attn.to_add_out.weight": (C, C), "attn.to_add_out.bias": (C,),
        "img_mlp.net.0.proj.weight": (F_, C), "img_mlp.net.0.proj.bias": (F_,),
        "img_mlp.net.2.weight": (C, F_), "img_mlp.net.2.bias": (C,),
        "txt_mlp.net.0.proj.weight": (F_, C), "txt_mlp.net.0.proj.bias": (F_,),
        "txt_mlp.net.2.weight": (C, F_), "txt_mlp.net.2.bias": (C,),
    }


def stem_param_shapes(cfg: QwenConfig) -> dict[str, tuple[int, ...]]:
    C = cfg.dim
    return {
        "img_in.weight": (C, cfg.in_channels), "img_in.bias": (C,),
        "txt_norm.weight": (cfg.joint_attention_dim,),
        "txt_in.weight": (C, cfg.joint_attention_dim), "txt_in.bias": (C,),
        "time_text_embed.timestep_embedder.linear_1.weight": (C, 256),
        "time_text_embed.timestep_embedder.linear_1.bias": (C,),
        "time_text_embed.timestep_embedder.linear_2.weight": (C, C),
        "time_text_embed.timestep_embedder.linear_2.bias": (C,),
        "norm_out.linear.weight": (2 * C, C), "norm_out.linear.bias": (2 * C,),
        "proj_out.weight": (cfg.proj_out_dim, C), "proj_out.bias": (cfg.proj_out_dim,),
    }


def init_params(cfg: QwenConfig, seed: int = 0, dtype: torch.dtype = torch.float32,
                std: float = 0.02, bias_std: float = 0.0, device: str = "cpu") -> dict[str, torch.Tensor]:
    """Synthetic weights: matrices N(0, std), RMSNorm weights 1, biases N(0, bias_std) (0 by default)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    out: dict[str, torch.Tensor] = {}

    def make(name: str, shape: tuple[int, ...]):
        if name.endswith("norm_q.weight") or name.endswith("norm_k.weight") or name.endswith("txt_norm.weight"):
            t = torch.ones(shape)
        elif name.endswith(".bias"):
            t = torch.randn(shape, generator=g) * bias_std if bias_std > 0 else torch.zeros(shape)
        else:
            t = torch.randn(shape, generator=g) * std
        out[name] = t.to(dtype).to(device)

    for n, s in stem_param_shapes(cfg).items():
        make(n, s)
    for i in range(cfg.num_layers):
        for n, s in block_param_shapes(cfg).items():
            make(f"transformer_blocks.{i}.{n}", s)
    return out


# ------------------------------------------------------------------------------------- rope tables
def _axis_freqs(index: torch.Tensor, dim: int, theta: int) -> torch.Tensor:
    """exp(i * pos * theta^(-2j/dim)), complex64. qit.py:322-335."""
    inv = 1.0 / torch.pow(theta, torch.arange(0, dim, 2).to(torch.float32).div(dim))
    ang = torch.outer(index.to(torch.float32), inv)
    return torch.polar(torch.ones_like(ang), ang)


def qwen_rope_freqs(cfg: QwenConfig, frame: int, height: int, width: int, txt_len: int):
    """(vid_freqs [F*H*W, D/2], txt_freqs [txt_len, D/2]) complex64 with scale_rope=True: rows/cols
    are centred ([-ceil(n/2) .. -1, 0 .. floor(n/2)-1]), frame index starts at 0, and text positions
    start at max(H//2, W//2) on all three axes. qit.py:298-396."""
    return qwen_rope_freqs_images(cfg, [(frame, height, width)], txt_len)


def qwen_rope_freqs_images(cfg: QwenConfig, shapes, txt_len: int, layer3d: bool = False):
    """The same tables for a sample made of several images (editing: source, then targets): image
    number ``idx`` takes frame positions idx .. idx+frame-1, its rows and columns are centred on its own
    grid, the token rows of all images are concatenated, and text positions start after the largest
    half-extent of any image. qit.py:340-396.

    ``layer3d`` (QwenEmbedLayer3DRope, qit.py:183-296, the layered-image variant): the LAST image of the
    list is the condition image and sits at frame position -1 instead of its list index, and the text
    start is also at least the number of layers (= len(shapes) - 1)."""
    a0, a1, a2 = cfg.axes_dims_rope
    pos = torch.arange(4096)
    neg = torch.arange(4096).flip(0) * -1 - 1
    pos_f = [_axis_freqs(pos, a, cfg.theta) for a in (a0, a1, a2)]
    neg_f = [_axis_freqs(neg, a, cfg.theta) for a in (a0, a1, a2)]
    vids, start = [], 0
    layer_num = len(shapes) - 1
    for idx, (frame, height, width) in enumerate(shapes):
        if layer3d and idx == layer_num:
            f_frame = neg_f[0][-1:].view(frame, 1, 1, -1).expand(frame, height, width, -1)  # frame must be 1
        else:
            f_frame = pos_f[0][idx:idx + frame].view(frame, 1, 1, -1).expand(frame, height, width, -1)
        f_h = torch.cat([neg_f[1][-(height - height // 2):], pos_f[1][: height // 2]], dim=0)
        f_h = f_h.view(1, height, 1, -1).expand(frame, height, width, -1)
        f_w = torch.cat([neg_f[2][-(width - width // 2):], pos_f[2][: width // 2]], dim=0)
        f_w = f_w.view(1, 1, width, -1).expand(frame, height, width, -1)
        vids.append(torch.cat([f_frame, f_h, f_w], dim=-1).reshape(frame * height * width, -1))
        start = max(start, height // 2, width // 2)
    if layer3d:
        start = max(start, layer_num)
    txt = torch.cat(pos_f, dim=1)[start:start + txt_len].contiguous()
    return torch.cat(vids, dim=0).contiguous(), txt


def modulate_index(img_shapes) -> torch.Tensor:
    """[B, S_img] int32 for the editing variant (``zero_cond_t``): 0 for the tokens of each sample's first
    image, 1 for those of every later image; ``img_shapes`` = per sample a list of (frame, height,
    width). qit.py:141-154."""
    rows = []
    for sample in img_shapes:
        first = sample[0][0] * sample[0][1] * sample[0][2]
        rest = sum(f * h * w for f, h, w in sample[1:])
        rows.append([0] * first + [1] * rest)
    return torch.tensor(rows, dtype=torch.int32)


# ------------------------------------------------------------------------------------- forward
def _lin(w, prefix, x):
    return F.linear(x, w[prefix + ".weight"], w.get(prefix + ".bias"))


def attention_forward(w, pre, cfg: QwenConfig, img, txt, vid_freqs, txt_freqs, key_mask=None):
    """QwenImageCrossAttention.forward, qit.py:561-661: fused QKV projections, per-head RMSNorm of
    q and k, interleaved rotary with cos/sin cast to the activation dtype, [txt;img] concatenation,
    joint attention, split, output projections."""
    H, D = cfg.num_heads, cfg.head_dim
    iq, ik, iv = _lin(w, pre + "to_qkv", img).chunk(3, dim=-1)
    tq, tk, tv = _lin(w, pre + "add_kv_proj", txt).chunk(3, dim=-1)
    iq, ik, iv, tq, tk, tv = (t.unflatten(-1, (H, D)) for t in (iq, ik, iv, tq, tk, tv))
    iq = ops.rms_norm_head(iq, w[pre + "norm_q.weight"], cfg.eps)
    ik = ops.rms_norm_head(ik, w[pre + "norm_k.weight"], cfg.eps)
    tq = ops.rms_norm_head(tq, w[pre + "norm_added_q.weight"], cfg.eps)
    tk = ops.rms_norm_head(tk, w[pre + "norm_added_k.weight"], cfg.eps)
    icos, isin = vid_freqs.real.to(iq.dtype), vid_freqs.imag.to(iq.dtype)
    tcos, tsin = txt_freqs.real.to(tq.dtype), txt_freqs.imag.to(tq.dtype)
    iq, ik = ops.apply_rotary(iq, icos, isin), ops.apply_rotary(ik, icos, isin)
    tq, tk = ops.apply_rotary(tq, tcos, tsin), ops.apply_rotary(tk, tcos, tsin)
    S_txt = txt.shape[1]
    jq = torch.cat([tq, iq], dim=1)
    jk = torch.cat([tk, ik], dim=1)
    jv = torch.cat([tv, iv], dim=1)
    o = ops.sdpa(jq, jk, jv, 1.0 / (D ** 0.5), key_mask).flatten(2, 3).to(jq.dtype)
    return _lin(w, pre + "to_out", o[:, S_txt:]), _lin(w, pre + "to_add_out", o[:, :S_txt])


def feed_forward(w, pre, x):
    """Linear -> GELU(tanh) -> Linear. qit.py:399-466."""
    return _lin(w, pre + "net.2", ops.gelu_tanh(_lin(w, pre + "net.0.proj", x)))


def block_forward(w, i: int, cfg: QwenConfig, img, txt, temb, vid_freqs, txt_freqs, key_mask=None,
                  modulate_index=None, zero_cond_t: bool = False):
    """QwenImageTransformerBlock.forward, qit.py:746-814. Returns (txt, img) like the reference.
    With ``zero_cond_t`` temb is [2B, C] (real timestep rows, then timestep-zero rows): the image stream
    picks per token through ``modulate_index``, the text stream uses the first half (qit.py:758-767)."""
    pre = f"transformer_blocks.{i}."
    img_mod = _lin(w, pre + "img_mod.1", F.silu(temb))
    if zero_cond_t:
        temb = torch.chunk(temb, 2, dim=0)[0]
    txt_mod = _lin(w, pre + "txt_mod.1", F.silu(temb))
    img_mod1, img_mod2 = img_mod.chunk(2, dim=-1)
    txt_mod1, txt_mod2 = txt_mod.chunk(2, dim=-1)
    img_n, img_g1 = ops.ada_layer_norm(img, img_mod1, modulate_index, cfg.eps)
    txt_n, txt_g1 = ops.ada_layer_norm(txt, txt_mod1, None, cfg.eps)
    img_a, txt_a = attention_forward(w, pre + "attn.", cfg, img_n, txt_n, vid_freqs, txt_freqs, key_mask)
    img = ops.gated_residual(img, img_a, img_g1)
    txt = ops.gated_residual(txt, txt_a, txt_g1)
    img_n2, img_g2 = ops.ada_layer_norm(img, img_mod2, modulate_index, cfg.eps)
    img = ops.gated_residual(img, feed_forward(w, pre + "img_mlp.", img_n2), img_g2)
    txt_n2, txt_g2 = ops.ada_layer_norm(txt, txt_mod2, None, cfg.eps)
    txt = ops.gated_residual(txt, feed_forward(w, pre + "txt_mlp.", txt_n2), txt_g2)
    return txt, img


def time_text_embed(w, timestep: torch.Tensor, dtype: torch.dtype, addition_t_cond=None) -> torch.Tensor:
    """QwenTimestepProjEmbeddings: sinusoid(256, scale 1000) -> Linear -> SiLU -> Linear, plus, when the
    checkpoint has ``addition_t_embedding`` (use_additional_t_cond), the row of that 2-entry table picked
    by ``addition_t_cond`` [N] (integers 0/1). qit.py:159-181."""
    proj = ops.timestep_embedding(timestep).to(dtype)
    h = _lin(w, "time_text_embed.timestep_embedder.linear_1", proj)
    out = _lin(w, "time_text_embed.timestep_embedder.linear_2", F.silu(h))
    table = w.get("time_text_embed.addition_t_embedding.weight")
    if table is not None:
        if addition_t_cond is None:
            raise ValueError("When additional_t_cond is True, addition_t_cond must be provided.")
        out = out + F.embedding(addition_t_cond, table).to(dtype)
    return out


def stem(w, cfg: QwenConfig, latents, text, timestep, addition_t_cond=None):
    """img_in, txt_norm, txt_in, time_text_embed. qit.py:1003-1024."""
    img = _lin(w, "img_in", latents)
    timestep = timestep.to(dtype=img.dtype)
    txt = ops.rms_norm_head(text, w["txt_norm.weight"], cfg.eps)
    txt = _lin(w, "txt_in", txt)
    temb = time_text_embed(w, timestep, img.dtype, addition_t_cond)
    return img, txt, temb


def head(w, cfg: QwenConfig, img, temb):
    """norm_out (AdaLayerNormContinuous) + proj_out. qit.py:1065-1066."""
    x = ops.ada_layer_norm_continuous(img, temb, w["norm_out.linear.weight"], w.get("norm_out.linear.bias"), cfg.eps)
    return _lin(w, "proj_out", x)


def modulated_input(w, cfg: QwenConfig, img, temb):
    """TeaCache's decision tensor: block 0's img_norm1 applied to the stem output.
    cache/teacache/extractors.py:210-213."""
    mod = _lin(w, "transformer_blocks.0.img_mod.1", F.silu(temb))
    return ops.ada_layer_norm(img, mod.chunk(2, dim=-1)[0], None, cfg.eps)[0]


def transformer_forward(w, cfg: QwenConfig, latents, text, timestep, img_shape, key_mask=None,
                        collect_blocks: bool = False, zero_cond_t: bool = False, layer3d_rope: bool = False,
                        addition_t_cond=None):
    """QwenImageTransformer2DModel.forward, qit.py:951-1071. latents [B,S_img,in], text [B,S_txt,J],
    timestep [B] in [0,1]; img_shape = (frame, height, width) of the patch grid, or a list of them when the
    sample is several images (rotary tables and, with ``zero_cond_t``, the per-token conditioning index
    follow the first sample's list, like the reference's). ``zero_cond_t``: the timestep is doubled to
    [t, 0*t] (qit.py:141-145), the head uses the first half of temb (qit.py:1062-1063)."""
    shapes = [tuple(img_shape)] if isinstance(img_shape[0], int) else [tuple(s) for s in img_shape]
    index = None
    if zero_cond_t:
        timestep = torch.cat([timestep, timestep * 0], dim=0)
        index = modulate_index([shapes] * latents.shape[0]).to(latents.device)
    img, txt, temb = stem(w, cfg, latents, text, timestep, addition_t_cond)
    vid_freqs, txt_freqs = qwen_rope_freqs_images(cfg, shapes, txt_len=text.shape[1], layer3d=layer3d_rope)
    per_block = []
    for i in range(cfg.num_layers):
        txt, img = block_forward(w, i, cfg, img, txt, temb, vid_freqs, txt_freqs, key_mask,
                                 modulate_index=index, zero_cond_t=zero_cond_t)
        if collect_blocks:
            per_block.append((img, txt))
    out = head(w, cfg, img, temb.chunk(2, dim=0)[0] if zero_cond_t else temb)
    return (out, per_block) if collect_blocks else out
