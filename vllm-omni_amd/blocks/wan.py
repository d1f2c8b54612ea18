"""Wan video DiT (text-to-video form) composed from the gfx950 kernels.

Module tree, parameter names and call signatures follow
vllm_omni/diffusion/models/wan2_2/wan2_2_transformer.py (``wan.py`` below) so a reference state dict
loads unchanged (fused ``attn1.to_qkv`` as after its ``load_weights`` stacking). Below the module
interfaces:

  * FP32LayerNorm + fp32 shift/scale modulation + cast (wan.py:659, 669) is one fused pass with
    float32 modulation rows; norm2 (fp32 LayerNorm with affine, wan.py:664) is the same kernel with
    LayerNorm weight/bias and no modulation;
  * whole-row fp32 RMSNorm of q and k + 3D rotary (wan.py:406-420) is one pass in row mode; V is read
    in place from the fused QKV projection;
  * the fp32 gated residuals (wan.py:661, 673) and the plain residual after cross-attention
    (wan.py:666) are one pass each;
  * the 6 modulation rows of every block (scale_shift_table + temb, wan.py:654-656) depend on the
    timestep only and are formed for all blocks in one small op per step;
  * self-attention (S x S) and cross-attention (S x 512, no rotary) both run on the flash kernel.

Per-token timesteps (``timestep`` [B,S], ``temb`` [B,S,6,C], wan.py:641-652): the table + temb sums are
never formed in memory; the modulation and gating kernels read the per-token 16-bit rows and add the
float32 table rows in registers. Image conditioning (``image_dim`` / ``added_kv_proj_dim``,
wan.py:224-248, 541-575): a second attention of the same queries over the embedded image tokens, added
to the text attention before the output projection.
"""

from __future__ import annotations

import math
from functools import lru_cache
from typing import Any

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import kernels
from .._lib import ODIT_NORM_ROW
from ..attention.layer import Attention
from .qwen_image import (ApproxGELU, QwenTimestepProjEmbeddings, TimestepEmbedding, Transformer2DModelOutput,
                         project_residual)


class DistributedRMSNorm(nn.Module):
    """Whole-row RMSNorm holder (wan.py:59-89); on one GPU the statistics are local. The arithmetic
    runs inside the fused q/k kernel; ``forward`` applies it stand-alone through the same kernel."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, S, C = x.shape
        x4 = x.view(B, S, 1, C) if x.is_contiguous() else x.contiguous().view(B, S, 1, C)
        out = torch.empty((B, S, 1, C), dtype=x.dtype, device=x.device)
        kernels.qknorm_rope(x4, None, None, out, None, None, self.weight, None, None, None, eps=self.eps,
                            norm_mode=ODIT_NORM_ROW)
        return out.view(B, S, C)


class WanRotary:
    """(freqs_cos, freqs_sin) [1,S,1,D] as the reference passes them (each value repeated twice along
    D) plus the float32 [S, D/2] tables the fused kernel reads: cos from the even, sin from the odd
    columns, as apply_rotary_emb_wan does (wan.py:50-55)."""

    def __init__(self, freqs_cos: torch.Tensor, freqs_sin: torch.Tensor):
        self.freqs_cos, self.freqs_sin = freqs_cos, freqs_sin
        self.cos32 = freqs_cos[0, :, 0, 0::2].float().contiguous()
        self.sin32 = freqs_sin[0, :, 0, 1::2].float().contiguous()

    def __iter__(self):
        return iter((self.freqs_cos, self.freqs_sin))


def _rotary(rotary_emb) -> WanRotary | None:
    if rotary_emb is None or isinstance(rotary_emb, WanRotary):
        return rotary_emb
    return WanRotary(*rotary_emb)


class WanRotaryPosEmbed(nn.Module):
    """3D rotary tables over the (frames, height, width) patch grid (wan.py:147-222)."""

    def __init__(self, attention_head_dim: int, patch_size: tuple[int, int, int], max_seq_len: int,
                 theta: float = 10000.0):
        super().__init__()
        self.attention_head_dim, self.patch_size, self.max_seq_len = attention_head_dim, tuple(patch_size), max_seq_len
        h_dim = w_dim = 2 * (attention_head_dim // 6)
        t_dim = attention_head_dim - h_dim - w_dim
        cos, sin = [], []
        for dim in (t_dim, h_dim, w_dim):
            inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
            ang = torch.outer(torch.arange(max_seq_len, dtype=torch.float64), inv)
            cos.append(ang.cos().float().repeat_interleave(2, dim=-1))
            sin.append(ang.sin().float().repeat_interleave(2, dim=-1))
        self.register_buffer("freqs_cos", torch.cat(cos, dim=1), persistent=False)
        self.register_buffer("freqs_sin", torch.cat(sin, dim=1), persistent=False)
        self._tables = lru_cache(maxsize=8)(self._build)

    def _build(self, ppf: int, pph: int, ppw: int, device: str) -> WanRotary:
        D = self.attention_head_dim
        sizes = [D - 2 * (D // 3), D // 3, D // 3]

        def grid(table):
            f, h, w = table.to(device).split(sizes, dim=1)
            return torch.cat([f[:ppf].view(ppf, 1, 1, -1).expand(ppf, pph, ppw, -1),
                              h[:pph].view(1, pph, 1, -1).expand(ppf, pph, ppw, -1),
                              w[:ppw].view(1, 1, ppw, -1).expand(ppf, pph, ppw, -1)],
                             dim=-1).reshape(1, ppf * pph * ppw, 1, -1)

        return WanRotary(grid(self.freqs_cos), grid(self.freqs_sin))

    def forward(self, hidden_states: torch.Tensor) -> WanRotary:
        _, _, nf, hh, ww = hidden_states.shape
        p_t, p_h, p_w = self.patch_size
        if max(nf // p_t, hh // p_h, ww // p_w) > self.max_seq_len:
            raise ValueError("patch grid exceeds rope_max_seq_len")
        return self._tables(nf // p_t, hh // p_h, ww // p_w, str(hidden_states.device))


class WanFeedForward(nn.Module):
    """net_0 = Linear + GELU(tanh), net_2 = Linear (wan.py:112-144)."""

    def __init__(self, dim: int, inner_dim: int, dim_out: int | None = None, bias: bool = True):
        super().__init__()
        self.net_0 = ApproxGELU(dim, inner_dim, bias=bias)
        self.net_1 = nn.Identity()
        self.net_2 = nn.Linear(inner_dim, dim_out or dim, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.net_2(self.net_0(x))


class WanSelfAttention(nn.Module):
    """wan.py:340-430."""

    def __init__(self, dim: int, num_heads: int, head_dim: int, eps: float = 1e-5):
        super().__init__()
        self.dim, self.num_heads, self.num_kv_heads, self.head_dim = dim, num_heads, num_heads, head_dim
        self.inner_dim = num_heads * head_dim
        self.to_qkv = nn.Linear(dim, 3 * self.inner_dim, bias=True)
        self.norm_q = DistributedRMSNorm(self.inner_dim, eps=eps)
        self.norm_k = DistributedRMSNorm(self.inner_dim, eps=eps)
        self.to_out = nn.Linear(self.inner_dim, dim, bias=True)
        self.attn = Attention(num_heads=num_heads, head_size=head_dim, num_kv_heads=num_heads,
                              softmax_scale=1.0 / (head_dim ** 0.5), causal=False)

    def forward(self, hidden_states: torch.Tensor, rotary_emb=None, residual: torch.Tensor | None = None,
                gate: torch.Tensor | None = None, pre=None) -> torch.Tensor:
        """With ``residual``: residual + gate * attention output (a new tensor), formed in the output
        projection's epilogue; ``pre`` = caller-made float32 (gate, gate * bias) rows."""
        rot = _rotary(rotary_emb)
        B, S, _ = hidden_states.shape
        H, D = self.num_heads, self.head_dim
        qkv = self.to_qkv(hidden_states).view(B, S, 3, H, D)
        q = torch.empty((B, S, H, D), dtype=qkv.dtype, device=qkv.device)
        k = torch.empty_like(q)
        cos, sin = (rot.cos32, rot.sin32) if rot is not None else (None, None)
        kernels.qknorm_rope(qkv[:, :, 0], qkv[:, :, 1], None, q, k, None, self.norm_q.weight, self.norm_k.weight,
                            cos, sin, eps=self.norm_q.eps, norm_mode=ODIT_NORM_ROW)
        o = self.attn(q, k, qkv[:, :, 2]).flatten(2, 3)
        if residual is not None:
            return project_residual(self.to_out, o, residual, gate, pre=pre)
        return self.to_out(o)


class WanCrossAttention(nn.Module):
    """wan.py:433-586. With ``added_kv_proj_dim`` the context is [image tokens; ``text_context_len`` text
    tokens] (the reference hardcodes 512, wan.py:540-543) and the image tokens get their own k/v
    projections, k norm and softmax."""

    def __init__(self, dim: int, num_heads: int, head_dim: int, eps: float = 1e-5,
                 added_kv_proj_dim: int | None = None, text_context_len: int = 512):
        super().__init__()
        self.added_kv_proj_dim, self.text_context_len = added_kv_proj_dim, text_context_len
        if added_kv_proj_dim is not None:
            self.add_k_proj = nn.Linear(added_kv_proj_dim, num_heads * head_dim, bias=True)
            self.add_v_proj = nn.Linear(added_kv_proj_dim, num_heads * head_dim, bias=True)
            self.norm_added_k = DistributedRMSNorm(num_heads * head_dim, eps=eps)
        else:
            self.add_k_proj = self.add_v_proj = self.norm_added_k = None
        self.dim, self.num_heads, self.head_dim = dim, num_heads, head_dim
        self.inner_dim = num_heads * head_dim
        self.to_q = nn.Linear(dim, self.inner_dim, bias=True)
        self.to_k = nn.Linear(dim, self.inner_dim, bias=True)
        self.to_v = nn.Linear(dim, self.inner_dim, bias=True)
        self.norm_q = DistributedRMSNorm(self.inner_dim, eps=eps)
        self.norm_k = DistributedRMSNorm(self.inner_dim, eps=eps)
        self.to_out = nn.Linear(self.inner_dim, dim, bias=True)
        self.attn = Attention(num_heads=num_heads, head_size=head_dim, num_kv_heads=num_heads,
                              softmax_scale=1.0 / (head_dim ** 0.5), causal=False)

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor,
                residual: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        """With ``residual``: residual + attention output (written to ``out`` when given)."""
        B, S, _ = hidden_states.shape
        H, D = self.num_heads, self.head_dim
        ctx_img = None
        if self.add_k_proj is not None:
            n_img = encoder_hidden_states.shape[1] - self.text_context_len
            if n_img <= 0:
                raise ValueError(f"image-conditioned cross-attention expects image tokens in front of "
                                 f"{self.text_context_len} text tokens, got {encoder_hidden_states.shape[1]} in all")
            ctx_img, encoder_hidden_states = encoder_hidden_states[:, :n_img], encoder_hidden_states[:, n_img:]
        T = encoder_hidden_states.shape[1]

        def normed(x_in: torch.Tensor, norm: DistributedRMSNorm) -> torch.Tensor:
            out_ = torch.empty_like(x_in)
            kernels.qknorm_rope(x_in, None, None, out_, None, None, norm.weight, None, None, None,
                                eps=norm.eps, norm_mode=ODIT_NORM_ROW)
            return out_

        q = normed(self.to_q(hidden_states).view(B, S, H, D), self.norm_q)
        k = normed(self.to_k(encoder_hidden_states).view(B, T, H, D), self.norm_k)
        v = self.to_v(encoder_hidden_states).view(B, T, H, D)
        o = self.attn(q, k, v).flatten(2, 3)
        if ctx_img is not None:
            k_img = normed(self.add_k_proj(ctx_img).view(B, n_img, H, D), self.norm_added_k)
            v_img = self.add_v_proj(ctx_img).view(B, n_img, H, D)
            o_img = self.attn(q, k_img, v_img).flatten(2, 3)
            o = kernels.gated_residual(o, o_img, None, out=o)  # two separate softmaxes, summed (wan.py:577-579)
        if residual is not None:
            return project_residual(self.to_out, o, residual, None, out=out)
        return self.to_out(o)


class FP32LayerNorm(nn.LayerNorm):
    """Parameter holder with the reference's name and shapes; evaluated by the fused kernel."""


class WanTransformerBlock(nn.Module):
    """wan.py:589-675: self-attention, cross-attention, feed-forward."""

    def __init__(self, dim: int, ffn_dim: int, num_heads: int, eps: float = 1e-6,
                 added_kv_proj_dim: int | None = None, cross_attn_norm: bool = False,
                 text_context_len: int = 512):
        super().__init__()
        head_dim = dim // num_heads
        self.eps = eps
        self.norm1 = FP32LayerNorm(dim, eps, elementwise_affine=False)
        self.attn1 = WanSelfAttention(dim=dim, num_heads=num_heads, head_dim=head_dim, eps=eps)
        self.attn2 = WanCrossAttention(dim=dim, num_heads=num_heads, head_dim=head_dim, eps=eps,
                                       added_kv_proj_dim=added_kv_proj_dim, text_context_len=text_context_len)
        self.norm2 = FP32LayerNorm(dim, eps, elementwise_affine=True) if cross_attn_norm else nn.Identity()
        self.ffn = WanFeedForward(dim=dim, inner_dim=ffn_dim, dim_out=dim)
        self.norm3 = FP32LayerNorm(dim, eps, elementwise_affine=False)
        self.scale_shift_table = nn.Parameter(torch.randn(1, 6, dim) / dim ** 0.5)
        self._ln2_f32: tuple[int, torch.Tensor, torch.Tensor] | None = None
        self._table_f32: tuple[tuple, torch.Tensor] | None = None

    def _table(self) -> torch.Tensor:
        """float32 [6, C] copy of scale_shift_table, refreshed when the parameter changes."""
        p = self.scale_shift_table
        tag = (p._version, p.data_ptr(), p.device)
        if self._table_f32 is None or self._table_f32[0] != tag:
            self._table_f32 = (tag, p.detach().float().reshape(6, -1).contiguous())
        return self._table_f32[1]

    def _norm2_affine(self):
        """float32 copies of norm2's weight/bias, refreshed when the parameters change."""
        w, b = self.norm2.weight, self.norm2.bias
        tag = (w._version, b._version, w.data_ptr(), w.device)
        if self._ln2_f32 is None or self._ln2_f32[0] != tag:
            self._ln2_f32 = (tag, w.detach().float().contiguous(), b.detach().float().contiguous())
        return self._ln2_f32[1], self._ln2_f32[2]

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
                rotary_emb=None, mod: torch.Tensor | None = None,
                gate_bias: torch.Tensor | None = None) -> torch.Tensor:
        """``mod`` = float32 [B, 6, C] = scale_shift_table + temb when the caller formed it for all
        blocks at once; otherwise it is formed here as in the reference. ``gate_bias`` = float32 [B, 2, C]:
        the two gates times the biases of the projections they scale (attn1.to_out, ffn.net_2)."""
        if mod is None and temb.ndim == 4:
            return self._forward_per_token(hidden_states, encoder_hidden_states, temb, rotary_emb)
        if mod is None:
            mod = self.scale_shift_table + temb.float()
        shift_msa, scale_msa, gate_msa, c_shift, c_scale, c_gate = (mod[:, i] for i in range(6))
        x = hidden_states
        n = kernels.adaln_modulate(x, shift_msa, scale_msa, eps=self.eps)
        pre1 = (gate_msa, gate_bias[:, 0]) if gate_bias is not None else None
        pre2 = (c_gate, gate_bias[:, 1]) if gate_bias is not None else None
        x = self.attn1(n, rotary_emb, residual=x, gate=gate_msa, pre=pre1)   # new tensor: the input is not written
        if isinstance(self.norm2, nn.Identity):
            n = x
        else:
            lw, lb = self._norm2_affine()
            n = kernels.adaln_modulate(x, None, None, eps=self.eps, ln_weight=lw, ln_bias=lb, out=n)
        x = self.attn2(n, encoder_hidden_states, residual=x, out=x)
        n = kernels.adaln_modulate(x, c_shift, c_scale, eps=self.eps, out=n if n is not x else None)
        return project_residual(self.ffn.net_2, self.ffn.net_0(n), x, c_gate, out=x, pre=pre2)


    def _forward_per_token(self, x: torch.Tensor, ctx: torch.Tensor, temb: torch.Tensor, rotary_emb) -> torch.Tensor:
        """temb [B, S, 6, C] (wan.py:641-652): every token has its own six modulation rows. The reference
        forms table + temb.float() as six float32 [B,S,C] tensors per block; here the kernels read the
        rows of ``temb`` as they are and add the float32 table row in registers — the same fp32 sum."""
        if temb.shape[:2] != x.shape[:2] or temb.shape[2] != 6 or temb.stride(-1) != 1:
            raise ValueError(f"per-token temb must be [B,S,6,C] matching x, got {tuple(temb.shape)}")
        tab = self._table()
        row = lambda i: temb[:, :, i]  # noqa: E731  ([B,S,C] view, token stride 6C)
        n = kernels.adaln_modulate(x, row(0), row(1), eps=self.eps, shift_bias=tab[0], scale_bias=tab[1])
        a = self.attn1(n, rotary_emb)
        x = kernels.gated_residual(x, a, row(2), gate_bias=tab[2])          # new tensor: the input is not written
        if isinstance(self.norm2, nn.Identity):
            n = x
        else:
            lw, lb = self._norm2_affine()
            n = kernels.adaln_modulate(x, None, None, eps=self.eps, ln_weight=lw, ln_bias=lb, out=n)
        x = self.attn2(n, ctx, residual=x, out=x)
        n = kernels.adaln_modulate(x, row(3), row(4), eps=self.eps, shift_bias=tab[3], scale_bias=tab[4],
                                   out=n if n is not x else None)
        return kernels.gated_residual(x, self.ffn(n), row(5), out=x, gate_bias=tab[5])


class PixArtAlphaTextProjection(nn.Module):
    """Linear -> GELU(tanh) -> Linear (the ``act_fn="gelu_tanh"`` form, wan.py:269)."""

    def __init__(self, in_features: int, hidden_size: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_features, hidden_size)
        self.linear_2 = nn.Linear(hidden_size, hidden_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = self.linear_1(x)
        return self.linear_2(kernels.gelu_tanh(y, out=y))


class _ImageFeedForward(nn.Module):
    """diffusers ``FeedForward(mult=1, activation_fn="gelu")`` of the image embedder: parameter names
    ``net.0.proj`` / ``net.2``, exact (erf) GELU between them."""

    def __init__(self, dim: int, dim_out: int):
        super().__init__()
        act = nn.Module()
        act.proj = nn.Linear(dim, dim)
        self.net = nn.ModuleList([act, nn.Identity(), nn.Linear(dim, dim_out)])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.net[2](F.gelu(self.net[0].proj(x)))


class WanImageEmbedding(nn.Module):
    """wan.py:224-248: (learned positions over the joined first/last-frame tokens) -> LayerNorm -> MLP ->
    LayerNorm on the image-encoder tokens; a few hundred rows once per step. The two norms are the
    reference's default-constructed FP32LayerNorm: eps 1e-5 with an affine pair."""

    def __init__(self, in_features: int, out_features: int, pos_embed_seq_len: int | None = None):
        super().__init__()
        self.norm1 = FP32LayerNorm(in_features)
        self.ff = _ImageFeedForward(in_features, out_features)
        self.norm2 = FP32LayerNorm(out_features)
        self.pos_embed = (nn.Parameter(torch.zeros(1, pos_embed_seq_len, in_features))
                          if pos_embed_seq_len is not None else None)

    @staticmethod
    def _norm(ln: nn.LayerNorm, x: torch.Tensor) -> torch.Tensor:
        return kernels.adaln_modulate(x, None, None, eps=ln.eps, ln_weight=ln.weight.detach().float().contiguous(),
                                      ln_bias=ln.bias.detach().float().contiguous())

    def forward(self, encoder_hidden_states_image: torch.Tensor) -> torch.Tensor:
        x = encoder_hidden_states_image
        if self.pos_embed is not None:
            _, n, e = x.shape
            x = x.reshape(-1, 2 * n, e) + self.pos_embed
        return self._norm(self.norm2, self.ff(self._norm(self.norm1, x.contiguous())))


class WanTimeTextImageEmbedding(nn.Module):
    """wan.py:251-296."""

    def __init__(self, dim: int, time_freq_dim: int, time_proj_dim: int, text_embed_dim: int,
                 image_embed_dim: int | None = None, pos_embed_seq_len: int | None = None):
        super().__init__()
        self.time_freq_dim = time_freq_dim
        self.time_embedder = TimestepEmbedding(time_freq_dim, dim)
        self.time_proj = nn.Linear(dim, time_proj_dim)
        self.text_embedder = PixArtAlphaTextProjection(text_embed_dim, dim)
        self.image_embedder = (WanImageEmbedding(image_embed_dim, dim, pos_embed_seq_len=pos_embed_seq_len)
                               if image_embed_dim is not None else None)

    def forward(self, timestep: torch.Tensor, encoder_hidden_states: torch.Tensor,
                encoder_hidden_states_image: torch.Tensor | None = None, timestep_seq_len: int | None = None):
        """timestep [B] -> temb [B,C], timestep_proj [B,6C]; flattened per-token timesteps [B*S] with
        ``timestep_seq_len`` = S -> temb [B,S,C], timestep_proj [B,S,6C] (wan.py:282-296)."""
        t = QwenTimestepProjEmbeddings.time_proj(timestep, dim=self.time_freq_dim, scale=1.0)
        if timestep_seq_len is not None:
            t = t.unflatten(0, (-1, timestep_seq_len))
        t = t.to(self.time_embedder.linear_1.weight.dtype)
        temb = self.time_embedder(t).type_as(encoder_hidden_states)
        timestep_proj = self.time_proj(kernels.silu(temb))
        image = None
        if encoder_hidden_states_image is not None:
            if self.image_embedder is None:
                raise ValueError("image features given to a model built without image_dim")
            image = self.image_embedder(encoder_hidden_states_image)
        return temb, timestep_proj, self.text_embedder(encoder_hidden_states), image


class OutputScaleShiftPrepare(nn.Module):
    def __init__(self, inner_dim: int):
        super().__init__()
        self.scale_shift_table = nn.Parameter(torch.randn(1, 2, inner_dim) / inner_dim ** 0.5)

    def forward(self, temb: torch.Tensor):
        """temb [B,C] -> shift, scale [B,C]; per-token temb [B,S,C] -> [B,S,C] each (wan.py:324-337)."""
        if temb.ndim == 3:
            shift, scale = (self.scale_shift_table.unsqueeze(0) + temb.unsqueeze(2)).chunk(2, dim=2)
            return shift.squeeze(2), scale.squeeze(2)
        shift, scale = (self.scale_shift_table + temb.unsqueeze(1)).chunk(2, dim=1)
        return shift.squeeze(1), scale.squeeze(1)


class WanTransformer3DModel(nn.Module):
    """wan.py:678-910: patch embedding, condition embeddings, N blocks, modulated output norm,
    projection, unpatchify. ``prepare`` / ``run_blocks`` / ``finish`` split it into stages."""

    _repeated_blocks = ["WanTransformerBlock"]
    packed_modules_mapping = {"to_qkv": ["to_q", "to_k", "to_v"]}

    def __init__(self, patch_size: tuple[int, int, int] = (1, 2, 2), num_attention_heads: int = 40,
                 attention_head_dim: int = 128, in_channels: int = 16, out_channels: int = 16, text_dim: int = 4096,
                 freq_dim: int = 256, ffn_dim: int = 13824, num_layers: int = 40, cross_attn_norm: bool = True,
                 eps: float = 1e-6, image_dim: int | None = None, added_kv_proj_dim: int | None = None,
                 rope_max_seq_len: int = 1024, pos_embed_seq_len: int | None = None,
                 text_context_len: int = 512):
        super().__init__()
        # attribute bag with the constructor arguments, as pipelines read it (wan.py:775-797)
        self.config = type("Config", (), dict(
            patch_size=patch_size, num_attention_heads=num_attention_heads, attention_head_dim=attention_head_dim,
            in_channels=in_channels, out_channels=out_channels, text_dim=text_dim, freq_dim=freq_dim, ffn_dim=ffn_dim,
            num_layers=num_layers, cross_attn_norm=cross_attn_norm, eps=eps, image_dim=image_dim,
            added_kv_proj_dim=added_kv_proj_dim, rope_max_seq_len=rope_max_seq_len,
            pos_embed_seq_len=pos_embed_seq_len))()
        inner_dim = num_attention_heads * attention_head_dim
        self.patch_size, self.inner_dim, self.eps = tuple(patch_size), inner_dim, eps
        self.in_channels, self.out_channels = in_channels, out_channels or in_channels
        self.rope = WanRotaryPosEmbed(attention_head_dim, patch_size, rope_max_seq_len)
        self.patch_embedding = nn.Conv3d(in_channels, inner_dim, kernel_size=patch_size, stride=patch_size)
        self.condition_embedder = WanTimeTextImageEmbedding(dim=inner_dim, time_freq_dim=freq_dim,
                                                            time_proj_dim=inner_dim * 6, text_embed_dim=text_dim,
                                                            image_embed_dim=image_dim,
                                                            pos_embed_seq_len=pos_embed_seq_len)
        self.blocks = nn.ModuleList([
            WanTransformerBlock(inner_dim, ffn_dim, num_attention_heads, eps, added_kv_proj_dim, cross_attn_norm,
                                text_context_len=text_context_len)
            for _ in range(num_layers)])
        self.norm_out = FP32LayerNorm(inner_dim, eps, elementwise_affine=False)
        self.proj_out = nn.Linear(inner_dim, self.out_channels * math.prod(patch_size))
        self.output_scale_shift_prepare = OutputScaleShiftPrepare(inner_dim)

    @property
    def dtype(self) -> torch.dtype:
        return next(self.parameters()).dtype

    def patchify(self, video: torch.Tensor) -> torch.Tensor:
        """Conv3d with kernel = stride = patch is a Linear over non-overlapping patches: gather each
        patch's (C_in, p_t, p_h, p_w) values into a row and run ONE dense GEMM (the conv path would pick
        an implicit-GEMM kernel for a shape that is a plain matrix product)."""
        B, Cin, nf, hh, ww = video.shape
        p_t, p_h, p_w = self.patch_size
        x = video.view(B, Cin, nf // p_t, p_t, hh // p_h, p_h, ww // p_w, p_w)
        x = x.permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(B, -1, Cin * p_t * p_h * p_w)
        return F.linear(x, self.patch_embedding.weight.view(self.inner_dim, -1), self.patch_embedding.bias)

    def prepare(self, hidden_states: torch.Tensor, timestep: torch.Tensor, encoder_hidden_states: torch.Tensor,
                encoder_hidden_states_image: torch.Tensor | None = None):
        """-> tokens, context, temb, timestep_proj ([B,6,C], or [B,S,6,C] for per-token timesteps [B,S]),
        rotary. Image tokens, when given, are embedded and put in front of the text tokens (wan.py:878-879)."""
        rotary = self.rope(hidden_states)
        x = self.patchify(hidden_states)
        ts_len = None
        if timestep.ndim == 2:
            if timestep.shape[1] != x.shape[1]:
                raise ValueError(f"per-token timesteps need one value per token: {timestep.shape[1]} vs {x.shape[1]}")
            ts_len, timestep = timestep.shape[1], timestep.flatten()
        temb, tproj, ctx, image = self.condition_embedder(timestep, encoder_hidden_states,
                                                          encoder_hidden_states_image, timestep_seq_len=ts_len)
        if image is not None:
            ctx = torch.cat([image, ctx], dim=1)
        return x, ctx, temb, tproj.unflatten(tproj.ndim - 1, (6, -1)), rotary

    def all_modulations(self, timestep_proj: torch.Tensor) -> torch.Tensor:
        """float32 [L, B, 6, C]: every block's scale_shift_table + temb in one op."""
        tables = torch.cat([blk.scale_shift_table for blk in self.blocks], dim=0)  # [L, 6, C]
        return tables.unsqueeze(1) + timestep_proj.float().unsqueeze(0)

    def run_blocks(self, x, ctx, timestep_proj, rotary):
        if timestep_proj.ndim == 4:  # per-token timesteps: the blocks read the rows of timestep_proj directly
            for block in self.blocks:
                x = block(x, ctx, timestep_proj, rotary)
            return x
        mods = self.all_modulations(timestep_proj)
        gb = None
        if x.dtype != torch.float32:  # gates (rows 2 and 5) times the biases they scale, [L, B, 2, C]
            biases = torch.stack([torch.stack([blk.attn1.to_out.bias, blk.ffn.net_2.bias]) for blk in self.blocks])
            gb = mods[:, :, 2::3] * biases.float().unsqueeze(1)
        for i, block in enumerate(self.blocks):
            x = block(x, ctx, None, rotary, mod=mods[i], gate_bias=None if gb is None else gb[i])
        return x

    def finish(self, x: torch.Tensor, temb: torch.Tensor, grid: tuple[int, int, int], return_dict: bool = True):
        shift, scale = self.output_scale_shift_prepare(temb)
        if shift.ndim == 2:
            shift, scale = shift.contiguous(), scale.contiguous()
        x = kernels.adaln_modulate(x, shift, scale, eps=self.eps)
        x = self.proj_out(x)
        p_t, p_h, p_w = self.patch_size
        x = x.reshape(x.shape[0], *grid, p_t, p_h, p_w, -1).permute(0, 7, 1, 4, 2, 5, 3, 6)
        out = x.flatten(6, 7).flatten(4, 5).flatten(2, 3)
        return Transformer2DModelOutput(sample=out) if return_dict else (out,)

    def forward(self, hidden_states: torch.Tensor, timestep: torch.Tensor, encoder_hidden_states: torch.Tensor,
                encoder_hidden_states_image: torch.Tensor | None = None, return_dict: bool = True,
                attention_kwargs: dict[str, Any] | None = None):
        _, _, nf, hh, ww = hidden_states.shape
        p_t, p_h, p_w = self.patch_size
        x, ctx, temb, tproj, rotary = self.prepare(hidden_states, timestep, encoder_hidden_states,
                                                   encoder_hidden_states_image)
        x = self.run_blocks(x, ctx, tproj, rotary)
        return self.finish(x, temb, (nf // p_t, hh // p_h, ww // p_w), return_dict=return_dict)

    def load_weights(self, weights) -> set[str]:
        """Load a diffusers-layout checkpoint stream (wan.py:907-990): attn1 q/k/v are stacked, attn2's
        stay separate, ``ffn.net.N`` maps to ``ffn.net_N``, ``to_out.0`` to ``to_out``, the top-level
        ``scale_shift_table`` to ``output_scale_shift_prepare.scale_shift_table``; unknown names are skipped."""
        from .weights import load_stacked_weights

        mapping = [(".attn1.to_qkv", ".attn1.to_q", "q"), (".attn1.to_qkv", ".attn1.to_k", "k"),
                   (".attn1.to_qkv", ".attn1.to_v", "v")]
        renames = ((".ffn.net.0.", ".ffn.net_0."), (".ffn.net.2.", ".ffn.net_2."), (".to_out.0.", ".to_out."))
        return load_stacked_weights(self, weights, mapping, substring_renames=renames,
                                    exact_renames={"scale_shift_table": "output_scale_shift_prepare.scale_shift_table"},
                                    skip_unknown=True)

    def load_flat_state(self, weights: dict[str, torch.Tensor]) -> None:
        """Load a flat name->tensor dict keyed with the reference's parameter names."""
        own = dict(self.named_parameters())
        missing = [k for k in own if k not in weights]
        extra = [k for k in weights if k not in own]
        if missing or extra:
            raise KeyError(f"state mismatch: missing {missing[:4]}..., unexpected {extra[:4]}...")
        with torch.no_grad():
            for k, p in own.items():
                p.copy_(weights[k].to(device=p.device, dtype=p.dtype))
