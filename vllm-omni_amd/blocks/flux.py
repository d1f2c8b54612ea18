"""Flux dual-stream + single-stream MMDiT composed from the gfx950 kernels.

Module tree, parameter names and call signatures follow
vllm_omni/diffusion/models/flux/flux_transformer.py (``flux.py`` below) so a reference state dict
loads unchanged (fused ``to_qkv`` / ``add_kv_proj`` as after its ``load_weights`` stacking,
flux.py:588-596). What differs sits below the module interfaces:

  * per-head QK-RMSNorm, rotary and the [txt;img] concatenation are one fused pass per stream that
    writes into the joint buffers (flux.py:181-208); text rows read the (identity) head of the joint
    cos/sin table, image rows its tail;
  * AdaLayerNormZero / ZeroSingle / norm2+modulate are the fused LayerNorm+modulate kernel; their
    SiLU+Linear projections depend on ``temb`` only and can run for all blocks at once
    (``fuse_modulation``);
  * the single-stream blocks keep ONE joint [B, S_txt+S_img, C] tensor across all 38 blocks instead of
    cat/split per block, read V straight out of the fused QKV projection, and replace
    ``proj_out(cat([attn, mlp]))`` (flux.py:356-358) by two accumulating GEMMs on the two column
    ranges of the same weight, so the 5C-wide concatenation is never materialised.
"""

from __future__ import annotations

from typing import Any

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import kernels
from .._lib import ODIT_NORM_HEAD
from ..attention.backends.abstract import AttentionMetadata
from ..attention.layer import Attention
from ..layers.rmsnorm import RMSNorm
from ..layers.rope import RotaryEmbedding
from .qwen_image import (AdaLayerNormContinuous, FeedForward, QwenTimestepProjEmbeddings, TimestepEmbedding,
                         Transformer2DModelOutput, _require_single_gpu, project_residual)


class FluxRotary:
    """(cos, sin) of the joint [txt;img] sequence as the reference passes them, plus the float32
    [S, D/2] tables the fused kernel reads."""

    def __init__(self, cos: torch.Tensor, sin: torch.Tensor):
        self.cos, self.sin = cos, sin
        self.cos32, self.sin32 = cos.float().contiguous(), sin.float().contiguous()

    def __iter__(self):
        return iter((self.cos, self.sin))


def _rotary(image_rotary_emb) -> FluxRotary | None:
    if image_rotary_emb is None or isinstance(image_rotary_emb, FluxRotary):
        return image_rotary_emb
    return FluxRotary(*image_rotary_emb)


class AdaLayerNormZero(nn.Module):
    """diffusers AdaLayerNormZero as Flux uses it (flux.py:240-241, 269-273): emb = Linear(SiLU(temb)),
    chunk(6) = shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp."""

    def __init__(self, embedding_dim: int, eps: float = 1e-6, ref_rounding: bool = False):
        super().__init__()
        self.linear = nn.Linear(embedding_dim, 6 * embedding_dim, bias=True)
        self.eps, self.ref_rounding = eps, ref_rounding

    def forward(self, x: torch.Tensor, emb: torch.Tensor | None = None, mod: torch.Tensor | None = None):
        if mod is None:
            mod = self.linear(kernels.silu(emb))
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = mod.chunk(6, dim=1)
        x = kernels.adaln_modulate(x, shift_msa, scale_msa, eps=self.eps, ref_rounding=self.ref_rounding)
        return x, gate_msa, shift_mlp, scale_mlp, gate_mlp


class AdaLayerNormZeroSingle(nn.Module):
    """diffusers AdaLayerNormZeroSingle (flux.py:322, 350): chunk(3) = shift, scale, gate."""

    def __init__(self, embedding_dim: int, eps: float = 1e-6, ref_rounding: bool = False):
        super().__init__()
        self.linear = nn.Linear(embedding_dim, 3 * embedding_dim, bias=True)
        self.eps, self.ref_rounding = eps, ref_rounding

    def forward(self, x: torch.Tensor, emb: torch.Tensor | None = None, mod: torch.Tensor | None = None):
        if mod is None:
            mod = self.linear(kernels.silu(emb))
        shift, scale, gate = mod.chunk(3, dim=1)
        return kernels.adaln_modulate(x, shift, scale, eps=self.eps, ref_rounding=self.ref_rounding), gate


class FluxAttention(nn.Module):
    """flux.py:85-231. With ``added_kv_proj_dim`` the joint attention of a dual block (returns
    (hidden, encoder) after the output projections); with ``pre_only`` the attention of a single
    block over an already joint sequence (returns the raw [B,S,C] attention output)."""

    def __init__(self, query_dim: int, heads: int = 8, dim_head: int = 64, bias: bool = False,
                 added_kv_proj_dim: int | None = None, added_proj_bias: bool | None = True, out_bias: bool = True,
                 eps: float = 1e-5, out_dim: int | None = None, context_pre_only: bool | None = None,
                 pre_only: bool = False, ref_rounding: bool = False):
        super().__init__()
        self.head_dim = dim_head
        self.inner_dim = out_dim if out_dim is not None else dim_head * heads
        self.query_dim = query_dim
        self.out_dim = out_dim if out_dim is not None else query_dim
        self.heads = out_dim // dim_head if out_dim is not None else heads
        self.pre_only, self.added_kv_proj_dim, self.eps = pre_only, added_kv_proj_dim, eps
        self.norm_q = RMSNorm(dim_head, eps=eps)
        self.norm_k = RMSNorm(dim_head, eps=eps)
        self.to_qkv = nn.Linear(query_dim, 3 * self.inner_dim, bias=bias)
        if not pre_only:
            self.to_out = nn.ModuleList([nn.Linear(self.inner_dim, self.out_dim, bias=out_bias), nn.Dropout(0.0)])
        if added_kv_proj_dim is not None:
            self.norm_added_q = RMSNorm(dim_head, eps=eps)
            self.norm_added_k = RMSNorm(dim_head, eps=eps)
            self.add_kv_proj = nn.Linear(added_kv_proj_dim, 3 * self.inner_dim, bias=bool(added_proj_bias))
            self.to_add_out = nn.Linear(self.inner_dim, query_dim, bias=out_bias)
        self.rope = RotaryEmbedding(is_neox_style=False)
        self.attn = Attention(num_heads=self.heads, head_size=dim_head, softmax_scale=1.0 / (dim_head ** 0.5),
                              causal=False, num_kv_heads=self.heads)
        self.ref_rounding = ref_rounding

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor | None = None,
                image_rotary_emb=None, residuals=None, **kwargs):
        """``residuals`` = (residual, gate, context_residual, context_gate[, pre, context_pre]) (dual blocks
        only): return residual + gate * projection for both streams instead of the bare projections; the
        ``pre`` pairs are caller-made float32 (gate, gate * bias) rows."""
        rot = _rotary(image_rotary_emb)
        B, S_x, _ = hidden_states.shape
        H, D = self.heads, self.head_dim
        rr = self.ref_rounding
        qkv = self.to_qkv(hidden_states).view(B, S_x, 3, H, D)
        if self.added_kv_proj_dim is None:
            # single stream: q,k normalised+rotated into dense buffers, v read in place from the projection
            q = torch.empty((B, S_x, H, D), dtype=qkv.dtype, device=qkv.device)
            k = torch.empty_like(q)
            cos, sin = (rot.cos32, rot.sin32) if rot is not None else (None, None)
            kernels.qknorm_rope(qkv[:, :, 0], qkv[:, :, 1], None, q, k, None, self.norm_q.weight,
                                self.norm_k.weight, cos, sin, eps=self.eps, norm_mode=ODIT_NORM_HEAD,
                                ref_rounding=rr)
            return self.attn(q, k, qkv[:, :, 2]).flatten(2, 3)
        S_c = encoder_hidden_states.shape[1]
        cqkv = self.add_kv_proj(encoder_hidden_states).view(B, S_c, 3, H, D)
        S = S_c + S_x
        jq = torch.empty((B, S, H, D), dtype=qkv.dtype, device=qkv.device)
        jk = torch.empty_like(jq)
        # v is only moved, never changed: read in place from the two projections when the kernel can
        v_in_place = S_c % 64 == 0 and qkv.dtype != torch.float32 and not rr
        jv = None if v_in_place else torch.empty_like(jq)
        tc = ts = ic = isn = None
        if rot is not None:
            tc, ts, ic, isn = rot.cos32[:S_c], rot.sin32[:S_c], rot.cos32[S_c:], rot.sin32[S_c:]
        # context rows [0, S_c) and image rows [S_c, S) of the joint buffers, one launch for both streams
        kernels.qknorm_rope_pair(
            (cqkv[:, :, 0], cqkv[:, :, 1], None if v_in_place else cqkv[:, :, 2],
             self.norm_added_q.weight, self.norm_added_k.weight, tc, ts, 0),
            (qkv[:, :, 0], qkv[:, :, 1], None if v_in_place else qkv[:, :, 2],
             self.norm_q.weight, self.norm_k.weight, ic, isn, S_c),
            jq, jk, jv, eps=self.eps, norm_mode=ODIT_NORM_HEAD, ref_rounding=rr)
        meta = AttentionMetadata(output_split=S_c)
        if v_in_place:
            jv, meta.value_tail = cqkv[:, :, 2], qkv[:, :, 2]
        ctx_attn, x_attn = self.attn(jq, jk, jv, meta)
        if residuals is not None:
            res, gate, c_res, c_gate = residuals[:4]
            pre, c_pre = residuals[4:] if len(residuals) == 6 else (None, None)
            return (project_residual(self.to_out[0], x_attn.flatten(2, 3), res, gate, ref_rounding=rr, pre=pre),
                    project_residual(self.to_add_out, ctx_attn.flatten(2, 3), c_res, c_gate, ref_rounding=rr,
                                     pre=c_pre))
        return self.to_out[0](x_attn.flatten(2, 3)), self.to_add_out(ctx_attn.flatten(2, 3))


class FluxTransformerBlock(nn.Module):
    """One dual-stream block (flux.py:234-314); returns (encoder_hidden_states, hidden_states)."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, qk_norm: str = "rms_norm",
                 eps: float = 1e-6, ref_rounding: bool = False):
        super().__init__()
        rr = ref_rounding
        self.norm1 = AdaLayerNormZero(dim, ref_rounding=rr)
        self.norm1_context = AdaLayerNormZero(dim, ref_rounding=rr)
        self.attn = FluxAttention(query_dim=dim, added_kv_proj_dim=dim, dim_head=attention_head_dim,
                                  heads=num_attention_heads, out_dim=dim, context_pre_only=False, bias=True,
                                  eps=eps, ref_rounding=rr)
        self.norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff = FeedForward(dim=dim, dim_out=dim, fused=not rr)
        self.norm2_context = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff_context = FeedForward(dim=dim, dim_out=dim, fused=not rr)
        self.ref_rounding = rr

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
                image_rotary_emb=None, joint_attention_kwargs: dict[str, Any] | None = None,
                mod_params: tuple[torch.Tensor, torch.Tensor] | None = None,
                gate_rows: tuple[torch.Tensor, torch.Tensor] | None = None):
        """``mod_params`` = (norm1 [B,6C], norm1_context [B,6C]) when the caller projected ``temb`` for
        all blocks at once; otherwise they are computed here as in the reference. ``gate_rows`` = float32
        (gates, gates * biases), each [B, 2 (hidden, context), 2 (attention, feed-forward), C]."""
        rr = self.ref_rounding
        pre = [[None, None], [None, None]]
        if gate_rows is not None:
            pre = [[(gate_rows[0][:, s, j], gate_rows[1][:, s, j]) for j in range(2)] for s in range(2)]
        m_x, m_c = mod_params if mod_params is not None else (None, None)
        # the two streams' norms are one launch each time (norm1 / norm1_context, norm2 / norm2_context)
        if m_x is None:
            m_x = self.norm1.linear(kernels.silu(temb))
        if m_c is None:
            m_c = self.norm1_context.linear(kernels.silu(temb))
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = m_x.chunk(6, dim=1)
        c_shift_msa, c_scale_msa, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = m_c.chunk(6, dim=1)
        n_x, n_c = kernels.adaln_modulate_pair((hidden_states, shift_msa, scale_msa),
                                               (encoder_hidden_states, c_shift_msa, c_scale_msa),
                                               eps=self.norm1.eps, ref_rounding=rr)
        # inputs are never written (callers such as TeaCache keep them to form residuals): the attention
        # residuals land in new tensors, the feed-forward residuals then update those in place
        hidden_states, encoder_hidden_states = self.attn(
            hidden_states=n_x, encoder_hidden_states=n_c, image_rotary_emb=image_rotary_emb,
            residuals=(hidden_states, gate_msa, encoder_hidden_states, c_gate_msa, pre[0][0], pre[1][0]),
            **(joint_attention_kwargs or {}))
        n2, c2 = kernels.adaln_modulate_pair((hidden_states, shift_mlp, scale_mlp),
                                             (encoder_hidden_states, c_shift_mlp, c_scale_mlp),
                                             eps=self.norm2.eps, ref_rounding=rr)
        hidden_states = self.ff.forward_residual(n2, hidden_states, gate_mlp, out=hidden_states, ref_rounding=rr,
                                                 pre=pre[0][1])
        encoder_hidden_states = self.ff_context.forward_residual(c2, encoder_hidden_states, c_gate_mlp,
                                                                 out=encoder_hidden_states, ref_rounding=rr,
                                                                 pre=pre[1][1])
        if encoder_hidden_states.dtype == torch.float16:
            encoder_hidden_states = encoder_hidden_states.clip(-65504, 65504)
        return encoder_hidden_states, hidden_states


class FluxSingleTransformerBlock(nn.Module):
    """One single-stream block (flux.py:317-366). ``forward`` keeps the reference signature
    (two streams in, two streams out); ``forward_joint`` is the same block on an already joint
    sequence, which the model uses to avoid a concatenation and a split per block."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, mlp_ratio: float = 4.0,
                 ref_rounding: bool = False):
        super().__init__()
        self.dim = dim
        self.mlp_hidden_dim = int(dim * mlp_ratio)
        self.norm = AdaLayerNormZeroSingle(dim, ref_rounding=ref_rounding)
        self.proj_mlp = nn.Linear(dim, self.mlp_hidden_dim)
        self.proj_out = nn.Linear(dim + self.mlp_hidden_dim, dim)
        self.attn = FluxAttention(query_dim=dim, dim_head=attention_head_dim, heads=num_attention_heads,
                                  out_dim=dim, bias=True, eps=1e-6, pre_only=True, ref_rounding=ref_rounding)
        self.ref_rounding = ref_rounding

    def forward_joint(self, x: torch.Tensor, temb: torch.Tensor, image_rotary_emb=None,
                      mod: torch.Tensor | None = None, in_place: bool = False,
                      gate_rows: tuple[torch.Tensor, torch.Tensor] | None = None) -> torch.Tensor:
        """``gate_rows`` = float32 (gate [B,C], gate * proj_out.bias [B,C]) made by the caller."""
        B, S, C = x.shape
        n, gate = self.norm(x, emb=temb, mod=mod)
        fused = not self.ref_rounding and x.dtype != torch.float32
        if fused:
            mlp = kernels.linear(n, self.proj_mlp.weight, self.proj_mlp.bias, activation="gelu_tanh")
        else:
            mlp = self.proj_mlp(n)
            mlp = kernels.gelu_tanh(mlp, out=mlp)
        att = self.attn(hidden_states=n, image_rotary_emb=image_rotary_emb)
        # gate * proj_out(cat([att, mlp], -1)) + x as two GEMMs over the two column ranges of the weight,
        # each accumulating onto the residual stream through its epilogue
        w = self.proj_out.weight
        if fused and gate_rows is not None:
            out = kernels.linear(mlp, w[:, C:], None, residual=x, gate=gate_rows[0], gate_bias=gate_rows[1],
                                 prescaled=True, out=x if in_place else None)
            out = kernels.linear(att, w[:, :C], None, residual=out, gate=gate_rows[0], prescaled=True, out=out)
        elif fused:
            out = kernels.linear(mlp, w[:, C:], self.proj_out.bias, residual=x, gate=gate, out=x if in_place else None)
            out = kernels.linear(att, w[:, :C], None, residual=out, gate=gate, out=out)
        else:
            y = F.linear(mlp.view(B * S, -1), w[:, C:], self.proj_out.bias)
            y.addmm_(att.reshape(B * S, C), w[:, :C].t())
            out = kernels.gated_residual(x, y.view(B, S, C), gate, out=x if in_place else None,
                                         ref_rounding=self.ref_rounding)
        if out.dtype == torch.float16:
            out = out.clip(-65504, 65504)
        return out

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
                image_rotary_emb=None, joint_attention_kwargs: dict[str, Any] | None = None):
        n_txt = encoder_hidden_states.shape[1]
        x = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        x = self.forward_joint(x, temb, image_rotary_emb, in_place=True)
        return x[:, :n_txt], x[:, n_txt:]


class FluxPosEmbed(nn.Module):
    """Per-axis rotary tables from position ids, evaluated in float64 (flux.py:369-396)."""

    def __init__(self, theta: int, axes_dim: list[int]):
        super().__init__()
        self.theta, self.axes_dim = theta, list(axes_dim)

    def forward(self, ids: torch.Tensor):
        pos = ids.float()
        cos_out, sin_out = [], []
        for i, d in enumerate(self.axes_dim):
            inv = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float64, device=ids.device)[: d // 2] / d))
            ang = torch.outer(pos[:, i].to(torch.float64), inv)
            cos_out.append(torch.cos(ang))
            sin_out.append(torch.sin(ang))
        return torch.cat(cos_out, dim=-1), torch.cat(sin_out, dim=-1)


class PixArtAlphaTextProjection(nn.Module):
    def __init__(self, in_features: int, hidden_size: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_features, hidden_size)
        self.linear_2 = nn.Linear(hidden_size, hidden_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.linear_2(kernels.silu(self.linear_1(x)))


class CombinedTimestepGuidanceTextProjEmbeddings(nn.Module):
    """Timestep (+ guidance) sinusoid -> MLP, pooled text -> MLP, summed (flux.py:462-466, 537-541)."""

    def __init__(self, embedding_dim: int, pooled_projection_dim: int, guidance_embeds: bool = True):
        super().__init__()
        self.timestep_embedder = TimestepEmbedding(256, embedding_dim)
        if guidance_embeds:
            self.guidance_embedder = TimestepEmbedding(256, embedding_dim)
        self.text_embedder = PixArtAlphaTextProjection(pooled_projection_dim, embedding_dim)

    def forward(self, timestep: torch.Tensor, guidance: torch.Tensor | None, pooled_projection: torch.Tensor):
        proj = QwenTimestepProjEmbeddings.time_proj
        emb = self.timestep_embedder(proj(timestep, scale=1.0).to(pooled_projection.dtype))
        if guidance is not None:
            emb = emb + self.guidance_embedder(proj(guidance, scale=1.0).to(pooled_projection.dtype))
        return emb + self.text_embedder(pooled_projection)


class FluxTransformer2DModel(nn.Module):
    """Stem, dual blocks, single blocks, head (flux.py:399-586). ``prepare`` / ``run_blocks`` /
    ``finish`` are the stages TeaCache calls separately."""

    _repeated_blocks = ["FluxTransformerBlock"]

    def __init__(self, od_config: Any | None = None, patch_size: int = 1, in_channels: int = 64,
                 out_channels: int | None = None, num_layers: int = 19, num_single_layers: int = 38,
                 attention_head_dim: int = 128, num_attention_heads: int = 24, joint_attention_dim: int = 4096,
                 pooled_projection_dim: int = 768, guidance_embeds: bool = True,
                 axes_dims_rope: tuple[int, int, int] = (16, 56, 56), ref_rounding: bool = False):
        """The reference's arguments (flux.py:436-450), ``od_config`` included: its ``tf_model_config.num_layers``
        overrides ``num_layers`` as there, its ``parallel_config`` has to describe one GPU."""
        super().__init__()
        _require_single_gpu(od_config)
        tf_cfg = getattr(od_config, "tf_model_config", None)
        if tf_cfg is not None and getattr(tf_cfg, "num_layers", None) is not None:
            num_layers = tf_cfg.num_layers
        self.parallel_config = getattr(od_config, "parallel_config", None)
        self.in_channels = in_channels
        self.out_channels = out_channels or in_channels
        self.inner_dim = num_attention_heads * attention_head_dim
        self.guidance_embeds = guidance_embeds
        self.pos_embed = FluxPosEmbed(theta=10000, axes_dim=list(axes_dims_rope))
        self.time_text_embed = CombinedTimestepGuidanceTextProjEmbeddings(
            embedding_dim=self.inner_dim, pooled_projection_dim=pooled_projection_dim, guidance_embeds=guidance_embeds)
        self.context_embedder = nn.Linear(joint_attention_dim, self.inner_dim)
        self.x_embedder = nn.Linear(in_channels, self.inner_dim)
        self.transformer_blocks = nn.ModuleList([
            FluxTransformerBlock(self.inner_dim, num_attention_heads, attention_head_dim, ref_rounding=ref_rounding)
            for _ in range(num_layers)])
        self.single_transformer_blocks = nn.ModuleList([
            FluxSingleTransformerBlock(self.inner_dim, num_attention_heads, attention_head_dim,
                                       ref_rounding=ref_rounding)
            for _ in range(num_single_layers)])
        self.norm_out = AdaLayerNormContinuous(self.inner_dim, self.inner_dim, eps=1e-6)
        self.proj_out = nn.Linear(self.inner_dim, patch_size * patch_size * self.out_channels, bias=True)
        self.parallel_config = None
        self.do_true_cfg = False
        self._res_bias = None

    # -- stages ---------------------------------------------------------------------------------
    @property
    def dtype(self) -> torch.dtype:
        return next(self.parameters()).dtype

    def prepare(self, hidden_states, encoder_hidden_states, pooled_projections, timestep, img_ids, txt_ids,
                guidance=None):
        img = self.x_embedder(hidden_states)
        timestep = timestep.to(device=img.device, dtype=img.dtype) * 1000
        if guidance is not None:
            guidance = guidance.to(device=img.device, dtype=img.dtype) * 1000
        temb = self.time_text_embed(timestep, guidance, pooled_projections)
        txt = self.context_embedder(encoder_hidden_states)
        if txt_ids.ndim == 3:
            txt_ids = txt_ids[0]
        if img_ids.ndim == 3:
            img_ids = img_ids[0]
        rotary = FluxRotary(*self.pos_embed(torch.cat((txt_ids, img_ids), dim=0)))
        return img, txt, temb, rotary

    def fuse_modulation(self) -> None:
        """Stack the SiLU->Linear projections of every AdaLayerNormZero / ZeroSingle into one weight so
        all modulation parameters of a step come from ONE pass over those weights (each is an M=B
        weight-streaming GEMV on its own). Per-block parameters become views of the stacked tensors."""
        lins = []
        for blk in self.transformer_blocks:
            lins += [blk.norm1.linear, blk.norm1_context.linear]
        lins += [blk.norm.linear for blk in self.single_transformer_blocks]
        ref = lins[0].weight
        rows = sum(l.weight.shape[0] for l in lins)
        w_all = torch.empty((rows, self.inner_dim), dtype=ref.dtype, device=ref.device)
        b_all = torch.empty((rows,), dtype=ref.dtype, device=ref.device)
        r = 0
        with torch.no_grad():
            for l in lins:
                n = l.weight.shape[0]
                w_all[r:r + n].copy_(l.weight)
                b_all[r:r + n].copy_(l.bias)
                l.weight.data, l.bias.data = w_all[r:r + n], b_all[r:r + n]
                r += n
        self._mod_weight, self._mod_bias = w_all, b_all
        self._res_bias = None

    def _gated_biases(self):
        """float32 biases of the gated output projections, dual [L, 2 (hidden, context), 2, C] and single
        [Ls, C] (None where there are no such blocks); rebuilt when any of them has been written since."""
        dual = [p for blk in self.transformer_blocks
                for p in (blk.attn.to_out[0].bias, blk.ff.net[2].bias, blk.attn.to_add_out.bias, blk.ff_context.net[2].bias)]
        single = [blk.proj_out.bias for blk in self.single_transformer_blocks]
        ps = dual + single
        tag = (sum(p._version for p in ps), ps[0].device, ps[0].dtype)
        if self._res_bias is None or self._res_bias[0] != tag:
            C = self.inner_dim
            d = torch.stack(dual).detach().float().view(len(self.transformer_blocks), 2, 2, C) if dual else None
            sgl = torch.stack(single).detach().float() if single else None
            self._res_bias = (tag, d, sgl)
        return self._res_bias[1], self._res_bias[2]

    def all_gate_rows(self, mods):
        """float32 (gates, gates * biases) of every gated projection, two small elementwise ops per step:
        dual [B, L, 2, 2, C] pairs and single [B, Ls, C] pairs (None where there are no such blocks)."""
        if mods is None or mods[0].dtype == torch.float32:
            return None, None
        C = self.inner_dim
        bias_dual, bias_single = self._gated_biases()
        dual = single = None
        if bias_dual is not None:
            B, L = mods[0].shape[:2]
            g = mods[0].view(B, L, 2, 2, 3 * C)[..., 2 * C:].float()
            dual = (g, g * bias_dual)
        if bias_single is not None:
            g = mods[1][..., 2 * C:].float()
            single = (g, g * bias_single)
        return dual, single

    def all_modulations(self, temb: torch.Tensor):
        """(dual [B, L, 2, 6C], single [B, Ls, 3C]) or None when not fused."""
        w = getattr(self, "_mod_weight", None)
        if w is None:
            return None
        C, L, Ls = self.inner_dim, len(self.transformer_blocks), len(self.single_transformer_blocks)
        out = F.linear(kernels.silu(temb), w, self._mod_bias)
        B = temb.shape[0]
        return out[:, :L * 12 * C].view(B, L, 2, 6 * C), out[:, L * 12 * C:].view(B, Ls, 3 * C)

    def run_blocks(self, img, txt, temb, rotary, joint_attention_kwargs=None):
        mods = self.all_modulations(temb)
        dual_rows, single_rows = self.all_gate_rows(mods)
        for i, block in enumerate(self.transformer_blocks):
            mp = (mods[0][:, i, 0], mods[0][:, i, 1]) if mods is not None else None
            gr = (dual_rows[0][:, i], dual_rows[1][:, i]) if dual_rows is not None else None
            txt, img = block(hidden_states=img, encoder_hidden_states=txt, temb=temb, image_rotary_emb=rotary,
                             joint_attention_kwargs=joint_attention_kwargs, mod_params=mp, gate_rows=gr)
        if len(self.single_transformer_blocks) == 0:
            return img, txt
        n_txt = txt.shape[1]
        x = torch.cat([txt, img], dim=1)  # once for the whole single-stream stack
        for i, block in enumerate(self.single_transformer_blocks):
            gr = (single_rows[0][:, i], single_rows[1][:, i]) if single_rows is not None else None
            x = block.forward_joint(x, temb, rotary, mod=mods[1][:, i] if mods is not None else None, in_place=True,
                                    gate_rows=gr)
        return x[:, n_txt:], x[:, :n_txt]

    def finish(self, img, temb, return_dict: bool = True):
        out = self.proj_out(self.norm_out(img, temb))
        return Transformer2DModelOutput(sample=out) if return_dict else (out,)

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor = None,
                pooled_projections: torch.Tensor = None, timestep: torch.Tensor = None,
                img_ids: torch.Tensor = None, txt_ids: torch.Tensor = None, guidance: torch.Tensor | None = None,
                joint_attention_kwargs: dict[str, Any] | None = None, return_dict: bool = True):
        img, txt, temb, rotary = self.prepare(hidden_states, encoder_hidden_states, pooled_projections, timestep,
                                              img_ids, txt_ids, guidance)
        img, txt = self.run_blocks(img, txt, temb, rotary, joint_attention_kwargs)
        return self.finish(img, temb, return_dict=return_dict)

    # -- weights --------------------------------------------------------------------------------
    def load_weights(self, weights) -> set[str]:
        """Load a diffusers-layout checkpoint stream, stacking separate q/k/v projections (flux.py:588-628)."""
        from .weights import QKV_JOINT_MAPPING, load_stacked_weights

        return load_stacked_weights(self, weights, QKV_JOINT_MAPPING, substring_renames=((".to_out.0.", ".to_out."),))

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
