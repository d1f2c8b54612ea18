"""Qwen-Image dual-stream MMDiT composed from the gfx950 kernels.

Module tree, parameter names and call signatures follow
vllm_omni/diffusion/models/qwen_image/qwen_image_transformer.py (``qit.py`` below) so a reference
state dict loads unchanged (fused ``to_qkv`` / ``add_kv_proj`` as after its ``load_weights`` stacking,
qit.py:1073-1113). Differences are all below the module interfaces:

  * QK-RMSNorm + rotary + the three ``torch.cat([txt, img])`` copies are one fused pass per stream that
    writes straight into the joint [B, S_txt+S_img, H, D] buffers (qit.py:588-606);
  * adaLN LayerNorm+modulate and the gated residual are one pass each (qit.py:770-773, 794-806);
  * GELU(tanh) runs in place on the MLP-up output (qit.py:424);
  * dense projections are ``torch.nn.functional.linear`` (hipBLASLt MFMA GEMMs).
"""

from __future__ import annotations

import math
from functools import lru_cache
from typing import Any

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import kernels
from .._lib import ODIT_NORM_HEAD
from ..attention.backends.abstract import AttentionMetadata
from ..attention.layer import Attention
from ..layers.adalayernorm import AdaLayerNorm, adaln_pair
from ..layers.rmsnorm import RMSNorm
from ..layers.rope import RotaryEmbedding


def _require_single_gpu(od_config: Any | None) -> None:
    """The reference models read their parallel degrees from ``od_config.parallel_config``
    (vllm_omni/diffusion/data.py); this package runs one GPU and refuses anything else."""
    pc = getattr(od_config, "parallel_config", None)
    if pc is None:
        return
    for name in ("sequence_parallel_size", "ulysses_degree", "ring_degree", "tensor_parallel_size",
                 "cfg_parallel_size", "pipeline_parallel_size", "data_parallel_size"):
        degree = getattr(pc, name, 1)
        if degree not in (None, 1):
            raise NotImplementedError(f"{name}={degree}: this package runs on one GPU")


class Transformer2DModelOutput:
    """Minimal stand-in for diffusers' output object: ``.sample`` and ``[0]`` both work."""

    def __init__(self, sample: torch.Tensor):
        self.sample = sample

    def __getitem__(self, i: int):
        return (self.sample,)[i]


class SiLU(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return kernels.silu(x)


class ApproxGELU(nn.Module):
    """Linear + GELU(tanh) (qit.py:399-424) as one GEMM whose epilogue applies bias and activation.
    ``fused = False`` runs the projection and then the activation in place on its output, which rounds
    the pre-activation to the tensor dtype like the reference's two ops do."""

    def __init__(self, dim_in: int, dim_out: int, bias: bool = True, fused: bool = True):
        super().__init__()
        self.proj = nn.Linear(dim_in, dim_out, bias=bias)
        self.fused = fused

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fused and x.dtype != torch.float32 and x.is_contiguous():
            return kernels.linear(x, self.proj.weight, self.proj.bias, activation="gelu_tanh")
        y = self.proj(x)
        return kernels.gelu_tanh(y, out=y)


class FeedForward(nn.Module):
    """net.0 = Linear+GELU(tanh), net.1 = placeholder, net.2 = Linear (qit.py:427-466)."""

    def __init__(self, dim: int, dim_out: int | None = None, mult: int = 4, inner_dim: int | None = None,
                 bias: bool = True, fused: bool = True):
        super().__init__()
        inner = inner_dim or dim * mult
        self.net = nn.ModuleList([ApproxGELU(dim, inner, bias=bias, fused=fused), nn.Identity(),
                                  nn.Linear(inner, dim_out or dim, bias=bias)])
        self.fused = fused

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        for m in self.net:
            x = m(x)
        return x

    def forward_residual(self, x: torch.Tensor, residual: torch.Tensor, gate: torch.Tensor | None,
                         out: torch.Tensor | None = None, ref_rounding: bool = False, pre=None) -> torch.Tensor:
        """residual + gate * FF(x): with ``fused`` the down-projection's epilogue adds the gated result
        onto the residual; otherwise the projection is followed by the gated-residual kernel."""
        return project_residual(self.net[2], self.net[0](x), residual, gate, out=out,
                                fused=self.fused, ref_rounding=ref_rounding, pre=pre)


def project(lin: nn.Linear, x: torch.Tensor) -> torch.Tensor:
    """lin(x). A bf16 projection that a hand-written GEMM kernel would run (the engine asked for, or the one
    a tuning call found faster for this problem) goes through ``kernels.linear``; everything else through
    torch's linear (hipBLASLt with the solution table tuned offline)."""
    if (x.dtype == torch.bfloat16 and x.is_cuda and x.is_contiguous()
            and kernels.linear(x, lin.weight, lin.bias, plan_only=True)[0]):
        return kernels.linear(x, lin.weight, lin.bias)
    return lin(x)


# The gate differs per batch entry. The hand-written GEMM takes one gate vector per batch entry in one
# launch; the library needs one GEMM per entry, and below this many rows per entry (the 256-token text
# stream of a CFG batch: two GEMMs of 256 rows) one library GEMM over all entries plus the
# gated-residual kernel is faster than that (measured: 1.2 ms of a 135 ms step).
FUSE_MIN_ROWS = 1024


def project_residual(lin: nn.Linear, x: torch.Tensor, residual: torch.Tensor, gate: torch.Tensor | None,
                     out: torch.Tensor | None = None, fused: bool = True, ref_rounding: bool = False,
                     pre: tuple[torch.Tensor, torch.Tensor | None] | None = None) -> torch.Tensor:
    """residual + gate * lin(x) (gate [B,N] or [B,1,N], None = plain add) in one GEMM, or, unfused, as
    projection + gated-residual kernel (qit.py:794-806). ``pre`` = (float32 gate [B,N], float32
    gate * bias [B,N] or None) made by the caller for all blocks at once replaces ``gate`` on the fused path."""
    per_token_gate = gate is not None and gate.dim() == 3 and gate.shape[1] != 1
    few_rows = gate is not None and x.dim() == 3 and x.shape[0] > 1 and x.shape[1] < FUSE_MIN_ROWS
    if (fused and not ref_rounding and not per_token_gate and x.dtype != torch.float32
            and x.is_contiguous() and residual.is_contiguous()):
        if pre is not None:
            args = dict(residual=residual, gate=pre[0], gate_bias=pre[1], prescaled=True)
            bias = None
        else:
            args = dict(residual=residual, gate=gate)
            bias = lin.bias
        if not few_rows or kernels.linear(x, lin.weight, bias, plan_only=True, **args)[0]:
            return kernels.linear(x, lin.weight, bias, out=out, **args)
    return kernels.gated_residual(residual, lin(x), gate, out=out, ref_rounding=ref_rounding)


class QwenEmbedRope(nn.Module):
    """3-axis rotary tables (frame, row, column) of qit.py:298-396, built from integer token positions.

    Token (f, r, c) of image number ``i`` of the list sits at frame ``i + f``; with ``scale_rope`` rows
    and columns are centred (row r of an image with ``h`` rows sits at ``r - (h - h // 2)``), otherwise
    they count from zero. Text token ``j`` sits at ``(p, p, p)`` with ``p = start + j`` where ``start``
    is the largest half-extent (full extent without ``scale_rope``) over the images. A position ``x`` on
    an axis of ``d`` channels gives the d/2 angles ``x * theta ** (-2k / d)``, evaluated in float32.
    ``forward`` returns complex64 (vid_freqs, txt_freqs) like the reference, cached per (shapes, device)."""

    layer3d = False  # QwenEmbedLayer3DRope sets it

    def __init__(self, theta: int, axes_dim: list[int], scale_rope: bool = True):
        super().__init__()
        self.theta, self.axes_dim, self.scale_rope = theta, list(axes_dim), scale_rope
        if any(d % 2 for d in self.axes_dim):
            raise ValueError("every rotary axis needs an even number of channels")
        # inverse frequencies of the three axes, side by side: [sum(d) / 2]
        # table construction runs on the host whatever default device the model is built under
        cpu = torch.device("cpu")
        self.inv_freq = torch.cat([
            1.0 / torch.pow(theta, torch.arange(0, d, 2, device=cpu).to(torch.float32).div(d)) for d in self.axes_dim])
        self.axis_of = torch.repeat_interleave(torch.arange(len(self.axes_dim), device=cpu),
                                               torch.tensor([d // 2 for d in self.axes_dim], device=cpu))
        self._tables = lru_cache(maxsize=16)(self._build)

    def _table(self, positions: torch.Tensor) -> torch.Tensor:
        """positions: int64 [N, 3] -> complex64 [N, sum(d) / 2] unit phasors."""
        ang = positions.to(torch.float32)[:, self.axis_of] * self.inv_freq
        return torch.polar(torch.ones_like(ang), ang)

    def _image_positions(self, frame: int, height: int, width: int, first_frame: int) -> torch.Tensor:
        r0 = -(height - height // 2) if self.scale_rope else 0
        c0 = -(width - width // 2) if self.scale_rope else 0
        cpu = torch.device("cpu")
        grid = torch.stack(torch.meshgrid(torch.arange(first_frame, first_frame + frame, device=cpu),
                                          torch.arange(r0, r0 + height, device=cpu),
                                          torch.arange(c0, c0 + width, device=cpu), indexing="ij"), dim=-1)
        return grid.reshape(-1, 3)

    def _build(self, shapes: tuple[tuple[int, int, int], ...], txt_len: int, device: str):
        last = len(shapes) - 1
        pos, start = [], 0
        for i, (f, h, w) in enumerate(shapes):
            first = i
            if self.layer3d and i == last:  # the condition image: one frame before the origin (qit.py:278-296)
                if f != 1:
                    raise ValueError("the condition image of the layered variant has one frame")
                first = -1
            pos.append(self._image_positions(f, h, w, first))
            start = max(start, max(h // 2, w // 2) if self.scale_rope else max(h, w))
        if self.layer3d:
            start = max(start, last)
        vid = self._table(torch.cat(pos, dim=0)).to(device)
        txt = self._table(torch.arange(start, start + txt_len, device="cpu").view(-1, 1).expand(-1, 3)).to(device)
        return vid, txt

    @staticmethod
    def _norm_shapes(video_fhw) -> tuple[tuple[int, int, int], ...]:
        if isinstance(video_fhw, list) and video_fhw and isinstance(video_fhw[0], list):
            video_fhw = video_fhw[0]  # per-sample list of shapes: the first sample's (qit.py:349-352)
        if isinstance(video_fhw, tuple) and len(video_fhw) == 3 and all(isinstance(v, int) for v in video_fhw):
            video_fhw = [video_fhw]
        return tuple(tuple(int(v) for v in s) for s in video_fhw)

    def forward(self, video_fhw, txt_seq_lens, device):
        return self._tables(self._norm_shapes(video_fhw), int(max(txt_seq_lens)), str(device))


class QwenEmbedLayer3DRope(QwenEmbedRope):
    """The layered-image variant's tables (qit.py:183-296): as QwenEmbedRope for the layers, the last
    image of the list (the condition image) at frame position -1, text after the larger of the images'
    half-extents and the number of layers."""

    layer3d = True


class RotaryTables:
    """Complex tables as the reference passes them between modules, plus float32 cos/sin views."""

    def __init__(self, vid_freqs: torch.Tensor, txt_freqs: torch.Tensor):
        self.vid_freqs, self.txt_freqs = vid_freqs, txt_freqs
        self.img_cos, self.img_sin = vid_freqs.real.contiguous(), vid_freqs.imag.contiguous()
        self.txt_cos, self.txt_sin = txt_freqs.real.contiguous(), txt_freqs.imag.contiguous()

    def __iter__(self):  # unpacks like the reference's (vid_freqs, txt_freqs) tuple
        return iter((self.vid_freqs, self.txt_freqs))

    def __getitem__(self, i: int):
        return (self.vid_freqs, self.txt_freqs)[i]


class QwenImageCrossAttention(nn.Module):
    """Joint text+image attention of one block (qit.py:469-661)."""

    def __init__(self, dim: int, num_heads: int, head_dim: int, added_kv_proj_dim: int,
                 out_bias: bool = True, eps: float = 1e-6, ref_rounding: bool = False, fused: bool = True):
        super().__init__()
        assert dim % num_heads == 0
        self.fused = fused
        self.dim, self.head_dim, self.total_num_heads, self.eps = dim, head_dim, num_heads, eps
        inner = head_dim * num_heads
        self.inner_dim = inner
        self.to_qkv = nn.Linear(dim, 3 * inner, bias=True)
        self.add_kv_proj = nn.Linear(added_kv_proj_dim, 3 * inner, bias=True)
        self.query_num_heads = self.kv_num_heads = num_heads
        self.norm_q = RMSNorm(head_dim, eps=eps)
        self.norm_k = RMSNorm(head_dim, eps=eps)
        self.norm_added_q = RMSNorm(head_dim, eps=eps)
        self.norm_added_k = RMSNorm(head_dim, eps=eps)
        self.to_out = nn.Linear(inner, dim, bias=out_bias)
        self.to_add_out = nn.Linear(inner, dim, bias=out_bias)
        self.attn = Attention(num_heads=num_heads, head_size=head_dim, softmax_scale=1.0 / (head_dim ** 0.5),
                              causal=False, num_kv_heads=num_heads)
        self.rope = RotaryEmbedding(is_neox_style=False)
        self.ref_rounding = ref_rounding

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, vid_freqs, txt_freqs=None,
                hidden_states_mask: torch.Tensor | None = None,
                encoder_hidden_states_mask: torch.Tensor | None = None, residuals=None):
        """``residuals`` = (img_residual, img_gate, txt_residual, txt_gate[, img_pre, txt_pre]): return
        residual + gate * projection for both streams (new tensors) instead of the bare projections;
        the ``*_pre`` pairs are caller-made float32 (gate, gate * bias) rows (see project_residual)."""
        tables = vid_freqs if isinstance(vid_freqs, RotaryTables) else RotaryTables(vid_freqs, txt_freqs)
        B, S_img, _ = hidden_states.shape
        S_txt = encoder_hidden_states.shape[1]
        H, D = self.total_num_heads, self.head_dim
        img_qkv = project(self.to_qkv, hidden_states).view(B, S_img, 3, H, D)
        txt_qkv = project(self.add_kv_proj, encoder_hidden_states).view(B, S_txt, 3, H, D)
        S = S_txt + S_img
        jq = torch.empty((B, S, H, D), dtype=img_qkv.dtype, device=img_qkv.device)
        jk = torch.empty_like(jq)
        # q and k are rewritten by norm + rotary into the joint buffers; v is only moved, so when the
        # attention kernel can read the two value halves where the projections left them it is not copied
        v_in_place = (S_txt % 64 == 0 and img_qkv.dtype != torch.float32
                      and not self.ref_rounding)
        jv = None if v_in_place else torch.empty_like(jq)
        rr = self.ref_rounding
        # text rows [0, S_txt) and image rows [S_txt, S) of the joint buffers, one launch for both streams
        kernels.qknorm_rope_pair(
            (txt_qkv[:, :, 0], txt_qkv[:, :, 1], None if v_in_place else txt_qkv[:, :, 2],
             self.norm_added_q.weight, self.norm_added_k.weight, tables.txt_cos, tables.txt_sin, 0),
            (img_qkv[:, :, 0], img_qkv[:, :, 1], None if v_in_place else img_qkv[:, :, 2],
             self.norm_q.weight, self.norm_k.weight, tables.img_cos, tables.img_sin, S_txt),
            jq, jk, jv, eps=self.eps, norm_mode=ODIT_NORM_HEAD, ref_rounding=rr)
        # the backend writes the text and image rows of the output to two dense tensors
        meta = AttentionMetadata(output_split=S_txt)
        if v_in_place:
            jv, meta.value_tail = txt_qkv[:, :, 2], img_qkv[:, :, 2]
        if hidden_states_mask is not None or encoder_hidden_states_mask is not None:
            ones = lambda n: torch.ones((B, n), dtype=torch.bool, device=jq.device)  # noqa: E731
            txt_m = encoder_hidden_states_mask if encoder_hidden_states_mask is not None else ones(S_txt)
            img_m = hidden_states_mask if hidden_states_mask is not None else ones(S_img)
            meta.attn_mask = torch.cat([txt_m.bool(), img_m.bool()], dim=1)
            # the model drops an all-true mask once per forward (run_blocks); for a direct call of a block
            # with one the masked kernel gives the same values, and testing here would synchronise per block
            meta.attn_mask_checked = True
        txt_attn, img_attn = self.attn(jq, jk, jv, meta)
        if residuals is not None:
            img_res, img_gate, txt_res, txt_gate = residuals[:4]
            img_pre, txt_pre = residuals[4:] if len(residuals) == 6 else (None, None)
            img_out = project_residual(self.to_out, img_attn.flatten(2, 3), img_res, img_gate,
                                       fused=self.fused, ref_rounding=rr, pre=img_pre)
            txt_out = project_residual(self.to_add_out, txt_attn.flatten(2, 3), txt_res, txt_gate,
                                       fused=self.fused, ref_rounding=rr, pre=txt_pre)
            return img_out, txt_out
        img_out = self.to_out(img_attn.flatten(2, 3))
        txt_out = self.to_add_out(txt_attn.flatten(2, 3))
        return img_out, txt_out


class QwenImageTransformerBlock(nn.Module):
    """One dual-stream block (qit.py:664-814); returns (encoder_hidden_states, hidden_states)."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, eps: float = 1e-6,
                 zero_cond_t: bool = False, mlp_ratio: int = 4, ref_rounding: bool = False,
                 fuse_epilogues: bool = True):
        super().__init__()
        self.dim = dim
        fused = fuse_epilogues and not ref_rounding
        self.num_attention_heads, self.attention_head_dim = num_attention_heads, attention_head_dim
        self.img_mod = nn.Sequential(SiLU(), nn.Linear(dim, 6 * dim, bias=True))
        self.img_norm1 = AdaLayerNorm(dim, elementwise_affine=False, eps=eps, ref_rounding=ref_rounding)
        self.attn = QwenImageCrossAttention(dim=dim, num_heads=num_attention_heads, head_dim=attention_head_dim,
                                            added_kv_proj_dim=dim, eps=eps, ref_rounding=ref_rounding, fused=fused)
        self.img_norm2 = AdaLayerNorm(dim, elementwise_affine=False, eps=eps, ref_rounding=ref_rounding)
        self.img_mlp = FeedForward(dim=dim, dim_out=dim, mult=mlp_ratio, fused=fused)
        self.txt_mod = nn.Sequential(SiLU(), nn.Linear(dim, 6 * dim, bias=True))
        self.txt_norm1 = AdaLayerNorm(dim, elementwise_affine=False, eps=eps, ref_rounding=ref_rounding)
        self.txt_norm2 = AdaLayerNorm(dim, elementwise_affine=False, eps=eps, ref_rounding=ref_rounding)
        self.txt_mlp = FeedForward(dim=dim, dim_out=dim, mult=mlp_ratio, fused=fused)
        self.zero_cond_t = zero_cond_t
        self.ref_rounding = ref_rounding

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor,
                encoder_hidden_states_mask: torch.Tensor | None, temb: torch.Tensor, image_rotary_emb,
                joint_attention_kwargs: dict[str, Any] | None = None, modulate_index: torch.Tensor | None = None,
                hidden_states_mask: torch.Tensor | None = None,
                mod_params: tuple[torch.Tensor, torch.Tensor] | None = None,
                gate_rows: tuple[torch.Tensor, torch.Tensor] | None = None):
        """``mod_params`` = (img [B,6C], txt [B,6C]) computed by the caller for all blocks at once
        (they depend on ``temb`` only); when absent they are computed here as in the reference.
        ``gate_rows`` = float32 (gates, gates * biases), each [B, 2 (img, txt), 2 (attention, MLP), C],
        likewise made once per step: the fused output projections then need no per-call set-up."""
        pre = [[None, None], [None, None]]
        if gate_rows is not None and modulate_index is None:
            pre = [[(gate_rows[0][:, s, j], gate_rows[1][:, s, j]) for j in range(2)] for s in range(2)]
        rr = self.ref_rounding
        if mod_params is not None:
            img_mod_params, txt_mod_params = mod_params
        else:
            img_mod_params = self.img_mod(temb)
            if self.zero_cond_t:
                temb = torch.chunk(temb, 2, dim=0)[0]
            txt_mod_params = self.txt_mod(temb)
        img_mod1, img_mod2 = img_mod_params.chunk(2, dim=-1)
        txt_mod1, txt_mod2 = txt_mod_params.chunk(2, dim=-1)

        # without a per-token index the two streams' norms are one launch
        if modulate_index is None:
            (img_modulated, img_gate1), (txt_modulated, txt_gate1) = adaln_pair(
                self.img_norm1, hidden_states, img_mod1, self.txt_norm1, encoder_hidden_states, txt_mod1)
        else:
            img_modulated, img_gate1 = self.img_norm1(hidden_states, img_mod1, modulate_index)
            txt_modulated, txt_gate1 = self.txt_norm1(encoder_hidden_states, txt_mod1)
        tables = image_rotary_emb if isinstance(image_rotary_emb, RotaryTables) else RotaryTables(*image_rotary_emb)
        # the block's inputs are never written (callers such as TeaCache keep them to form residuals):
        # the attention residuals land in new tensors, the MLP residuals then update those in place
        hidden_states, encoder_hidden_states = self.attn(
            img_modulated, txt_modulated, tables, hidden_states_mask=hidden_states_mask,
            encoder_hidden_states_mask=encoder_hidden_states_mask,
            residuals=(hidden_states, img_gate1, encoder_hidden_states, txt_gate1, pre[0][0], pre[1][0]))

        if modulate_index is None:
            (img_modulated2, img_gate2), (txt_modulated2, txt_gate2) = adaln_pair(
                self.img_norm2, hidden_states, img_mod2, self.txt_norm2, encoder_hidden_states, txt_mod2)
        else:
            img_modulated2, img_gate2 = self.img_norm2(hidden_states, img_mod2, modulate_index)
            txt_modulated2, txt_gate2 = self.txt_norm2(encoder_hidden_states, txt_mod2)
        hidden_states = self.img_mlp.forward_residual(img_modulated2, hidden_states, img_gate2, out=hidden_states,
                                                      ref_rounding=rr, pre=pre[0][1])
        encoder_hidden_states = self.txt_mlp.forward_residual(txt_modulated2, encoder_hidden_states, txt_gate2,
                                                              out=encoder_hidden_states, ref_rounding=rr, pre=pre[1][1])
        if encoder_hidden_states.dtype == torch.float16:
            encoder_hidden_states = encoder_hidden_states.clip(-65504, 65504)
        if hidden_states.dtype == torch.float16:
            hidden_states = hidden_states.clip(-65504, 65504)
        return encoder_hidden_states, hidden_states


class TimestepEmbedding(nn.Module):
    def __init__(self, in_channels: int, time_embed_dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_channels, time_embed_dim)
        self.linear_2 = nn.Linear(time_embed_dim, time_embed_dim)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.linear_2(kernels.silu(self.linear_1(x)))


class QwenTimestepProjEmbeddings(nn.Module):
    """Sinusoid(256 channels, cos first, scale 1000) -> MLP, plus a 2-entry learned embedding picked by
    ``addition_t_cond`` when ``use_additional_t_cond`` (qit.py:159-181)."""

    def __init__(self, embedding_dim: int, use_additional_t_cond: bool = False):
        super().__init__()
        self.timestep_embedder = TimestepEmbedding(256, embedding_dim)
        self.use_additional_t_cond = use_additional_t_cond
        if use_additional_t_cond:
            self.addition_t_embedding = nn.Embedding(2, embedding_dim)

    @staticmethod
    def time_proj(t: torch.Tensor, dim: int = 256, max_period: int = 10000, scale: float = 1000.0):
        """diffusers ``Timesteps(dim, flip_sin_to_cos=True, downscale_freq_shift=0, scale)``: fp32
        frequencies times ``t.float()``, cosines first."""
        half = dim // 2
        freqs = torch.exp(-math.log(max_period) * torch.arange(half, dtype=torch.float32, device=t.device) / half)
        arg = scale * (t[:, None].float() * freqs[None, :])
        return torch.cat((torch.cos(arg), torch.sin(arg)), dim=-1)

    def forward(self, timestep: torch.Tensor, hidden_states: torch.Tensor, addition_t_cond=None):
        emb = self.timestep_embedder(self.time_proj(timestep).to(hidden_states.dtype))
        if self.use_additional_t_cond:
            if addition_t_cond is None:
                raise ValueError("When additional_t_cond is True, addition_t_cond must be provided.")
            emb = emb + self.addition_t_embedding(addition_t_cond).to(hidden_states.dtype)
        return emb


class AdaLayerNormContinuous(nn.Module):
    """Final norm: (scale, shift) = Linear(SiLU(cond)).chunk(2); LN(x)(1+scale)+shift (qit.py:936, 1065)."""

    def __init__(self, embedding_dim: int, conditioning_embedding_dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.linear = nn.Linear(conditioning_embedding_dim, 2 * embedding_dim, bias=True)

    def forward(self, x: torch.Tensor, cond: torch.Tensor) -> torch.Tensor:
        emb = self.linear(kernels.silu(cond).to(x.dtype))
        scale, shift = emb.chunk(2, dim=1)
        return kernels.adaln_modulate(x, shift, scale, eps=self.eps)


class QwenImageTransformer2DModel(nn.Module):
    """Stem, N dual-stream blocks, head (qit.py:817-1071). ``prepare`` / ``run_blocks`` / ``finish``
    are the three stages TeaCache needs to call separately (cache/teacache/extractors.py:147-279)."""

    _repeated_blocks = ["QwenImageTransformerBlock"]
    enable_separate_cfg = True   # class attribute of the reference's CachedTransformer base (cache/base.py:105-112)

    def __init__(self, od_config: Any | None = None, patch_size: int = 2, in_channels: int = 64,
                 out_channels: int | None = 16, num_layers: int = 60, attention_head_dim: int = 128,
                 num_attention_heads: int = 24, joint_attention_dim: int = 3584, guidance_embeds: bool = False,
                 axes_dims_rope: tuple[int, int, int] = (16, 56, 56), zero_cond_t: bool = False,
                 use_additional_t_cond: bool = False, use_layer3d_rope: bool = False, quant_config: Any | None = None,
                 mlp_ratio: int = 4, ref_rounding: bool = False, fuse_epilogues: bool = True):
        """Arguments up to ``quant_config`` are the reference's (qit.py:885-901), ``od_config`` included so a
        pipeline's ``Model(od_config=..., **transformer_kwargs)`` call works unchanged; only its
        ``parallel_config`` is looked at, and it has to describe one GPU."""
        super().__init__()
        _require_single_gpu(od_config)
        if quant_config is not None:
            raise NotImplementedError("quantised linears are not part of this package")
        self.guidance_embeds = guidance_embeds
        self.in_channels = in_channels
        self.out_channels = out_channels or in_channels
        self.inner_dim = num_attention_heads * attention_head_dim
        rope_cls = QwenEmbedLayer3DRope if use_layer3d_rope else QwenEmbedRope
        self.pos_embed = rope_cls(theta=10000, axes_dim=list(axes_dims_rope), scale_rope=True)
        self.time_text_embed = QwenTimestepProjEmbeddings(embedding_dim=self.inner_dim,
                                                          use_additional_t_cond=use_additional_t_cond)
        self.txt_norm = RMSNorm(joint_attention_dim, eps=1e-6)
        self.img_in = nn.Linear(in_channels, self.inner_dim)
        self.txt_in = nn.Linear(joint_attention_dim, self.inner_dim)
        self.transformer_blocks = nn.ModuleList([
            QwenImageTransformerBlock(self.inner_dim, num_attention_heads, attention_head_dim,
                                      mlp_ratio=mlp_ratio, ref_rounding=ref_rounding, fuse_epilogues=fuse_epilogues,
                                      zero_cond_t=zero_cond_t)
            for _ in range(num_layers)])
        self.norm_out = AdaLayerNormContinuous(self.inner_dim, self.inner_dim, eps=1e-6)
        self.proj_out = nn.Linear(self.inner_dim, patch_size * patch_size * self.out_channels, bias=True)
        self.zero_cond_t = zero_cond_t
        self._res_bias = None
        self.parallel_config = getattr(od_config, "parallel_config", None)
        self.do_true_cfg = False

    @property
    def dtype(self) -> torch.dtype:
        return next(self.parameters()).dtype

    # -- stages ---------------------------------------------------------------------------------
    def prepare(self, hidden_states, encoder_hidden_states, timestep, img_shapes, txt_seq_lens,
                additional_t_cond=None):
        """Stem. With ``zero_cond_t`` (editing checkpoints) the timestep is doubled to [t, 0 * t], so temb
        has 2B rows: real-timestep conditioning, then timestep-zero conditioning (qit.py:141-145)."""
        img = self.img_in(hidden_states)
        timestep = timestep.to(device=img.device, dtype=img.dtype)
        if self.zero_cond_t:
            timestep = torch.cat([timestep, timestep * 0], dim=0)
        txt = self.txt_in(self.txt_norm(encoder_hidden_states))
        if additional_t_cond is not None and self.zero_cond_t:
            additional_t_cond = torch.cat([additional_t_cond, additional_t_cond], dim=0)
        temb = self.time_text_embed(timestep, img, additional_t_cond)
        if txt_seq_lens is None:
            txt_seq_lens = [encoder_hidden_states.shape[1]]
        vid_freqs, txt_freqs = self.pos_embed(img_shapes, txt_seq_lens, device=img.device)
        return img, txt, temb, RotaryTables(vid_freqs, txt_freqs)

    def modulate_index(self, img_shapes, device) -> torch.Tensor | None:
        """[B, S_img] int32 per-token conditioning choice of the editing variant: 0 (real timestep) for the
        tokens of each sample's first image, 1 (timestep zero) for every later image; ``img_shapes`` is
        per sample a list of (frame, height, width) (qit.py:146-154). None for the plain model."""
        if not self.zero_cond_t:
            return None
        samples = [[s] if isinstance(s[0], int) else list(s) for s in img_shapes]  # bare (f, h, w) = one image
        rows = [[0] * math.prod(s[0]) + [1] * sum(math.prod(x) for x in s[1:]) for s in samples]
        return torch.tensor(rows, device=device, dtype=torch.int32)

    def fuse_modulation(self) -> None:
        """Stack every block's img_mod / txt_mod Linear into one [L, 2, 6C, C] weight so that the
        2L modulation projections of a step (each a weight-streaming M=B GEMV: the largest
        non-GEMM HBM stream of the model) run as ONE pass over the weights. The per-block parameters
        become views of the stacked tensors: names, shapes and values are unchanged."""
        L, C = len(self.transformer_blocks), self.inner_dim
        ref = self.transformer_blocks[0].img_mod[1].weight
        w_all = torch.empty((L, 2, 6 * C, C), dtype=ref.dtype, device=ref.device)
        b_all = torch.empty((L, 2, 6 * C), dtype=ref.dtype, device=ref.device)
        with torch.no_grad():
            for i, blk in enumerate(self.transformer_blocks):
                for j, lin in enumerate((blk.img_mod[1], blk.txt_mod[1])):
                    w_all[i, j].copy_(lin.weight)
                    b_all[i, j].copy_(lin.bias)
                    lin.weight.data = w_all[i, j]
                    lin.bias.data = b_all[i, j]
        self._mod_weight, self._mod_bias = w_all, b_all
        self._res_bias = None

    def _gated_biases(self) -> torch.Tensor:
        """float32 [L, 2 (img, txt), 2 (attention, MLP), C]: biases of the four gated output projections
        of every block; rebuilt when any of them has been written since (in-place loads bump _version)."""
        ps = [p for blk in self.transformer_blocks
              for p in (blk.attn.to_out.bias, blk.img_mlp.net[2].bias, blk.attn.to_add_out.bias, blk.txt_mlp.net[2].bias)]
        tag = (sum(p._version for p in ps), ps[0].device, ps[0].dtype)
        if self._res_bias is None or self._res_bias[0] != tag:
            L, C = len(self.transformer_blocks), self.inner_dim
            self._res_bias = (tag, torch.stack(ps).detach().float().view(L, 2, 2, C))
        return self._res_bias[1]

    def all_gate_rows(self, mods: torch.Tensor | None):
        """float32 (gates, gates * biases) [B, L, 2, 2, C] of the four gated projections of every block,
        from the stacked modulation parameters: two small elementwise ops per step."""
        if mods is None or mods.dtype == torch.float32 or self.zero_cond_t:
            return None  # per-token gates of the editing variant do not fit one row per batch entry
        B, L, C = mods.shape[0], mods.shape[1], self.inner_dim
        gates = mods.view(B, L, 2, 2, 3 * C)[..., 2 * C:].float()
        return gates, gates * self._gated_biases()

    def all_modulations(self, temb: torch.Tensor) -> torch.Tensor | None:
        """[B, L, 2, 6C] modulation parameters of every block, or None when not fused. For the editing
        variant temb has 2B rows and so has the result: the image stream reads all of them through the
        per-token index, the text stream the first B (qit.py:758-767)."""
        w = getattr(self, "_mod_weight", None)
        if w is None:
            return None
        L, C = w.shape[0], self.inner_dim
        out = F.linear(kernels.silu(temb), w.view(L * 2 * 6 * C, C), self._mod_bias.view(-1))
        return out.view(temb.shape[0], L, 2, 6 * C)

    def run_blocks(self, img, txt, temb, rotary, encoder_hidden_states_mask=None, attention_kwargs=None,
                   modulate_index=None):
        mask = encoder_hidden_states_mask
        if mask is not None and bool(mask.all()):
            mask = None  # all-true masks are dropped (qit.py:1044-1048)
        mods = self.all_modulations(temb)
        rows = self.all_gate_rows(mods)
        for i, block in enumerate(self.transformer_blocks):
            mp = (mods[:, i, 0], mods[:txt.shape[0], i, 1]) if mods is not None else None
            gr = (rows[0][:, i], rows[1][:, i]) if rows is not None else None
            txt, img = block(hidden_states=img, encoder_hidden_states=txt, encoder_hidden_states_mask=mask,
                             temb=temb, image_rotary_emb=rotary, joint_attention_kwargs=attention_kwargs,
                             modulate_index=modulate_index, mod_params=mp, gate_rows=gr)
        return img, txt

    def finish(self, img, temb, return_dict: bool = True):
        if self.zero_cond_t:
            temb = temb.chunk(2, dim=0)[0]  # the head is conditioned on the real timestep (qit.py:1062-1063)
        out = self.proj_out(self.norm_out(img, temb))
        return Transformer2DModelOutput(sample=out) if return_dict else (out,)

    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor = None,
                encoder_hidden_states_mask: torch.Tensor = None, timestep: torch.Tensor = None,
                img_shapes=None, txt_seq_lens=None, guidance: torch.Tensor = None,
                attention_kwargs: dict[str, Any] | None = None, additional_t_cond=None, return_dict: bool = True):
        if guidance is not None:
            # the reference forwards it to a time embedding whose forward has no such argument (qit.py:169,
            # 1017-1024) and fails there; no Qwen-Image checkpoint sets guidance_embeds
            raise TypeError("QwenImageTransformer2DModel: the timestep embedding takes no guidance; pass guidance=None")
        img, txt, temb, rotary = self.prepare(hidden_states, encoder_hidden_states, timestep, img_shapes, txt_seq_lens,
                                              additional_t_cond)
        index = self.modulate_index(img_shapes, img.device)
        img, txt = self.run_blocks(img, txt, temb, rotary, encoder_hidden_states_mask, attention_kwargs,
                                   modulate_index=index)
        return self.finish(img, temb, return_dict=return_dict)

    # -- weights --------------------------------------------------------------------------------
    def load_weights(self, weights) -> set[str]:
        """Load a diffusers-layout checkpoint stream: separate to_q/to_k/to_v and add_*_proj tensors are
        stacked into the fused projections, ``attn.to_out.0`` maps to ``attn.to_out`` (qit.py:1073-1113)."""
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
