"""Oracle restatement of the per-op arithmetic on the DiT block path (test infrastructure only).

All paths below are relative to the reference tree ``vllm_omni/diffusion/``.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# ------------------------------------------------------------------------------------- RMSNorm
def rms_norm_head(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6) -> torch.Tensor:
    """Per-last-axis RMSNorm in vLLM's order: fp32 normalise, cast to x.dtype, then multiply by weight.

    Call sites: models/qwen_image/qwen_image_transformer.py:505-506, 543-544, 588-591 (third-party
    vllm RMSNorm; cast order adopted from upstream — parity unpinned at that boundary; the same order is
    written out in the reference tree at model_executor/models/qwen3_tts/modeling_qwen3_tts.py:590-598).
    """
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    y = (xf * torch.rsqrt(var + eps)).to(x.dtype)
    return y if weight is None else y * weight


def rms_norm_row_fp32(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """Whole-row RMSNorm kept in fp32 including the weight, cast at the end.

    Follows DistributedRMSNorm.forward with tp_size == 1, models/wan2_2/wan2_2_transformer.py:70-89.
    """
    xf = x.float()
    rms = torch.sqrt(xf.pow(2).sum(dim=-1, keepdim=True) / x.shape[-1] + eps)
    return ((xf / rms) * weight.float()).to(x.dtype)


# ------------------------------------------------------------------------------------- rotary
def _rot_pairs(x: torch.Tensor, interleaved: bool) -> torch.Tensor:
    """(-x_odd, x_even) re-interleaved, or (-x_hi, x_lo) concatenated. layers/rope.py:12-18."""
    if interleaved:
        even, odd = x[..., 0::2], x[..., 1::2]
        return torch.stack((-odd, even), dim=-1).flatten(-2)
    lo, hi = x.chunk(2, dim=-1)
    return torch.cat((-hi, lo), dim=-1)


def apply_rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, interleaved: bool = True) -> torch.Tensor:
    """x [B,S,H,D]; cos/sin [S, rot/2] (or [B,S,rot/2], first row used by the HIP path). All products
    are taken in x's dtype exactly as the torch path does. layers/rope.py:21-36."""
    rot = cos.shape[-1] * 2
    assert rot <= x.shape[-1]
    if interleaved:
        cos_f = cos.repeat_interleave(2, dim=-1)
        sin_f = sin.repeat_interleave(2, dim=-1)
    else:
        cos_f = torch.cat((cos, cos), dim=-1)
        sin_f = torch.cat((sin, sin), dim=-1)
    cos_f = cos_f.unsqueeze(-2)  # [..., S, 1, rot]
    sin_f = sin_f.unsqueeze(-2)
    head = x[..., :rot]
    rotated = head * cos_f + _rot_pairs(head, interleaved) * sin_f
    return torch.cat((rotated, x[..., rot:]), dim=-1)


def apply_rotary_complex(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """Independent statement of the interleaved rotation as a complex product, used to cross-check
    ``apply_rotary``: (x0 + i x1) * (cos + i sin). models/qwen_image/pipeline_qwen_image.py:233-238."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    out = torch.view_as_real(xc * freqs.unsqueeze(-2)).flatten(-2)
    return out.type_as(x)


def apply_rotary_wan(x: torch.Tensor, freqs_cos: torch.Tensor, freqs_sin: torch.Tensor) -> torch.Tensor:
    """Wan's rotation: tables are [1,S,1,D] repeat-interleaved; cos read at even, sin at odd columns.
    models/wan2_2/wan2_2_transformer.py:34-56."""
    x1, x2 = x.unflatten(-1, (-1, 2)).unbind(-1)
    cos = freqs_cos[..., 0::2]
    sin = freqs_sin[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = x1 * cos - x2 * sin
    out[..., 1::2] = x1 * sin + x2 * cos
    return out.type_as(x)


# ------------------------------------------------------------------------------------- adaLN
def select_modulation(mod_params: torch.Tensor, index: torch.Tensor | None):
    """shift, scale, gate = chunk(3); with `index` [B,L] the [2B,3C] tensor supplies two candidate
    rows per sample and each token picks row b (index 0) or b+B. layers/adalayernorm.py:23-60."""
    shift, scale, gate = mod_params.chunk(3, dim=-1)
    if index is None:
        return shift.unsqueeze(1), scale.unsqueeze(1), gate.unsqueeze(1)
    nb = shift.size(0) // 2
    pick = (index.unsqueeze(-1) == 0)

    def sel(t):
        return torch.where(pick, t[:nb].unsqueeze(1), t[nb:].unsqueeze(1))

    return sel(shift), sel(scale), sel(gate)


def ada_layer_norm(x: torch.Tensor, mod_params: torch.Tensor, index: torch.Tensor | None = None,
                   eps: float = 1e-6):
    """(LayerNorm(x) * (1 + scale) + shift, gate), LayerNorm without affine. layers/adalayernorm.py:102-110."""
    shift, scale, gate = select_modulation(mod_params, index)
    normed = F.layer_norm(x, (x.shape[-1],), None, None, eps)
    return normed * (1 + scale) + shift, gate


def ada_layer_norm_continuous(x: torch.Tensor, cond: torch.Tensor, weight: torch.Tensor,
                              bias: torch.Tensor | None, eps: float = 1e-6) -> torch.Tensor:
    """diffusers AdaLayerNormContinuous(elementwise_affine=False): emb = Linear(SiLU(cond));
    scale, shift = emb.chunk(2); LN(x) * (1 + scale) + shift. Call site
    models/qwen_image/qwen_image_transformer.py:936, 1065 (third-party; chunk order from upstream, written out
    in the reference tree at model_executor/models/qwen3_tts/tokenizer_25hz/modeling_qwen3_tts_tokenizer_v1.py:492-507)."""
    emb = F.linear(F.silu(cond).to(x.dtype), weight, bias)
    scale, shift = emb.chunk(2, dim=1)
    normed = F.layer_norm(x, (x.shape[-1],), None, None, eps)
    return normed * (1 + scale)[:, None, :] + shift[:, None, :]


def gated_residual(h: torch.Tensor, y: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """h + gate * y. models/qwen_image/qwen_image_transformer.py:794-795, 801, 806."""
    return h + gate * y


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """models/qwen_image/qwen_image_transformer.py:424."""
    return F.gelu(x, approximate="tanh")


# ------------------------------------------------------------------------------------- attention
def sdpa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
         key_mask: torch.Tensor | None = None) -> torch.Tensor:
    """softmax(q k^T * scale) v on BSHD tensors, explicit fp32 softmax, result in q.dtype.

    Same mathematics as the SDPA backend (attention/backends/sdpa.py:73-92: permute to BHSD,
    F.scaled_dot_product_attention, permute back); key_mask [B,Sk] bool excludes keys like the
    key-padding mask of attention/backends/flash_attn.py:80-102.
    """
    qf, kf, vf = (t.permute(0, 2, 1, 3).float() for t in (q, k, v))
    if kf.shape[1] != qf.shape[1]:  # grouped KV heads
        rep = qf.shape[1] // kf.shape[1]
        kf = kf.repeat_interleave(rep, dim=1)
        vf = vf.repeat_interleave(rep, dim=1)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if key_mask is not None:
        s = s.masked_fill(~key_mask.bool()[:, None, None, :], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vf).permute(0, 2, 1, 3).to(q.dtype)


def sdpa_tiled(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, tile: int = 64):
    """Flash-style evaluation over key tiles with the online-softmax rescale; returns (out, lse).
    Identical in exact arithmetic to ``sdpa``; the merge algebra is the one the reference uses for
    ring attention, attention/backends/ring/ring_utils.py:13-89."""
    qf, kf, vf = (t.permute(0, 2, 1, 3).float() for t in (q, k, v))
    B, H, Sq, D = qf.shape
    m = torch.full((B, H, Sq, 1), float("-inf"))
    l = torch.zeros((B, H, Sq, 1))
    acc = torch.zeros((B, H, Sq, D))
    for j in range(0, kf.shape[2], tile):
        s = torch.matmul(qf, kf[:, :, j:j + tile].transpose(-1, -2)) * scale
        m_new = torch.maximum(m, s.amax(dim=-1, keepdim=True))
        alpha = torch.exp(m - m_new)
        p = torch.exp(s - m_new)
        l = l * alpha + p.sum(dim=-1, keepdim=True)
        acc = acc * alpha + torch.matmul(p, vf[:, :, j:j + tile])
        m = m_new
    out = (acc / l).permute(0, 2, 1, 3).to(q.dtype)
    lse = (m + torch.log(l)).squeeze(-1)
    return out, lse


def merge_lse(out_a, lse_a, out_b, lse_b):
    """Combine two partial attentions over disjoint key sets: out - sigmoid(lse_b - lse)(out - out_b)
    with lse = lse_a - logsigmoid(lse_a - lse_b). attention/backends/ring/ring_utils.py:60-89.
    out_* are [B,S,H,D] float, lse_* [B,H,S]."""
    la = lse_a.transpose(1, 2).unsqueeze(-1)
    lb = lse_b.transpose(1, 2).unsqueeze(-1)
    out = out_a - torch.sigmoid(lb - la) * (out_a - out_b)
    lse = la - F.logsigmoid(la - lb)
    return out, lse.squeeze(-1).transpose(1, 2)


# ------------------------------------------------------------------------------------- TeaCache
def rel_l1(cur: torch.Tensor, prev: torch.Tensor) -> float:
    """mean|cur - prev| / (mean|prev| + 1e-8) evaluated op by op in the tensors' dtype and returned
    as a Python float, exactly as cache/teacache/hook.py:214-221 does (for bf16 tensors the
    difference, both means and the quotient are each rounded to bf16)."""
    return ((cur - prev).abs().mean() / (prev.abs().mean() + 1e-8)).cpu().item()


def rel_l1_from_sums(sum_diff: float, sum_prev: float, n: int, dtype: torch.dtype) -> float:
    """The same scalar from the two raw sums, reproducing torch's rounding points: each mean is
    rounded to `dtype`, then + 1e-8 and the division happen in `dtype`."""
    md = torch.tensor(sum_diff / n, dtype=torch.float64).to(torch.float32).to(dtype)
    mp = torch.tensor(sum_prev / n, dtype=torch.float64).to(torch.float32).to(dtype)
    return (md / (mp + 1e-8)).item()


def poly_horner(coeffs, x: float) -> float:
    """Highest-degree-first polynomial, float64 Horner — what numpy.poly1d(coeffs)(x) evaluates.
    cache/teacache/hook.py:62, 224."""
    acc = 0.0
    for c in coeffs:
        acc = acc * x + float(c)
    return acc


def timestep_embedding(t: torch.Tensor, dim: int = 256, flip_sin_to_cos: bool = True,
                       downscale_freq_shift: float = 0.0, scale: float = 1000.0,
                       max_period: int = 10000, cast_freqs: bool = False) -> torch.Tensor:
    """Sinusoidal embedding of (possibly fractional or integer) timesteps, fp32: what diffusers'
    ``Timesteps`` module evaluates at models/qwen_image/qwen_image_transformer.py:163,
    models/flux/flux_transformer.py:462-466 and models/wan2_2/wan2_2_transformer.py:265 (third-party:
    frequencies stay fp32 and multiply ``t.float()``). ``cast_freqs=True`` is the variant of the in-tree
    function models/qwen_image/pipeline_qwen_image.py:141-190, which first casts the frequencies to
    t's dtype; no transformer on this path calls that one."""
    half = dim // 2
    freqs = torch.exp(-math.log(max_period) * torch.arange(half, dtype=torch.float32) / (half - downscale_freq_shift))
    if cast_freqs:
        freqs = freqs.to(t.dtype)
    arg = scale * (t[:, None].float() * freqs[None, :])
    emb = torch.cat((torch.sin(arg), torch.cos(arg)), dim=-1)
    if flip_sin_to_cos:
        emb = torch.cat((emb[:, half:], emb[:, :half]), dim=-1)
    return emb
