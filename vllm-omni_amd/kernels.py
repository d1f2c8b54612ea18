"""Tensor-level wrappers over the C ABI of libomni_dit_hip.so.

Each function validates on the host what the kernel assumes (device, dtype, contiguity of the last
axis, alignment is checked again inside the library), passes raw device pointers, element strides and
torch's current HIP stream, and raises if the library reports an error. Nothing here computes: a
missing library or a CPU tensor is an error, never a fallback.
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import (
    ODIT_EPI_BIAS,
    ODIT_EPI_BIAS_GELU_TANH,
    ODIT_EPI_GATED_RESIDUAL,
    ODIT_EPI_GATED_RESIDUAL_PRE,
    ODIT_EPI_GELU_TANH,
    ODIT_EPI_NONE,
    ODIT_BF16,
    ODIT_F16,
    ODIT_F32,
    ODIT_FLAG_NEOX,
    ODIT_FLAG_REF_ROUNDING,
    ODIT_LINEAR_HANDWRITTEN,
    ODIT_LINEAR_LIBRARY,
    ODIT_NORM_HEAD,
    ODIT_NORM_NONE,
    ODIT_NORM_ROW,
)

_DTYPE_CODE = {torch.bfloat16: ODIT_BF16, torch.float16: ODIT_F16, torch.float32: ODIT_F32}


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected bfloat16, float16 or float32") from None


def _dev(*tensors: torch.Tensor | None) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "omni_dit HIP kernels need tensors on a GPU (got device "
                f"{t.device}); there is no CPU path in this package"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _last_contig(t: torch.Tensor, name: str) -> None:
    if t.stride(-1) != 1:
        raise ValueError(f"{name}: last dimension must be contiguous (stride {t.stride(-1)})")


# Copies this module makes on the caller's behalf where a kernel could not take the operands as given
# (a path whose point is having none): counted so that a model run can assert it made none.
HIDDEN_COPIES: dict[str, int] = {"attn_value_pair_concatenated": 0, "made_contiguous": 0}


# --------------------------------------------------------------------------------------------- K1
def attn_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor | tuple[torch.Tensor, torch.Tensor],
    scale: float,
    key_mask: torch.Tensor | None = None,
    return_lse: bool = False,
    split: int | None = None,
    use_workspace: bool = True,
):
    """softmax(q k^T * scale) v for q [B,Sq,H,D], k/v [B,Sk,Hkv,D] (BSHD, bf16/fp16).

    ``v`` may be a pair (v_head [B,s,Hkv,D], v_tail [B,Sk-s,Hkv,D]) holding the value rows of keys
    [0, s) and [s, Sk): the kernel reads both in place when s is a multiple of 64 and they share their
    row stride (two fused-QKV projection outputs do); otherwise they are concatenated first.

    key_mask: optional [B,Sk] bool/uint8, False/0 = key excluded. Returns o [B,Sq,H,D]
    (and lse [B,H,Sq] float32 when return_lse). With ``split`` = s the output comes back as two dense
    tensors (o[:, :s], o[:, s:]) written directly by the kernel. ``use_workspace=False`` keeps the launch
    from cutting its last round of workgroups along the keys (no scratch buffer, one kernel).
    """
    v_tail = None
    if isinstance(v, (tuple, list)):
        v, v_tail = v
        if v.dim() != 4 or v_tail.dim() != 4 or k.dim() != 4 or v.shape[1] + v_tail.shape[1] != k.shape[1]:
            raise ValueError(f"value pair {tuple(v.shape)} + {tuple(v_tail.shape)} does not cover k {tuple(k.shape)}")
        direct = (v.dim() == 4 and v_tail.dim() == 4 and v.shape[1] % 64 == 0 and 0 < v.shape[1] and v_tail.shape[1] > 0
                  and v.stride(1) == v_tail.stride(1) and v.dtype == v_tail.dtype
                  and all(t.stride(-1) == 1 and all(x % 8 == 0 for x in t.stride()[:3]) and t.data_ptr() % 16 == 0
                          for t in (v, v_tail)))
        if not direct:
            HIDDEN_COPIES["attn_value_pair_concatenated"] += 1
            v, v_tail = torch.cat([v, v_tail], dim=1), None
    _dev(q, k, v, v_tail, key_mask)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("attn_fwd expects 4-D [B,S,H,D] tensors")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k, v must share a dtype")
    B, Sq, H, D = q.shape
    Bk, Sk, Hkv, Dk = k.shape
    k_split = 0
    if v_tail is not None:
        k_split = v.shape[1]
        if (v.shape[0], v.shape[2], v.shape[3]) != (B, Hkv, D) or tuple(v_tail.shape) != (B, Sk - k_split, Hkv, D):
            raise ValueError(f"value pair {tuple(v.shape)} + {tuple(v_tail.shape)} does not cover k {tuple(k.shape)}")
    elif (Bk, Dk) != (B, D) or tuple(v.shape) != tuple(k.shape):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if Bk != B or Dk != D:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}")

    def _prep(t):
        ok = t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:3]) and t.data_ptr() % 16 == 0
        if not ok:
            HIDDEN_COPIES["made_contiguous"] += 1
        return t if ok else t.contiguous()

    q, k = _prep(q), _prep(k)
    if v_tail is None:
        v = _prep(v)
    if split is not None and not 0 <= split <= Sq:
        raise ValueError(f"split={split} outside [0, {Sq}]")
    o = torch.empty((B, Sq if split is None else split, H, D), dtype=q.dtype, device=q.device)
    o_tail = None if split is None else torch.empty((B, Sq - split, H, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device) if return_lse else None
    mask_u8 = None
    if key_mask is not None:
        if tuple(key_mask.shape) != (B, Sk):
            raise ValueError(f"key_mask must be [B,Sk]={B, Sk}, got {tuple(key_mask.shape)}")
        mask_u8 = (key_mask != 0).to(torch.uint8).contiguous()
    lib = _lib.load()
    # dense [B, n, H, D] strides even when n == 0 or B == 1 (torch may report arbitrary ones there)
    if split is None or split == Sq:
        head_t, tail_t, cut = o, None, 0
    elif split == 0:  # the first output is empty: everything goes to the second
        head_t, tail_t, cut = o_tail, None, 0
    else:
        head_t, tail_t, cut = o, o_tail, int(split)
    n_head = head_t.shape[1]
    o_str = (n_head * H * D, H * D, D)
    t_str = None if tail_t is None else _lib.i64_array(((Sq - cut) * H * D, H * D, D))
    ws = _attn_workspace(lib, q.device, B, Sq, Sk, H, D) if use_workspace else None
    rc = lib.odit_attn_fwd_ex(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), _ptr(v_tail), k_split, head_t.data_ptr(), _ptr(tail_t), cut,
        _ptr(mask_u8), _ptr(lse), B, Sq, Sk, H, Hkv, D,
        _lib.i64_array(q.stride()[:3]), _lib.i64_array(k.stride()[:3]),
        _lib.i64_array(v.stride()[:3]), None if v_tail is None else _lib.i64_array(v_tail.stride()[:3]),
        _lib.i64_array(o_str), t_str,
        float(scale), _code(q), _ptr(ws), 0 if ws is None else ws.numel(), _stream(),
    )
    if rc == -2 and v_tail is not None:  # ODIT_ENOTSUP: spans too large for the kernel that reads value pairs
        HIDDEN_COPIES["attn_value_pair_concatenated"] += 1
        return attn_fwd(q, k, torch.cat([v, v_tail], dim=1), scale, key_mask=key_mask, return_lse=return_lse,
                        split=split, use_workspace=use_workspace)
    _lib.check(rc, "odit_attn_fwd_ex")
    if split is None:
        return (o, lse) if return_lse else o
    return (o, o_tail, lse) if return_lse else (o, o_tail)


def attn_plan(B: int, Sq: int, Sk: int, H: int, D: int, k_seq_stride: int | None = None,
              v_seq_stride: int | None = None, use_workspace: bool = True) -> str:
    """The launches ``attn_fwd`` makes for a problem, as "<kernel> units=<n>" joined by "; " (kernel names as
    a profiler reports them). Strides default to those of dense [B,S,H,D] tensors."""
    lib = _lib.load()
    buf = _lib.C.create_string_buffer(512)
    dense = H * D
    rc = lib.odit_attn_fwd_plan(B, Sq, Sk, H, D, dense if k_seq_stride is None else int(k_seq_stride),
                                dense if v_seq_stride is None else int(v_seq_stride), int(use_workspace), buf, 512)
    if rc < 0:
        _lib.check(rc, "odit_attn_fwd_plan")
    return buf.value.decode()


_ATTN_SCRATCH: dict[tuple[int, int], torch.Tensor] = {}


def _attn_workspace(lib, device: torch.device, B: int, Sq: int, Sk: int, H: int, D: int) -> torch.Tensor | None:
    """Scratch for the key-split tail of the attention launch, one growing buffer per (device, stream):
    launches on one stream are ordered, so they can share it."""
    need = int(lib.odit_attn_fwd_workspace_bytes(B, Sq, Sk, H, D))
    if need == 0:
        return None
    key = (device.index or 0, _stream())
    ws = _ATTN_SCRATCH.get(key)
    if ws is None or ws.numel() < need:
        # zero-filled once: the first kilobyte holds the ticket words the persistent kernel draws its units from
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _ATTN_SCRATCH[key] = ws
    return ws


# --------------------------------------------------------------------------------------------- K2
def qknorm_rope(
    q: torch.Tensor,
    k: torch.Tensor | None,
    v: torch.Tensor | None,
    q_out: torch.Tensor,
    k_out: torch.Tensor | None,
    v_out: torch.Tensor | None,
    wq: torch.Tensor | None,
    wk: torch.Tensor | None,
    cos: torch.Tensor | None,
    sin: torch.Tensor | None,
    *,
    eps: float = 1e-6,
    out_seq_offset: int = 0,
    norm_mode: int = ODIT_NORM_HEAD,
    neox: bool = False,
    ref_rounding: bool = False,
) -> None:
    """RMS-normalise q,k (per head or per row), rotate them, and write q,k,v rows into joint buffers.

    q,k,v: [B,S,H,D] views sharing (batch, seq) strides with heads D apart (e.g. the three slices of
    a fused-QKV projection). *_out: dense [B,S_total,H,D]; input row s goes to row out_seq_offset+s.
    cos/sin: float32 [S, rot/2] or None.
    """
    B, S, H, D, S_total, rot, w_dtype, cos, sin = _qk_problem(q, k, v, q_out, k_out, v_out, wq, wk, cos, sin, norm_mode)
    flags = (ODIT_FLAG_NEOX if neox else 0) | (ODIT_FLAG_REF_ROUNDING if ref_rounding else 0)
    lib = _lib.load()
    rc = lib.odit_qknorm_rope(
        q.data_ptr(), _ptr(k), _ptr(v), q_out.data_ptr(), _ptr(k_out), _ptr(v_out),
        _ptr(wq), _ptr(wk), _ptr(cos), _ptr(sin),
        B, S, H, D, rot, _lib.i64_array(q.stride()[:2]), int(out_seq_offset), int(S_total),
        float(eps), int(norm_mode), w_dtype, _code(q), flags, _stream(),
    )
    _lib.check(rc, "odit_qknorm_rope")


def _qk_problem(q, k, v, q_out, k_out, v_out, wq, wk, cos, sin, norm_mode):
    """Checks of one qknorm_rope problem; returns (B, S, H, D, S_total, rot, w_dtype, cos, sin)."""
    _dev(q, k, v, q_out, k_out, v_out, wq, wk, cos, sin)
    if q.dim() != 4:
        raise ValueError("qknorm_rope expects [B,S,H,D] inputs")
    B, S, H, D = q.shape
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t is None:
            continue
        if tuple(t.shape) != (B, S, H, D) or t.dtype != q.dtype:
            raise ValueError(f"{name}: expected shape {(B, S, H, D)} and dtype {q.dtype}")
        if t.stride(3) != 1 or t.stride(2) != D:
            raise ValueError(f"{name}: heads must be laid out D apart with a contiguous last axis")
        if t.stride()[:2] != q.stride()[:2]:
            raise ValueError(f"{name}: (batch, seq) strides must match q's")
    S_total = q_out.shape[1]
    for name, t, src in (("q_out", q_out, q), ("k_out", k_out, k), ("v_out", v_out, v)):
        if (t is None) != (src is None):
            raise ValueError(f"{name} must be given exactly when its input is")
        if t is None:
            continue
        if tuple(t.shape) != (B, S_total, H, D) or t.dtype != q.dtype or not t.is_contiguous():
            raise ValueError(f"{name}: expected dense {(B, S_total, H, D)} of {q.dtype}")
    rot = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[0] != S:
            raise ValueError("cos/sin must both be [S, rot/2]")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32:
            raise TypeError("cos/sin must be float32")
        cos, sin = cos.contiguous(), sin.contiguous()
        rot = 2 * cos.shape[1]
    w_dtype = _code(q)
    if norm_mode != ODIT_NORM_NONE:
        for name, w in (("wq", wq), ("wk", wk)):
            if w is None:
                continue
            want = D if norm_mode == ODIT_NORM_HEAD else H * D
            if w.numel() != want or not w.is_contiguous():
                raise ValueError(f"{name}: expected {want} contiguous elements")
        ws = [w for w in (wq, wk) if w is not None]
        if ws:
            if any(w.dtype != ws[0].dtype for w in ws):
                raise TypeError("wq and wk must share a dtype")
            w_dtype = _code(ws[0])
    return B, S, H, D, S_total, rot, w_dtype, cos, sin


def qknorm_rope_pair(first: tuple, second: tuple, q_out: torch.Tensor, k_out: torch.Tensor | None,
                     v_out: torch.Tensor | None, *, eps: float = 1e-6, norm_mode: int = ODIT_NORM_HEAD,
                     neox: bool = False, ref_rounding: bool = False) -> None:
    """Two ``qknorm_rope`` problems that fill different rows of the same joint buffers (the text rows and
    the image rows of a dual-stream block) in ONE launch. Each problem is
    (q, k, v, wq, wk, cos, sin, out_seq_offset) with the meaning of ``qknorm_rope``'s arguments; both take the
    same optional operands, head layout, rotary width and dtypes."""
    probs = []
    for (q, k, v, wq, wk, cos, sin, off) in (first, second):
        B, S, H, D, S_total, rot, w_dtype, cos, sin = _qk_problem(
            q, k, v, q_out, k_out if k is not None else None, v_out if v is not None else None, wq, wk, cos, sin,
            norm_mode)
        probs.append(dict(q=q, k=k, v=v, wq=wq, wk=wk, cos=cos, sin=sin, off=int(off), S=S,
                          shared=(B, H, D, S_total, rot, w_dtype, q.dtype)))
    a, b = probs
    if a["shared"] != b["shared"]:
        raise ValueError("qknorm_rope_pair: the two problems must share batch, heads, rotary width and dtypes")
    for name in ("k", "v", "cos"):
        if (a[name] is None) != (b[name] is None):
            raise ValueError(f"qknorm_rope_pair: both problems take {name} or neither does")
    B, H, D, S_total, rot, w_dtype, _ = a["shared"]

    def both(name):  # the two problems' device addresses of one operand
        return _lib.ptr_array([_ptr(a[name]), _ptr(b[name])])

    flags = (ODIT_FLAG_NEOX if neox else 0) | (ODIT_FLAG_REF_ROUNDING if ref_rounding else 0)
    lib = _lib.load()
    rc = lib.odit_qknorm_rope_pair(
        both("q"), both("k"), both("v"), q_out.data_ptr(), _ptr(k_out), _ptr(v_out),
        both("wq"), both("wk"), both("cos"), both("sin"),
        B, _lib.int_array([a["S"], b["S"]]), H, D, rot,
        _lib.i64_array(tuple(a["q"].stride()[:2]) + tuple(b["q"].stride()[:2])), _lib.int_array([a["off"], b["off"]]),
        int(S_total), float(eps), int(norm_mode), w_dtype, _code(a["q"]), flags, _stream(),
    )
    _lib.check(rc, "odit_qknorm_rope_pair")


# --------------------------------------------------------------------------------------------- K3
def adaln_modulate(
    x: torch.Tensor,
    shift: torch.Tensor | None,
    scale: torch.Tensor | None,
    *,
    eps: float = 1e-6,
    index: torch.Tensor | None = None,
    ln_weight: torch.Tensor | None = None,
    ln_bias: torch.Tensor | None = None,
    shift_bias: torch.Tensor | None = None,
    scale_bias: torch.Tensor | None = None,
    ref_rounding: bool = False,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """LayerNorm(x) * (1 + scale) + shift for x [B,S,C]; shift/scale [Bm,C] views of one modulation
    tensor (Bm = B, or 2B with a per-token `index` [B,S] choosing row b or b+B), or [B,S,C] views with
    one row per token. ``shift_bias`` / ``scale_bias``: float32 [C] tables added to the rows in fp32."""
    _dev(x, shift, scale, index, ln_weight, ln_bias, shift_bias, scale_bias, out)
    if x.dim() != 3:
        raise ValueError("adaln_modulate expects x [B,S,C]")
    B, S, Cdim = x.shape
    _last_contig(x, "x")
    mod_dtype = _code(x)
    mod_stride, mod_stride_s = 0, 0
    rows_needed = 2 * B if index is not None else B
    first = shift if shift is not None else scale
    per_token = first is not None and first.dim() == 3
    if per_token and index is not None:
        raise ValueError("per-token shift/scale rows and an index exclude each other")
    for name, t in (("shift", shift), ("scale", scale)):
        if t is None:
            continue
        if per_token:
            if tuple(t.shape) != (B, S, Cdim):
                raise ValueError(f"{name}: expected [{B},{S},{Cdim}], got {tuple(t.shape)}")
        elif t.dim() != 2 or t.shape[1] != Cdim or t.shape[0] < rows_needed:
            raise ValueError(f"{name}: expected [{rows_needed},{Cdim}], got {tuple(t.shape)}")
        _last_contig(t, name)
        mod_dtype = _code(t)
    if shift is not None and scale is not None:
        if shift.dtype != scale.dtype or shift.stride()[:-1] != scale.stride()[:-1]:
            raise ValueError("shift and scale must share dtype and strides")
    if first is not None:
        mod_stride = first.stride(0) if first.shape[0] > 1 else 0
        if per_token:
            mod_stride_s = first.stride(1) if S > 1 else Cdim
            if mod_stride_s == 0:  # an expanded row: the same as one row per batch entry
                per_token = False
        elif first.shape[0] == 1:
            mod_stride = first.shape[1]
    if index is not None:
        if tuple(index.shape) != (B, S):
            raise ValueError(f"index must be [B,S]={B, S}")
        index = index.to(torch.int32).contiguous()
    for name, t in (("ln_weight", ln_weight), ("ln_bias", ln_bias), ("shift_bias", shift_bias),
                    ("scale_bias", scale_bias)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != Cdim or t.dim() == 0 or t.stride(-1) != 1
                              or t.numel() != t.shape[-1]):
            raise ValueError(f"{name}: expected float32 [{Cdim}] with unit stride")
    if out is None:
        out = torch.empty((B, S, Cdim), dtype=x.dtype, device=x.device)
    elif tuple(out.shape) != (B, S, Cdim) or out.dtype != x.dtype or out.stride(-1) != 1:
        raise ValueError("out must match x in shape and dtype with a contiguous last axis")
    lib = _lib.load()
    rc = lib.odit_adaln_modulate(
        x.data_ptr(), out.data_ptr(), _ptr(shift), _ptr(scale), _ptr(index), _ptr(ln_weight),
        _ptr(ln_bias), _ptr(shift_bias), _ptr(scale_bias), B, S, Cdim, _lib.i64_array(x.stride()[:2]),
        _lib.i64_array(out.stride()[:2]), int(mod_stride), int(mod_stride_s), float(eps), mod_dtype, _code(x),
        ODIT_FLAG_REF_ROUNDING if ref_rounding else 0, _stream(),
    )
    _lib.check(rc, "odit_adaln_modulate")
    return out


def adaln_modulate_pair(first: tuple, second: tuple, *, eps: float = 1e-6,
                        ref_rounding: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """``adaln_modulate`` for two tensors of the same width and batch (the image and the text stream of a
    dual-stream block) in ONE launch. Each problem is (x [B,S,C], shift [B,C], scale [B,C]): one modulation row per
    batch entry; returns the two results."""
    probs = []
    for (x, shift, scale) in (first, second):
        _dev(x, shift, scale)
        if x.dim() != 3:
            raise ValueError("adaln_modulate_pair expects x [B,S,C]")
        B, S, Cdim = x.shape
        _last_contig(x, "x")
        for name, t in (("shift", shift), ("scale", scale)):
            if t is None or t.dim() != 2 or tuple(t.shape) != (B, Cdim):
                raise ValueError(f"{name}: expected [{B},{Cdim}]")
            _last_contig(t, name)
        if shift.dtype != scale.dtype or shift.stride(0) != scale.stride(0):
            raise ValueError("shift and scale must share dtype and strides")
        probs.append(dict(x=x, out=torch.empty((B, S, Cdim), dtype=x.dtype, device=x.device), shift=shift, scale=scale,
                          S=S, mod_stride=shift.stride(0) if B > 1 else 0, shared=(B, Cdim, x.dtype, shift.dtype)))
    a, b = probs
    if a["shared"] != b["shared"]:
        raise ValueError("adaln_modulate_pair: the two problems must share batch, width and dtypes")
    B, Cdim = a["shared"][:2]

    def both(name):
        return _lib.ptr_array([a[name].data_ptr(), b[name].data_ptr()])

    def strides(name):  # (batch, seq) strides of both problems, side by side
        return _lib.i64_array(tuple(a[name].stride()[:2]) + tuple(b[name].stride()[:2]))

    lib = _lib.load()
    rc = lib.odit_adaln_modulate_pair(
        both("x"), both("out"), both("shift"), both("scale"), B, _lib.int_array([a["S"], b["S"]]), Cdim,
        strides("x"), strides("out"), _lib.i64_array([a["mod_stride"], b["mod_stride"]]), float(eps),
        _code(a["shift"]), _code(a["x"]), ODIT_FLAG_REF_ROUNDING if ref_rounding else 0, _stream(),
    )
    _lib.check(rc, "odit_adaln_modulate_pair")
    return a["out"], b["out"]


# --------------------------------------------------------------------------------------------- K4
def gated_residual(
    h: torch.Tensor,
    y: torch.Tensor,
    gate: torch.Tensor | None,
    *,
    out: torch.Tensor | None = None,
    ref_rounding: bool = False,
    gate_bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """h + gate * y for h,y [B,S,C]; gate [B,C], [B,1,C] (broadcast over S) or [B,S,C]; None = ones.
    ``gate_bias``: float32 [C] table added to the gate in fp32 (alone it is the gate)."""
    _dev(h, y, gate, out, gate_bias)
    if gate_bias is not None and (gate_bias.dtype != torch.float32 or gate_bias.numel() != h.shape[-1]
                                  or gate_bias.stride(-1) != 1 or gate_bias.numel() != gate_bias.shape[-1]):
        raise ValueError(f"gate_bias: expected float32 [{h.shape[-1]}] with unit stride")
    if h.dim() != 3 or tuple(y.shape) != tuple(h.shape) or y.dtype != h.dtype:
        raise ValueError("gated_residual expects h and y of identical [B,S,C] shape and dtype")
    B, S, Cdim = h.shape
    _last_contig(h, "h")
    _last_contig(y, "y")
    gate_dtype = _code(h)
    gs = (0, 0)
    if gate is not None:
        _last_contig(gate, "gate")
        gate_dtype = _code(gate)
        if gate.dim() == 2 and tuple(gate.shape) == (B, Cdim):
            gs = (gate.stride(0) if B > 1 else 0, 0)
        elif gate.dim() == 3 and gate.shape[0] == B and gate.shape[2] == Cdim and gate.shape[1] in (1, S):
            gs = (gate.stride(0) if B > 1 else 0, gate.stride(1) if gate.shape[1] == S and S > 1 else 0)
        else:
            raise ValueError(f"gate shape {tuple(gate.shape)} does not broadcast against {(B, S, Cdim)}")
    if out is None:
        out = torch.empty_like(h, memory_format=torch.contiguous_format)
    elif tuple(out.shape) != tuple(h.shape) or out.dtype != h.dtype or out.stride(-1) != 1:
        raise ValueError("out must match h in shape and dtype with a contiguous last axis")
    lib = _lib.load()
    rc = lib.odit_gated_residual(
        h.data_ptr(), y.data_ptr(), _ptr(gate), _ptr(gate_bias), out.data_ptr(), B, S, Cdim,
        _lib.i64_array(h.stride()[:2]), _lib.i64_array(y.stride()[:2]),
        _lib.i64_array(out.stride()[:2]), _lib.i64_array(gs), gate_dtype, _code(h),
        ODIT_FLAG_REF_ROUNDING if ref_rounding else 0, _stream(),
    )
    _lib.check(rc, "odit_gated_residual")
    return out


# --------------------------------------------------------------------------------------------- K5
_REL_L1_SCRATCH: dict[tuple[int, int], torch.Tensor] = {}


def rel_l1_sums(cur: torch.Tensor, prev: torch.Tensor, *, ref_rounding: bool = True) -> torch.Tensor:
    """Per-batch-row (sum |cur - prev|, sum |prev|) as a float64 [B,2] DEVICE tensor (no sync)."""
    _dev(cur, prev)
    if cur.shape != prev.shape or cur.dtype != prev.dtype or cur.dim() < 1:
        raise ValueError("rel_l1_sums expects two tensors of identical shape and dtype")
    B = cur.shape[0]
    c2 = cur.reshape(B, -1)
    p2 = prev.reshape(B, -1)
    if c2.stride(-1) != 1:
        c2 = c2.contiguous()
    if p2.stride(-1) != 1:
        p2 = p2.contiguous()
    n = c2.shape[1]
    lib = _lib.load()
    need = int(lib.odit_rel_l1_workspace_bytes(B, n))
    key = (cur.device.index or 0, _stream())  # launches on one stream are ordered and can share it
    ws = _REL_L1_SCRATCH.get(key)
    if ws is None or ws.numel() < need:
        # zero-filled once: the ticket words live in a region of fixed size at the start
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=cur.device)
        _REL_L1_SCRATCH[key] = ws
    sums = torch.empty((B, 2), dtype=torch.float64, device=cur.device)
    rc = lib.odit_rel_l1(
        c2.data_ptr(), p2.data_ptr(), sums.data_ptr(), ws.data_ptr(), ws.numel(), B, n,
        c2.stride(0) if B > 1 else n, p2.stride(0) if B > 1 else n, _code(cur),
        ODIT_FLAG_REF_ROUNDING if ref_rounding else 0, _stream(),
    )
    _lib.check(rc, "odit_rel_l1")
    return sums


# ------------------------------------------------------------------------------------- activations
def _unary(name: str, x: torch.Tensor, out: torch.Tensor | None) -> torch.Tensor:
    _dev(x, out)
    if not x.is_contiguous():
        x = x.contiguous()
    if out is None:
        out = torch.empty_like(x)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor matching x")
    lib = _lib.load()
    rc = getattr(lib, name)(x.data_ptr(), out.data_ptr(), x.numel(), _code(x), _stream())
    _lib.check(rc, name)
    return out


def gelu_tanh(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    return _unary("odit_gelu_tanh", x, out)


def silu(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    return _unary("odit_silu", x, out)


# --------------------------------------------------------------------------------------------- GEMM
_LINEAR_SCRATCH: dict[tuple[int, int], torch.Tensor] = {}
_LINEAR_AUTOTUNE_ITERS = 0
_LINEAR_TUNED: dict[tuple, float] = {}


_FLUSH_BYTES = 512 << 20  # twice the 256 MB last-level cache
_FLUSH: dict[int, torch.Tensor] = {}


def _flush_buffer(device: torch.device) -> int:
    """Device buffer the tuning call overwrites between timed launches; released by set_linear_autotune(0)."""
    idx = device.index or 0
    if idx not in _FLUSH:
        _FLUSH[idx] = torch.empty(_FLUSH_BYTES, dtype=torch.uint8, device=device)
    return _FLUSH[idx].data_ptr()


def set_linear_autotune(iters: int) -> None:
    """With iters > 0, the first ``linear`` call of every new problem (shape, strides, epilogue, dtype)
    first times the library's kernels for it on scratch copies of the output operands (a blocking,
    one-off cost of some tenths of a second) and keeps the fastest for the rest of the process. Meant to
    be switched on around a warm-up pass and off again; 0 = use the library's own first choice for
    problems not tuned yet."""
    global _LINEAR_AUTOTUNE_ITERS
    _LINEAR_AUTOTUNE_ITERS = int(iters)
    if _LINEAR_AUTOTUNE_ITERS <= 0:
        _FLUSH.clear()


_LINEAR_ENGINES = {"auto": 0, "library": ODIT_LINEAR_LIBRARY, "handwritten": ODIT_LINEAR_HANDWRITTEN}
_LINEAR_ENGINE_FLAGS = 0


def set_linear_engine(engine: str) -> None:
    """Which kernel later ``linear`` calls of this process ask for when they name none themselves: "auto" (a
    hand-written kernel where a tuning run found it faster or its default rule says so, the library
    elsewhere), "library" (hipBLASLt always) or "handwritten" (the hand-written kernel for the row count
    always; problems it does not take raise). The choice travels with every call as a flag of
    ``odit_linear_rows``; the library keeps no switch. For measurements and tests."""
    global _LINEAR_ENGINE_FLAGS
    if engine not in _LINEAR_ENGINES:
        raise ValueError(f"engine must be one of {sorted(_LINEAR_ENGINES)}")
    _LINEAR_ENGINE_FLAGS = _LINEAR_ENGINES[engine]


def linear_tuning_report() -> dict[tuple, float]:
    """{problem key: best time in microseconds} of everything tuned so far in this process."""
    return dict(_LINEAR_TUNED)


def _linear_workspace(lib, device: torch.device) -> torch.Tensor:
    key = (device.index or 0, _stream())
    ws = _LINEAR_SCRATCH.get(key)
    if ws is None:
        # zero-filled once: the stream-K kernel keeps its ticket words at the start
        ws = torch.zeros(int(lib.odit_linear_workspace_bytes()), dtype=torch.uint8, device=device)
        _LINEAR_SCRATCH[key] = ws
    return ws


def _rows2d(t: torch.Tensor, name: str) -> tuple[torch.Tensor, int]:
    """View of t as rows of its last axis with one row stride; returns (2-D view, row stride)."""
    if t.stride(-1) != 1:
        raise ValueError(f"{name}: last dimension must be contiguous")
    t2 = t.reshape(-1, t.shape[-1]) if t.is_contiguous() else (t if t.dim() == 2 else None)
    if t2 is None:
        raise ValueError(f"{name}: needs a contiguous tensor or a 2-D view with a row stride")
    return t2, (t2.stride(0) if t2.shape[0] > 1 else t2.shape[1])


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *, activation: str | None = None,
           residual: torch.Tensor | None = None, gate: torch.Tensor | None = None, out: torch.Tensor | None = None,
           gate_bias: torch.Tensor | None = None, prescaled: bool = False, tune_iters: int = 0,
           plan_only: bool = False, engine: str | None = None):
    """x W^T (+ bias) with the elementwise tail inside the GEMM's epilogue.

    activation="gelu_tanh": GELU(tanh) of the result. residual (same shape as the result) with optional
    gate [B,N] / [B,1,N] / [N]: ``residual + gate * (x W^T + bias)``; gates that differ per batch row go
    down as one call (one launch of the hand-written kernel, or one library launch per batch row). ``prescaled=True``: ``gate`` is float32 and ``gate_bias`` (float32, same shape, or
    None) already holds gate * bias — nothing is derived per call (``bias`` is then ignored).
    ``weight`` may be a column range of a Linear weight (row stride > K).
    ``tune_iters`` > 0 first times the library's kernels and the hand-written kernel for this problem
    (overwrites ``out``), keeps the faster for later calls and returns its time in microseconds instead
    of the result. ``plan_only`` launches nothing and returns (the hand-written kernel would run, number of
    kernel launches the call would make). ``engine``: "auto", "library" or "handwritten" for this call
    (default: what ``set_linear_engine`` chose).
    """
    if engine is not None and engine not in _LINEAR_ENGINES:
        raise ValueError(f"engine must be one of {sorted(_LINEAR_ENGINES)}")
    eflags = _LINEAR_ENGINE_FLAGS if engine is None else _LINEAR_ENGINES[engine]
    _dev(x, weight, bias, residual, gate, out)
    if weight.dim() != 2 or weight.stride(1) != 1 or x.shape[-1] != weight.shape[1]:
        raise ValueError(f"weight must be [N,K] rows with K = {x.shape[-1]}, got {tuple(weight.shape)}")
    if x.dtype != weight.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("x, weight and bias must share a dtype")
    N, K = weight.shape
    x2, ldx = _rows2d(x, "x")
    M = x2.shape[0]
    out_shape = (*x.shape[:-1], N)
    if out is None:
        out = (residual if plan_only and residual is not None
               else torch.empty(out_shape, dtype=x.dtype, device=x.device))
    elif tuple(out.shape) != out_shape or out.dtype != x.dtype:
        raise ValueError(f"out must be {out_shape} of {x.dtype}")
    o2, ldo = _rows2d(out, "out")
    if bias is not None and (bias.numel() != N or not bias.is_contiguous()):
        raise ValueError(f"bias must be contiguous [{N}]")
    lib = _lib.load()
    ws = _linear_workspace(lib, x.device)
    ldw = weight.stride(0) if N > 1 else K
    best = _lib.C.c_float(0.0)
    plan = [_lib.C.c_int(0), _lib.C.c_int(0)]

    def call(rp, gp, epi, gate_code, bp=_ptr(bias), rows_per_gate=0, gate_stride=0, row0=0, M=M):
        esz = x.element_size()
        prob = (x2.data_ptr() + row0 * ldx * esz, weight.data_ptr(), bp, o2.data_ptr() + row0 * ldo * esz,
                None if rp is None else rp + row0 * ldr * esz, gp, M, N, K, ldx, ldw, ldo, ldr, epi, gate_code,
                _code(x), rows_per_gate, gate_stride)
        if plan_only:
            _lib.check(lib.odit_linear_rows_plan(*prob, eflags, ws.data_ptr(), ws.numel(), _lib.C.byref(plan[0]),
                                                 _lib.C.byref(plan[1])), "odit_linear_rows_plan")
            return
        if _LINEAR_AUTOTUNE_ITERS > 0 and tune_iters == 0:
            key = (x.device.index or 0, M, N, K, epi, bp is not None, gp is not None, _code(x), ldx, ldw, ldo, ldr,
                   rows_per_gate)
            if key not in _LINEAR_TUNED:
                # time the candidates on scratch output operands: tuning overwrites (and, for the residual
                # forms, keeps accumulating into) whatever it is given
                t_out = torch.empty((M, ldo), dtype=x.dtype, device=x.device)
                t_res = torch.zeros((M, max(ldr, 1)), dtype=x.dtype, device=x.device) if rp is not None else None
                t_best = _lib.C.c_float(0.0)
                t_prob = prob[:3] + (t_out.data_ptr(), _ptr(t_res)) + prob[5:]
                _lib.check(lib.odit_linear_rows_tune(*t_prob, ws.data_ptr(), ws.numel(), _stream(),
                                                     _LINEAR_AUTOTUNE_ITERS, _flush_buffer(x.device), _FLUSH_BYTES,
                                                     _lib.C.byref(t_best), None), "odit_linear_rows_tune")
                _LINEAR_TUNED[key] = t_best.value
        if tune_iters > 0:
            _lib.check(lib.odit_linear_rows_tune(*prob, ws.data_ptr(), ws.numel(), _stream(), int(tune_iters),
                                                 _flush_buffer(x.device), _FLUSH_BYTES, _lib.C.byref(best), None),
                       "odit_linear_rows_tune")
        else:
            _lib.check(lib.odit_linear_rows(*prob, eflags, ws.data_ptr(), ws.numel(), _stream()), "odit_linear_rows")

    ldr = 0
    if residual is None:
        if gate is not None:
            raise ValueError("gate needs a residual")
        if activation is None:
            epi = ODIT_EPI_BIAS if bias is not None else ODIT_EPI_NONE
        elif activation == "gelu_tanh":
            epi = ODIT_EPI_BIAS_GELU_TANH if bias is not None else ODIT_EPI_GELU_TANH
        else:
            raise ValueError(f"unknown activation {activation!r}")
        call(None, None, epi, _code(x))
        if plan_only:
            return bool(plan[0].value), plan[1].value
        return best.value if tune_iters > 0 else out
    if activation is not None:
        raise ValueError("activation and residual cannot be combined")
    if tuple(residual.shape) != out_shape or residual.dtype != x.dtype:
        raise ValueError(f"residual must be {out_shape} of {x.dtype}")
    r2, ldr = _rows2d(residual, "residual")
    if gate is None or gate.dim() == 1:
        rows, g2 = 0, (None if gate is None else gate.reshape(1, N))
    else:
        B = x.shape[0]
        g2 = gate.reshape(B, N) if gate.numel() == B * N else None
        if g2 is None or x.dim() < 2:
            raise ValueError(f"gate shape {tuple(gate.shape)} does not give one row of {N} per batch row")
        rows = M // B if B > 1 else 0
    if g2 is not None:
        _last_contig(g2, "gate")
        if g2.dtype not in (x.dtype, torch.float32):
            raise TypeError("gate must have x's dtype or float32")
    gstride = g2.stride(0) if (g2 is not None and rows > 0) else 0
    if prescaled:
        if g2 is None or g2.dtype != torch.float32:
            raise TypeError("prescaled=True needs a float32 gate")
        gb2 = None
        if gate_bias is not None:
            gb2 = gate_bias.reshape(g2.shape)
            _last_contig(gb2, "gate_bias")
            if gb2.dtype != torch.float32:
                raise TypeError("gate_bias must be float32")
        if rows > 0 and gb2 is not None and gb2.stride(0) != gstride:
            # gate and gate * bias rows laid out differently: one call per batch row
            for b in range(g2.shape[0]):
                call(r2.data_ptr(), g2[b].data_ptr(), ODIT_EPI_GATED_RESIDUAL_PRE, ODIT_F32, gb2[b].data_ptr(),
                     row0=b * rows, M=rows)
                if tune_iters > 0 or plan_only:
                    break  # every batch row is the same problem
        else:
            call(r2.data_ptr(), g2.data_ptr(), ODIT_EPI_GATED_RESIDUAL_PRE, ODIT_F32, _ptr(gb2), rows, gstride)
    else:
        call(r2.data_ptr(), _ptr(g2), ODIT_EPI_GATED_RESIDUAL, _code(x) if g2 is None else _code(g2), _ptr(bias), rows,
             gstride)
    if plan_only:
        return bool(plan[0].value), plan[1].value
    return best.value if tune_iters > 0 else out
