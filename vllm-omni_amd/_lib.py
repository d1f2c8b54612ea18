"""ctypes binding of libomni_dit_hip.so (the C ABI declared in include/omni_dit.h).

The library is looked up next to this file only: it is built in-tree by ``csrc/build.py`` and travels
with the source tree. There is no fallback implementation — if the library is missing, every kernel
entry point raises :class:`OmniDitLibraryError`.
"""

from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

LIB_NAME = "libomni_dit_hip.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

ODIT_BF16, ODIT_F16, ODIT_F32 = 0, 1, 2
ODIT_FLAG_REF_ROUNDING = 1
ODIT_FLAG_NEOX = 2
ODIT_NORM_NONE, ODIT_NORM_HEAD, ODIT_NORM_ROW = 0, 1, 2
ODIT_EPI_NONE, ODIT_EPI_BIAS, ODIT_EPI_GELU_TANH, ODIT_EPI_BIAS_GELU_TANH, ODIT_EPI_GATED_RESIDUAL = 0, 1, 2, 3, 4
ODIT_EPI_GATED_RESIDUAL_PRE = 5
ODIT_LINEAR_LIBRARY, ODIT_LINEAR_HANDWRITTEN = 1, 2

# every symbol include/omni_dit.h declares: (name, restype, argtypes)
_i64p = C.POINTER(C.c_int64)
_intp = C.POINTER(C.c_int)
_vpp = C.POINTER(C.c_void_p)
_SIGNATURES = {
    "odit_version": (C.c_int, []),
    "odit_last_error": (C.c_char_p, []),
    "odit_attn_fwd": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
         _i64p, _i64p, _i64p, _i64p, C.c_float, C.c_int, C.c_void_p],
    ),
    "odit_attn_fwd_ex": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
         C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
         _i64p, _i64p, _i64p, _i64p, _i64p, _i64p, C.c_float, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "odit_attn_fwd_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "odit_attn_fwd_plan": (
        C.c_int,
        [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_char_p, C.c_size_t],
    ),
    "odit_qknorm_rope": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i64p, C.c_int, C.c_int, C.c_float,
         C.c_int, C.c_int, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_qknorm_rope_pair": (
        C.c_int,
        [_vpp, _vpp, _vpp, C.c_void_p, C.c_void_p, C.c_void_p, _vpp, _vpp, _vpp, _vpp,
         C.c_int, _intp, C.c_int, C.c_int, C.c_int, _i64p, _intp, C.c_int, C.c_float,
         C.c_int, C.c_int, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_adaln_modulate_pair": (
        C.c_int,
        [_vpp, _vpp, _vpp, _vpp, C.c_int, _intp, C.c_int, _i64p, _i64p, _i64p, C.c_float, C.c_int, C.c_int,
         C.c_uint, C.c_void_p],
    ),
    "odit_adaln_modulate": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, _i64p, _i64p, C.c_int64, C.c_int64,
         C.c_float, C.c_int, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_gated_residual": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         _i64p, _i64p, _i64p, _i64p, C.c_int, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_rel_l1_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int64]),
    "odit_rel_l1": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int64,
         C.c_int64, C.c_int64, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_rel_l1_static": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_uint, C.c_void_p],
    ),
    "odit_rel_l1_static_scratch": (C.c_void_p, [C.POINTER(C.c_size_t)]),
    "odit_linear_workspace_bytes": (C.c_size_t, []),
    "odit_linear": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "odit_linear_rows": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_uint,
         C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "odit_linear_rows_plan": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_uint,
         C.c_void_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int)],
    ),
    "odit_linear_rows_tune": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_void_p,
         C.c_size_t, C.c_void_p, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_float), C.POINTER(C.c_int)],
    ),
    "odit_linear_tune": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p,
         C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_float)],
    ),
    "odit_gelu_tanh": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p]),
    "odit_silu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


class OmniDitLibraryError(RuntimeError):
    """The HIP kernel library is missing or cannot be loaded."""


class OmniDitKernelError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""


_lib: C.CDLL | None = None


def load() -> C.CDLL:
    """Load the shared library once and attach prototypes; raise loudly when it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise OmniDitLibraryError(
            f"{LIB_PATH} not found: build it with `python {LIB_PATH.parent / 'csrc' / 'build.py'}` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no fallback path."
        )
    try:
        lib = C.CDLL(os.fspath(LIB_PATH))
    except OSError as e:  # unresolved HIP runtime, wrong arch, ...
        raise OmniDitLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (restype, argtypes) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise OmniDitLibraryError(f"{LIB_PATH} does not export {name}") from e
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def is_available() -> bool:
    try:
        load()
        return True
    except OmniDitLibraryError:
        return False


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().odit_last_error().decode("utf-8", "replace")
        raise OmniDitKernelError(f"{what} failed with status {status}: {msg}")


def i64_array(values) -> C.Array:
    vals = [int(v) for v in values]
    return (C.c_int64 * len(vals))(*vals)


def int_array(values) -> C.Array:
    vals = [int(v) for v in values]
    return (C.c_int * len(vals))(*vals)


def ptr_array(values) -> C.Array:
    """Array of device addresses (None = null)."""
    return (C.c_void_p * len(values))(*[None if not v else int(v) for v in values])
