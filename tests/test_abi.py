"""The C-ABI library loads and exports exactly what include/omni_dit.h declares; argument errors are
reported on the host before any launch (so these run without a GPU)."""

import ctypes as C
import os
import re

import pytest

from vllm_omni_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "omni_dit.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(odit_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_functions() == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared_functions():
        assert hasattr(lib, name), name
    assert lib.odit_version() == 200


def _strides(*v):
    return _lib.i64_array(v)


def test_argument_errors_are_caught_before_launch():
    lib = _lib.load()
    buf = C.create_string_buffer(4096)
    p = C.addressof(buf)
    p16 = (p + 15) & ~15
    s3 = _strides(1024, 128, 128)
    # unsupported head size
    rc = lib.odit_attn_fwd(p16, p16, p16, p16, None, None, 1, 4, 4, 1, 1, 48, s3, s3, s3, s3, 0.1, 0, None)
    assert rc == -2 and b"head size" in lib.odit_last_error()
    # fp32 attention is not offered (the reference routes fp32 to SDPA)
    rc = lib.odit_attn_fwd(p16, p16, p16, p16, None, None, 1, 4, 4, 1, 1, 64, s3, s3, s3, s3, 0.1, 2, None)
    assert rc == -2
    # misaligned pointer
    rc = lib.odit_attn_fwd(p16 + 2, p16, p16, p16, None, None, 1, 4, 4, 1, 1, 64, s3, s3, s3, s3, 0.1, 0, None)
    assert rc == -1 and b"aligned" in lib.odit_last_error()
    # heads not divisible by kv heads
    rc = lib.odit_attn_fwd(p16, p16, p16, p16, None, None, 1, 4, 4, 3, 2, 64, s3, s3, s3, s3, 0.1, 0, None)
    assert rc == -1
    # null pointers
    rc = lib.odit_adaln_modulate(None, p16, None, None, None, None, None, None, None, 1, 1, 8, _strides(8, 8),
                                 _strides(8, 8), 8, 0, 1e-6, 0, 0, 0, None)
    assert rc == -1
    # a row index and per-token modulation rows exclude each other
    rc = lib.odit_adaln_modulate(p16, p16, p16, p16, p16, None, None, None, None, 1, 1, 8, _strides(8, 8),
                                 _strides(8, 8), 8, 8, 1e-6, 0, 0, 0, None)
    assert rc == -1 and b"exclude" in lib.odit_last_error()
    # joint rows out of range
    rc = lib.odit_qknorm_rope(p16, None, None, p16, None, None, None, None, None, None, 1, 4, 1, 64, 0,
                              _strides(256, 64), 2, 4, 1e-6, 1, 0, 0, 0, None)
    assert rc == -1 and b"do not fit" in lib.odit_last_error()
    # workspace too small
    # a ticket word for each of the 65536 rows a call may have, 8 group words 1 KiB apart for each of the 7 rows that
    # can have more than 32 workgroups, then 32 workgroups per row of 2^20 elements
    assert lib.odit_rel_l1_workspace_bytes(2, 1 << 20) == 65536 * 8 + 7 * 8 * 1024 + 2 * 32 * 8
    rc = lib.odit_rel_l1(p16, p16, p16, p16, 8, 2, 1 << 20, 1 << 20, 1 << 20, 0, 0, None)
    assert rc == -4
    # empty problems succeed without touching the device
    assert lib.odit_gelu_tanh(None, None, 0, 0, None) == 0
    assert lib.odit_gated_residual(p16, p16, None, None, p16, 0, 4, 8, _strides(32, 8), _strides(32, 8), _strides(32, 8),
                                   None, 0, 0, 0, None) == 0


def test_wrappers_refuse_cpu_tensors():
    import torch

    from vllm_omni_amd import kernels

    x = torch.zeros(1, 4, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        kernels.adaln_modulate(x, None, None)
    with pytest.raises(RuntimeError, match="GPU"):
        kernels.gelu_tanh(x)


def test_product_code_never_reaches_the_oracle():
    """The oracle is test infrastructure: nothing in the package, and in bench.py / __graft_entry__.py only the
    CPU-baseline leg and smoke(), may import it (checked on the syntax trees, so comments do not count)."""
    import ast
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]

    def oracle_imports(path):
        found = []
        for node in ast.walk(ast.parse(path.read_text())):
            names = []
            if isinstance(node, ast.Import):
                names = [a.name for a in node.names]
            elif isinstance(node, ast.ImportFrom):
                names = [node.module or ""]
            found += [(node.lineno, n) for n in names if n == "oracle" or n.startswith("oracle.")]
        return found

    package = {p.resolve() for p in root.iterdir() if p.is_dir() and (p / "kernels.py").exists()}  # dir + its import alias
    assert len(package) == 1
    for path in package.pop().rglob("*.py"):
        assert oracle_imports(path) == [], path
    allowed = {"bench.py": "cpu_baseline", "__graft_entry__.py": "smoke"}
    for name, func in allowed.items():
        tree = ast.parse((root / name).read_text())
        inside = set()
        for node in ast.walk(tree):
            if isinstance(node, ast.FunctionDef) and node.name == func:
                inside = {n.lineno for n in ast.walk(node) if isinstance(n, (ast.Import, ast.ImportFrom))}
        for lineno, _ in oracle_imports(root / name):
            assert lineno in inside, f"{name}:{lineno} imports the oracle outside {func}()"


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libomni_dit_hip.so")
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(_lib.OmniDitLibraryError, match="no fallback"):
        _lib.load()
    from vllm_omni_amd import kernels

    with pytest.raises(_lib.OmniDitLibraryError):
        kernels.attn_workspace_bytes(1, 128, 128, 1, 128) if hasattr(kernels, "attn_workspace_bytes") else _lib.load()


def test_header_is_plain_c(tmp_path):
    """include/omni_dit.h is a C header: it compiles as C99 with pedantic warnings as errors, alone."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc on this machine")
    src = tmp_path / "h.c"
    src.write_text('#include "omni_dit.h"\nint main(void) { return ODIT_VERSION == 0; }\n')
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    proc = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I" + include, "-fsyntax-only", str(src)],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
