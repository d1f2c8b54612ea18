"""Build libomni_dit_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage:  python vllm-omni_amd/csrc/build.py [--force] [--jobs N]

Every translation unit is compiled to an object under csrc/build/ and linked into
``<package>/libomni_dit_hip.so`` next to the Python sources, so the library travels with the tree.
"""

from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
PKG = CSRC.parent
LIB_NAME = "libomni_dit_hip.so"
LIB_PATH = PKG / LIB_NAME
# bench.py's calibration probe (a bare MFMA loop): a library of its own, not part of the product's C ABI
PROBE_LIB_PATH = PKG / "libomni_dit_probe.so"
OBJ_DIR = CSRC / "build"
HEADERS = [CSRC / "odit_common.h", CSRC / "attn_common.h", CSRC / "attn_tail.h", CSRC / "gemm_bf16.h",
           CSRC / "gemm_epilogue.h", PKG.parent / "include" / "omni_dit.h"]

# (source file, extra defines, object stem)
UNITS: list[tuple[str, list[str], str]] = [
    ("api.hip", [], "api"),
    ("adaln.hip", [], "adaln"),
    ("pointwise.hip", [], "pointwise"),
    ("rel_l1.hip", [], "rel_l1"),
    ("qknorm_rope.hip", ["-DODIT_QK_TU=0"], "qknorm_rope_bf16"),
    ("qknorm_rope.hip", ["-DODIT_QK_TU=1"], "qknorm_rope_f16"),
    ("qknorm_rope.hip", ["-DODIT_QK_TU=2"], "qknorm_rope_f32"),
    ("attn_fwd.hip", [], "attn_fwd"),
    ("attn_fwd_dma.hip", [], "attn_fwd_dma"),
    ("linear.hip", [], "linear"),
    ("gemm_bf16.hip", [], "gemm_bf16"),
    ("gemm_bf16_tile.hip", [], "gemm_bf16_tile"),
]
PROBE_UNITS: list[tuple[str, list[str], str]] = [("probe.hip", [], "probe")]

# the dense projections call hipBLASLt (its MFMA GEMM kernels); everything else is self-contained
LINK_LIBS = ["-L/opt/rocm/lib", "-lhipblaslt"]

# -packed-fp32-ops is switched off on purpose: v_pk_*_f32 forms are not trusted on this target.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _stale(obj: Path, deps: list[Path]) -> bool:
    if not obj.exists():
        return True
    t = obj.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that line is noise
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> Path:
    hipcc = _hipcc()
    OBJ_DIR.mkdir(exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    work = []
    objs: dict[Path, list[Path]] = {LIB_PATH: [], PROBE_LIB_PATH: []}
    for lib, units in ((LIB_PATH, UNITS), (PROBE_LIB_PATH, PROBE_UNITS)):
        for src, defines, stem in units:
            src_path = CSRC / src
            if not src_path.exists():
                raise RuntimeError(f"missing source {src_path}")
            obj = OBJ_DIR / f"{stem}.o"
            objs[lib].append(obj)
            if force or _stale(obj, [src_path, *HEADERS, Path(__file__)]):
                work.append([hipcc, *HIPCC_FLAGS, *defines, "-c", str(src_path), "-o", str(obj)])
    if verbose:
        print(f"[omni_dit build] compiling {len(work)}/{len(UNITS) + len(PROBE_UNITS)} units with {jobs} jobs", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(_run, work))
    for lib, link in ((LIB_PATH, LINK_LIBS), (PROBE_LIB_PATH, [])):
        if work or force or not lib.exists():
            tmp = lib.with_suffix(".so.tmp")
            _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs[lib]), *link])
            os.replace(tmp, lib)
        if verbose:
            print(f"[omni_dit build] {lib} ({lib.stat().st_size} bytes)", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=None)
    a = ap.parse_args()
    build(force=a.force, jobs=a.jobs)
