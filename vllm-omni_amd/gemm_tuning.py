"""hipBLASLt solution selection for the dense projections of the DiT block.

The block's GEMMs are plain library GEMMs (torch.nn.functional.linear -> hipBLASLt). For a handful of
fixed shapes per model the library's default heuristic is measurably off its best solution, so the
shapes are tuned once with PyTorch's TunableOp (every candidate is checked numerically against the
default result) and the winning solution ids are kept in a small CSV next to this file.

    python -m vllm_omni_amd.gemm_tuning            # re-tune on the current GPU, rewrite the CSV
    gemm_tuning.enable()                           # at start-up: use the CSV, never tune

The CSV carries the library versions it was made with; TunableOp ignores it when they differ, which
silently falls back to the default heuristic.
"""

from __future__ import annotations

import os
from pathlib import Path

RESULTS = Path(__file__).resolve().parent / "tunableop_gfx950.csv"


def enable(path: os.PathLike | str = RESULTS) -> bool:
    """Use tuned GEMM solutions from `path` if it exists (tuning stays off). Returns whether enabled."""
    import torch
    import torch.cuda.tunable as tunable

    if not os.path.exists(path) or not torch.cuda.is_available():
        return False
    tunable.set_filename(os.fspath(path), insert_device_ordinal=False)
    tunable.tuning_enable(False)
    tunable.enable(True)
    tunable.read_file(os.fspath(path))
    return True


def tune(out: os.PathLike | str = RESULTS, max_seconds_per_gemm: int = 30) -> None:
    """Run one Qwen-Image-shape block (image M=8192, text M=512, modulation M=2) with tuning on."""
    import torch
    import torch.cuda.tunable as tunable

    from .blocks.qwen_image import QwenImageTransformer2DModel

    out = os.fspath(out)
    if os.path.exists(out):
        os.remove(out)
    tunable.set_filename(out, insert_device_ordinal=False)
    tunable.set_numerical_check_tolerances(True, 1e-2, 1e-2)
    tunable.set_max_tuning_duration(max_seconds_per_gemm * 1000)
    tunable.tuning_enable(True)
    tunable.enable(True)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("cuda"):
            model = QwenImageTransformer2DModel(num_layers=60 if os.environ.get("ODIT_TUNE_FULL") else 2)
    finally:
        torch.set_default_dtype(prev)
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.02)
    model.fuse_modulation()
    lat = torch.randn(2, 4096, 64, device="cuda", dtype=torch.bfloat16)
    txt = torch.randn(2, 256, 3584, device="cuda", dtype=torch.bfloat16)
    t = torch.full((2,), 0.5, device="cuda", dtype=torch.bfloat16)
    with torch.inference_mode():
        for _ in range(2):
            y = model(lat, txt, None, t, [(1, 64, 64)], [256, 256]).sample
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all()), "tuned GEMMs produced non-finite output"
    print(f"results go to {out} when the process exits (TunableOp writes its table at shutdown)")


if __name__ == "__main__":
    tune()
