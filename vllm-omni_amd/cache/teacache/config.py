"""TeaCache configuration and the per-model rescaling polynomials
(vllm_omni/diffusion/cache/teacache/config.py:9-84; values are the reference's)."""

from __future__ import annotations

from dataclasses import dataclass

# highest degree first, 5 coefficients per transformer class
_MODEL_COEFFICIENTS: dict[str, list[float]] = {
    "FluxTransformer2DModel": [4.98651651e02, -2.83781631e02, 5.58554382e01, -3.82021401e00, 2.64230861e-01],
    "QwenImageTransformer2DModel": [-4.50000000e02, 2.80000000e02, -4.50000000e01, 3.20000000e00, -2.00000000e-02],
    "Bagel": [1.33313129e06, -1.68644226e05, 7.95050740e03, -1.63747873e02, 1.26352397e00],
    "ZImageTransformer2DModel": [-4.50000000e02, 2.80000000e02, -4.50000000e01, 3.20000000e00, -2.00000000e-02],
}


@dataclass
class TeaCacheConfig:
    rel_l1_thresh: float = 0.2
    coefficients: list[float] | None = None
    transformer_type: str = "QwenImageTransformer2DModel"

    def __post_init__(self) -> None:
        if self.rel_l1_thresh <= 0:
            raise ValueError(f"rel_l1_thresh must be positive, got {self.rel_l1_thresh}")
        if self.coefficients is None:
            if self.transformer_type not in _MODEL_COEFFICIENTS:
                raise KeyError(f"Cannot find coefficients for {self.transformer_type}. "
                               f"Supported: {list(_MODEL_COEFFICIENTS.keys())}")
            self.coefficients = _MODEL_COEFFICIENTS[self.transformer_type]
        if len(self.coefficients) != 5:
            raise ValueError(f"coefficients must contain exactly 5 elements, got {len(self.coefficients)}")
