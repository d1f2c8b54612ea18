"""Oracle restatement of the denoise-loop harness around the transformer (test infrastructure only).

Reference: ``vllm_omni/diffusion/models/qwen_image/pipeline_qwen_image.py`` (shift schedule),
``vllm_omni/diffusion/distributed/cfg_parallel.py`` (CFG combine, scheduler step),
``vllm_omni/diffusion/models/qwen_image/cfg_parallel.py`` (loop). The Euler update itself is
diffusers' FlowMatchEulerDiscreteScheduler (third-party; parity unpinned at that boundary): with
dynamic shifting, sigma' = e^mu / (e^mu + (1/sigma - 1)), a terminal sigma of 0 appended,
timesteps = 1000 * sigma', and x <- x + (sigma_{i+1} - sigma_i) * model_output in fp32.
"""

from __future__ import annotations

import math

import numpy as np
import torch


def calculate_shift(image_seq_len: int, base_seq_len: int = 256, max_seq_len: int = 4096,
                    base_shift: float = 0.5, max_shift: float = 1.15) -> float:
    """pipeline_qwen_image.py:69-79."""
    m = (max_shift - base_shift) / (max_seq_len - base_seq_len)
    return image_seq_len * m + (base_shift - m * base_seq_len)


def shifted_sigmas(num_steps: int, image_seq_len: int) -> np.ndarray:
    """linspace(1, 1/N, N) -> exponential time shift with mu from the sequence length -> append 0.
    pipeline_qwen_image.py:501-517 + scheduler set_timesteps."""
    sig = np.linspace(1.0, 1.0 / num_steps, num_steps)
    mu = calculate_shift(image_seq_len)
    sig = math.exp(mu) / (math.exp(mu) + (1.0 / sig - 1.0))
    return np.concatenate([sig, [0.0]]).astype(np.float32)


def combine_cfg(pos: torch.Tensor, neg: torch.Tensor, scale: float, normalize: bool) -> torch.Tensor:
    """neg + s (pos - neg), optionally rescaled per token to pos's norm. distributed/cfg_parallel.py:99-137."""
    comb = neg + scale * (pos - neg)
    if not normalize:
        return comb
    cond_norm = torch.norm(pos, dim=-1, keepdim=True)
    noise_norm = torch.norm(comb, dim=-1, keepdim=True)
    return comb * (cond_norm / noise_norm)


def euler_step(latents: torch.Tensor, noise: torch.Tensor, sigma: float, sigma_next: float) -> torch.Tensor:
    """x + (sigma_next - sigma) * v, evaluated in fp32 and cast back."""
    return (latents.float() + (sigma_next - sigma) * noise.float()).to(latents.dtype)


def diffuse(predict, latents: torch.Tensor, pos_text: torch.Tensor, neg_text: torch.Tensor | None,
            num_steps: int, cfg_scale: float = 4.0, normalize: bool = True):
    """models/qwen_image/cfg_parallel.py:72-123 with sequential CFG (distributed/cfg_parallel.py:78-91):
    per step call predict(latents, text, timestep/1000) for the positive then the negative prompt."""
    sig = shifted_sigmas(num_steps, latents.shape[1])
    for i in range(num_steps):
        t = torch.full((latents.shape[0],), float(sig[i]) * 1000.0, dtype=latents.dtype) / 1000
        pos = predict(latents, pos_text, t)
        if neg_text is not None:
            neg = predict(latents, neg_text, t)
            noise = combine_cfg(pos, neg, cfg_scale, normalize)
        else:
            noise = pos
        latents = euler_step(latents, noise, float(sig[i]), float(sig[i + 1]))
    return latents
