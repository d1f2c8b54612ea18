"""CFG-batched flow-matching Euler denoise loop around a DiT transformer.

Host-side counterpart of the reference's step loop
(vllm_omni/diffusion/models/qwen_image/cfg_parallel.py:72-123), its sequential CFG branch
(vllm_omni/diffusion/distributed/cfg_parallel.py:78-91), CFG combine (:99-137) and scheduler step
(:185-197), with one change of schedule: the positive and negative prompts are stacked on the batch
axis and go through the transformer in ONE call per step (B = 2) instead of two B = 1 calls.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch


def calculate_shift(image_seq_len: int, base_seq_len: int = 256, max_seq_len: int = 4096,
                    base_shift: float = 0.5, max_shift: float = 1.15) -> float:
    """Linear map sequence length -> mu (pipeline_qwen_image.py:69-79)."""
    slope = (max_shift - base_shift) / (max_seq_len - base_seq_len)
    return image_seq_len * slope + (base_shift - slope * base_seq_len)


def flow_match_sigmas(num_inference_steps: int, image_seq_len: int) -> np.ndarray:
    """N+1 sigmas: linspace(1, 1/N, N) time-shifted by e^mu / (e^mu + 1/s - 1), then a terminal 0
    (pipeline_qwen_image.py:501-517 and the flow-match Euler scheduler's dynamic shifting)."""
    s = np.linspace(1.0, 1.0 / num_inference_steps, num_inference_steps)
    e = math.exp(calculate_shift(image_seq_len))
    return np.concatenate([e / (e + (1.0 / s - 1.0)), [0.0]]).astype(np.float32)


def combine_cfg_noise(noise_pred: torch.Tensor, neg_noise_pred: torch.Tensor, true_cfg_scale: float,
                      cfg_normalize: bool = False) -> torch.Tensor:
    """neg + s (pos - neg); with cfg_normalize, rescaled per token to the positive prediction's norm."""
    comb = neg_noise_pred + true_cfg_scale * (noise_pred - neg_noise_pred)
    if not cfg_normalize:
        return comb
    return comb * (torch.norm(noise_pred, dim=-1, keepdim=True) / torch.norm(comb, dim=-1, keepdim=True))


def euler_step(latents: torch.Tensor, noise_pred: torch.Tensor, sigma: float, sigma_next: float) -> torch.Tensor:
    return (latents.float() + (sigma_next - sigma) * noise_pred.float()).to(latents.dtype)


@dataclass
class DenoiseInputs:
    latents: torch.Tensor                 # [1, S_img, in_channels] packed latents
    prompt_embeds: torch.Tensor           # [1, S_txt, J]
    negative_prompt_embeds: torch.Tensor | None  # [1, S_txt, J]; None disables CFG
    img_shape: tuple[int, int, int]       # (frames, patch rows, patch cols)
    prompt_mask: torch.Tensor | None = None
    negative_prompt_mask: torch.Tensor | None = None


def diffuse(transformer, inp: DenoiseInputs, num_inference_steps: int, true_cfg_scale: float = 4.0,
            cfg_normalize: bool = True, on_step=None) -> torch.Tensor:
    """Run the denoise loop; returns the final latents [1, S_img, in_channels]."""
    do_cfg = inp.negative_prompt_embeds is not None
    transformer.do_true_cfg = do_cfg
    transformer.cfg_batched_branches = ("positive", "negative") if do_cfg else None
    latents = inp.latents
    sig = flow_match_sigmas(num_inference_steps, latents.shape[1])
    if do_cfg:
        text = torch.cat([inp.prompt_embeds, inp.negative_prompt_embeds], dim=0)
        mask = None
        if inp.prompt_mask is not None or inp.negative_prompt_mask is not None:
            ones = torch.ones(text.shape[1], dtype=torch.bool, device=text.device)[None]
            mask = torch.cat([inp.prompt_mask if inp.prompt_mask is not None else ones,
                              inp.negative_prompt_mask if inp.negative_prompt_mask is not None else ones], dim=0)
    else:
        text, mask = inp.prompt_embeds, inp.prompt_mask
    nb = text.shape[0]
    txt_lens = [text.shape[1]] * nb
    for i in range(num_inference_steps):
        # the reference feeds timestep = (1000 sigma) / 1000 in the latent dtype
        t = (torch.full((nb,), float(sig[i]) * 1000.0, device=latents.device, dtype=latents.dtype) / 1000)
        out = transformer(hidden_states=latents.expand(nb, -1, -1), encoder_hidden_states=text,
                          encoder_hidden_states_mask=mask, timestep=t, img_shapes=[inp.img_shape],
                          txt_seq_lens=txt_lens, return_dict=False)[0]
        noise = combine_cfg_noise(out[0:1], out[1:2], true_cfg_scale, cfg_normalize) if do_cfg else out
        latents = euler_step(latents, noise, float(sig[i]), float(sig[i + 1]))
        if on_step is not None:
            on_step(i, latents)
    return latents


def diffuse_flux(transformer, latents: torch.Tensor, prompt_embeds: torch.Tensor, pooled_prompt_embeds: torch.Tensor,
                 img_ids: torch.Tensor, txt_ids: torch.Tensor, num_inference_steps: int,
                 guidance_scale: float | None = 3.5, on_step=None) -> torch.Tensor:
    """Guidance-distilled Flux loop: one transformer call per step, no CFG pair
    (vllm_omni/diffusion/models/flux/pipeline_flux.py denoising loop: timestep / 1000, embedded
    guidance scale, flow-match Euler step)."""
    transformer.do_true_cfg = False
    transformer.cfg_batched_branches = None
    nb = latents.shape[0]
    sig = flow_match_sigmas(num_inference_steps, latents.shape[1])
    guidance = None
    if guidance_scale is not None and getattr(transformer, "guidance_embeds", True):
        guidance = torch.full((nb,), float(guidance_scale), device=latents.device, dtype=torch.float32)
    for i in range(num_inference_steps):
        t = (torch.full((nb,), float(sig[i]) * 1000.0, device=latents.device, dtype=latents.dtype) / 1000)
        noise = transformer(hidden_states=latents, encoder_hidden_states=prompt_embeds,
                            pooled_projections=pooled_prompt_embeds, timestep=t, img_ids=img_ids, txt_ids=txt_ids,
                            guidance=guidance, return_dict=False)[0]
        latents = euler_step(latents, noise, float(sig[i]), float(sig[i + 1]))
        if on_step is not None:
            on_step(i, latents)
    return latents
