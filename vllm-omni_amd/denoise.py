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
        # a dense copy per branch: a stride-0 batch would take torch's broadcasting matmul in the stem
        out = transformer(hidden_states=latents.repeat(nb, 1, 1), encoder_hidden_states=text,
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


# ------------------------------------------------------------------- the reference's mixin interface
class FlowMatchEulerScheduler:
    """The part of diffusers' FlowMatchEulerDiscreteScheduler the loop uses (set_timesteps with explicit
    sigmas and ``mu``, ``timesteps``, ``set_begin_index``, ``step``): dynamic exponential time shift
    e^mu / (e^mu + 1/s - 1), timesteps = 1000 sigma, x <- x + (sigma_next - sigma) * v in float32."""

    def __init__(self, num_train_timesteps: int = 1000):
        self.num_train_timesteps = num_train_timesteps
        self.sigmas: np.ndarray | None = None
        self.timesteps: torch.Tensor | None = None
        self._step_index = 0

    def set_timesteps(self, num_inference_steps: int | None = None, device=None, sigmas=None, mu: float | None = None):
        if sigmas is None:
            sigmas = np.linspace(1.0, 1.0 / num_inference_steps, num_inference_steps)
        s = np.asarray(sigmas, dtype=np.float64)
        if mu is not None:
            e = math.exp(mu)
            s = e / (e + (1.0 / s - 1.0))
        self.sigmas = np.concatenate([s, [0.0]]).astype(np.float32)
        self.timesteps = torch.tensor(self.sigmas[:-1] * self.num_train_timesteps, device=device)
        self._step_index = 0

    def set_begin_index(self, begin_index: int = 0) -> None:
        self._step_index = begin_index

    def step(self, model_output: torch.Tensor, timestep, sample: torch.Tensor, return_dict: bool = True):
        i = self._step_index
        out = euler_step(sample, model_output, float(self.sigmas[i]), float(self.sigmas[i + 1]))
        self._step_index = i + 1
        return (out,) if not return_dict else {"prev_sample": out}


def _pad_rows(t: torch.Tensor, n: int) -> torch.Tensor:
    if t.shape[1] == n:
        return t
    pad = torch.zeros((t.shape[0], n - t.shape[1], *t.shape[2:]), dtype=t.dtype, device=t.device)
    return torch.cat([t, pad], dim=1)


def batch_cfg_kwargs(positive: dict, negative: dict) -> dict | None:
    """One set of transformer arguments for both branches, stacked on the batch axis (positive rows first),
    or None when they cannot be stacked. Prompts of different lengths are padded to the longer one and masked
    out as keys (``encoder_hidden_states_mask``); arguments that are equal in both branches are passed once."""
    if positive.keys() != negative.keys():
        return None
    out = {}
    for k, p in positive.items():
        n = negative[k]
        if k in ("encoder_hidden_states", "encoder_hidden_states_mask", "txt_seq_lens"):
            continue
        if torch.is_tensor(p) and torch.is_tensor(n):
            if p.shape != n.shape or p.dtype != n.dtype:
                return None
            out[k] = torch.cat([p, n], dim=0)
        elif p is None and n is None:
            out[k] = None
        elif k == "img_shapes" and isinstance(p, list) and isinstance(n, list):
            if p != n:
                return None
            out[k] = p + n if p and isinstance(p[0], list) else p   # per-sample lists grow with the batch
        elif torch.is_tensor(p) or torch.is_tensor(n) or p != n:
            return None
        else:
            out[k] = p
    if "encoder_hidden_states" in positive:
        pe, ne = positive["encoder_hidden_states"], negative["encoder_hidden_states"]
        if pe.shape[0] != ne.shape[0] or pe.shape[2:] != ne.shape[2:] or pe.dtype != ne.dtype:
            return None
        length = max(pe.shape[1], ne.shape[1])
        out["encoder_hidden_states"] = torch.cat([_pad_rows(pe, length), _pad_rows(ne, length)], dim=0)
        pm, nm = positive.get("encoder_hidden_states_mask"), negative.get("encoder_hidden_states_mask")
        if pm is None and nm is None and pe.shape[1] == ne.shape[1]:
            out["encoder_hidden_states_mask"] = None
        else:
            def mask_of(m, e):
                m = torch.ones(e.shape[:2], dtype=torch.bool, device=e.device) if m is None else m.bool()
                return _pad_rows(m, length)   # padding rows are False
            out["encoder_hidden_states_mask"] = torch.cat([mask_of(pm, pe), mask_of(nm, ne)], dim=0)
        if "txt_seq_lens" in positive:
            out["txt_seq_lens"] = [length] * out["encoder_hidden_states"].shape[0]
    return out


class CFGParallelMixin:
    """Method-for-method the reference's mixin (vllm_omni/diffusion/distributed/cfg_parallel.py:28-230) for a
    pipeline object with ``self.transformer`` and ``self.scheduler``, on one GPU. Where the reference runs the
    positive and the negative branch as two calls (or on two ranks), ``predict_noise_maybe_with_cfg`` stacks
    them on the batch axis and calls the transformer once whenever the two argument sets allow it;
    ``batch_cfg_branches = False`` keeps the reference's two sequential calls."""

    batch_cfg_branches = True

    def predict_noise_maybe_with_cfg(self, do_true_cfg: bool, true_cfg_scale: float, positive_kwargs: dict,
                                     negative_kwargs: dict | None, cfg_normalize: bool = True,
                                     output_slice: int | None = None) -> torch.Tensor:
        if not do_true_cfg:
            pred = self.predict_noise(**positive_kwargs)
            return pred if output_slice is None else pred[:, :output_slice]
        both = batch_cfg_kwargs(positive_kwargs, negative_kwargs) if self.batch_cfg_branches else None
        transformer = getattr(self, "transformer", None)
        if both is not None:
            if transformer is not None:
                transformer.cfg_batched_branches = ("positive", "negative")   # TeaCache keeps one state per branch
            pos, neg = self.predict_noise(**both).chunk(2, dim=0)
        else:
            if transformer is not None:
                transformer.cfg_batched_branches = None
            pos = self.predict_noise(**positive_kwargs)
            neg = self.predict_noise(**negative_kwargs)
        if output_slice is not None:
            pos, neg = pos[:, :output_slice], neg[:, :output_slice]
        return self.combine_cfg_noise(pos, neg, true_cfg_scale, cfg_normalize)

    def cfg_normalize_function(self, noise_pred: torch.Tensor, comb_pred: torch.Tensor) -> torch.Tensor:
        cond_norm = torch.norm(noise_pred, dim=-1, keepdim=True)
        noise_norm = torch.norm(comb_pred, dim=-1, keepdim=True)
        return comb_pred * (cond_norm / noise_norm)

    def combine_cfg_noise(self, noise_pred: torch.Tensor, neg_noise_pred: torch.Tensor, true_cfg_scale: float,
                          cfg_normalize: bool = False) -> torch.Tensor:
        comb_pred = neg_noise_pred + true_cfg_scale * (noise_pred - neg_noise_pred)
        return self.cfg_normalize_function(noise_pred, comb_pred) if cfg_normalize else comb_pred

    def predict_noise(self, *args, **kwargs) -> torch.Tensor:
        return self.transformer(*args, **kwargs)[0]

    def diffuse(self, *args, **kwargs):
        raise NotImplementedError("Subclasses must implement diffuse")

    def scheduler_step(self, noise_pred: torch.Tensor, t: torch.Tensor, latents: torch.Tensor) -> torch.Tensor:
        return self.scheduler.step(noise_pred, t, latents, return_dict=False)[0]

    def scheduler_step_maybe_with_cfg(self, noise_pred: torch.Tensor, t: torch.Tensor, latents: torch.Tensor,
                                      do_true_cfg: bool) -> torch.Tensor:
        return self.scheduler_step(noise_pred, t, latents)


class QwenImageCFGParallelMixin(CFGParallelMixin):
    """The Qwen-Image step loop with the reference's signature
    (vllm_omni/diffusion/models/qwen_image/cfg_parallel.py:27-125)."""

    interrupt = False

    def diffuse(self, prompt_embeds: torch.Tensor, prompt_embeds_mask: torch.Tensor | None,
                negative_prompt_embeds: torch.Tensor | None, negative_prompt_embeds_mask: torch.Tensor | None,
                latents: torch.Tensor, img_shapes, txt_seq_lens, negative_txt_seq_lens, timesteps: torch.Tensor,
                do_true_cfg: bool, guidance: torch.Tensor | None, true_cfg_scale: float,
                image_latents: torch.Tensor | None = None, cfg_normalize: bool = True,
                additional_transformer_kwargs: dict | None = None) -> torch.Tensor:
        self.scheduler.set_begin_index(0)
        self.transformer.do_true_cfg = do_true_cfg
        extra = additional_transformer_kwargs or {}
        for t in timesteps:
            if self.interrupt:
                continue
            self._current_timestep = t
            timestep = t.expand(latents.shape[0]).to(device=latents.device, dtype=latents.dtype)
            model_input = latents if image_latents is None else torch.cat([latents, image_latents], dim=1)

            def branch(embeds, mask, lens):
                return {"hidden_states": model_input, "timestep": timestep / 1000, "guidance": guidance,
                        "encoder_hidden_states_mask": mask, "encoder_hidden_states": embeds,
                        "img_shapes": img_shapes, "txt_seq_lens": lens, **extra}

            positive = branch(prompt_embeds, prompt_embeds_mask, txt_seq_lens)
            negative = branch(negative_prompt_embeds, negative_prompt_embeds_mask, negative_txt_seq_lens) if do_true_cfg else None
            output_slice = latents.size(1) if image_latents is not None else None
            noise_pred = self.predict_noise_maybe_with_cfg(do_true_cfg, true_cfg_scale, positive, negative,
                                                           cfg_normalize, output_slice)
            latents = self.scheduler_step_maybe_with_cfg(noise_pred, t, latents, do_true_cfg)
        return latents
