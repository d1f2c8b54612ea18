"""TeaCacheHook: intercepts the transformer forward, decides per CFG branch whether the block stack
must run or the cached residual can be reused (vllm_omni/diffusion/cache/teacache/hook.py:30-272).

Two calling conventions are supported:
  * sequential CFG, as the reference runs it: the transformer is called twice per step with one
    branch each and branches alternate by call parity (hook.py:125-138);
  * CFG-batched: one call per step with the branches stacked on the batch axis
    (``module.cfg_batched_branches = ("positive", "negative")``). The relative-L1 reduction is done per
    batch row in one launch, each row drives its own branch state, and when the branches disagree only
    the rows that must compute are pushed through the blocks.
Either way there is exactly one blocking device-to-host copy per call (the [B,2] sums).
"""

from __future__ import annotations

from typing import Any

import numpy as np
import torch

from ... import kernels
from ...hooks.base import HookRegistry, ModelHook, StateManager
from .config import TeaCacheConfig
from .extractors import get_extractor
from .state import TeaCacheState


def rel_l1_from_sums(sum_diff: float, sum_prev: float, n: int, dtype: torch.dtype) -> float:
    """mean|cur-prev| / (mean|prev| + 1e-8) with torch's rounding points for tensors of `dtype`
    (each mean, the sum with 1e-8 and the quotient are rounded to `dtype`; hook.py:214-221)."""
    md = torch.tensor(sum_diff / n, dtype=torch.float64).to(torch.float32).to(dtype)
    mp = torch.tensor(sum_prev / n, dtype=torch.float64).to(torch.float32).to(dtype)
    return (md / (mp + 1e-8)).item()


class TeaCacheHook(ModelHook):
    _HOOK_NAME = "teacache"

    def __init__(self, config: TeaCacheConfig):
        super().__init__()
        self.config = config
        self.rescale_func = np.poly1d(config.coefficients)
        self.state_manager = StateManager(TeaCacheState)
        self.extractor_fn = None
        self._forward_cnt = 0
        self.decisions: list[dict] = []  # one record per (call, branch): rel, accumulated, compute

    def initialize_hook(self, module: torch.nn.Module) -> torch.nn.Module:
        self.extractor_fn = get_extractor(self.config.transformer_type)
        self.state_manager.set_context("teacache")
        return module

    # ------------------------------------------------------------------ decision
    def _decide(self, state: TeaCacheState, rel: float | None) -> bool:
        """hook.py:185-232 given the rel-L1 scalar (None = nothing to compare against)."""
        if state.cnt == 0:
            state.accumulated_rel_l1_distance = 0.0
            return True
        if rel is None:
            return True
        state.accumulated_rel_l1_distance += abs(float(self.rescale_func(rel)))
        if state.accumulated_rel_l1_distance < self.config.rel_l1_thresh:
            return False
        state.accumulated_rel_l1_distance = 0.0
        return True

    def _should_compute_full_transformer(self, state: TeaCacheState, modulated_inp: torch.Tensor) -> bool:
        rel = None
        if state.cnt > 0 and state.previous_modulated_input is not None:
            sums = kernels.rel_l1_sums(modulated_inp.reshape(1, -1), state.previous_modulated_input.reshape(1, -1))
            sd, sp = sums.cpu()[0].tolist()
            rel = rel_l1_from_sums(sd, sp, modulated_inp.numel(), modulated_inp.dtype)
        compute = self._decide(state, rel)
        self.decisions.append({"branch": self.state_manager.current_context, "rel": rel,
                               "acc": state.accumulated_rel_l1_distance, "compute": compute})
        return compute

    # ------------------------------------------------------------------ forward
    def new_forward(self, module: torch.nn.Module, *args: Any, **kwargs: Any) -> Any:
        ctx = self.extractor_fn(module, *args, **kwargs)
        branches = getattr(module, "cfg_batched_branches", None)
        if branches is not None and ctx.hidden_states.shape[0] == len(branches):
            return self._forward_batched(ctx, tuple(branches))
        return self._forward_single(module, ctx)

    def _forward_single(self, module, ctx):
        if getattr(module, "do_true_cfg", False):
            branch = "negative" if self._forward_cnt % 2 == 1 else "positive"
        else:
            branch = "positive"
        self.state_manager.set_context(f"teacache_{branch}")
        state = self.state_manager.get_state()
        if not self._should_compute_full_transformer(state, ctx.modulated_input) and state.previous_residual is not None:
            ctx.hidden_states = ctx.hidden_states + state.previous_residual
            if state.previous_residual_encoder is not None and ctx.encoder_hidden_states is not None:
                ctx.encoder_hidden_states = ctx.encoder_hidden_states + state.previous_residual_encoder
        else:
            h0, e0 = ctx.hidden_states, ctx.encoder_hidden_states  # blocks never write in place
            outs = ctx.run_transformer_blocks()
            ctx.hidden_states = outs[0]
            if len(outs) > 1 and e0 is not None:
                ctx.encoder_hidden_states = outs[1]
            state.previous_residual = (ctx.hidden_states - h0).detach()
            if e0 is not None:
                state.previous_residual_encoder = (ctx.encoder_hidden_states - e0).detach()
        state.previous_modulated_input = ctx.modulated_input.detach()
        state.cnt += 1
        self._forward_cnt += 1
        return ctx.postprocess(ctx.hidden_states)

    def _forward_batched(self, ctx, branches: tuple[str, ...]):
        nb = len(branches)
        states = []
        for br in branches:
            self.state_manager.set_context(f"teacache_{br}")
            states.append(self.state_manager.get_state())
        mod = ctx.modulated_input
        # one reduction launch + one D2H for all rows that have something to compare against
        have_prev = [st.cnt > 0 and st.previous_modulated_input is not None for st in states]
        rels: list[float | None] = [None] * nb
        if any(have_prev):
            prev = torch.cat([st.previous_modulated_input if ok else mod[i:i + 1]
                              for i, (st, ok) in enumerate(zip(states, have_prev))], dim=0)
            sums = kernels.rel_l1_sums(mod, prev).cpu().tolist()
            n_row = mod[0].numel()
            for i, ok in enumerate(have_prev):
                if ok:
                    rels[i] = rel_l1_from_sums(sums[i][0], sums[i][1], n_row, mod.dtype)
        compute = []
        for i, st in enumerate(states):
            c = self._decide(st, rels[i]) or st.previous_residual is None
            compute.append(c)
            self.decisions.append({"branch": f"teacache_{branches[i]}", "rel": rels[i],
                                   "acc": st.accumulated_rel_l1_distance, "compute": c})
        rows = [i for i, c in enumerate(compute) if c]
        hidden, enc = ctx.hidden_states, ctx.encoder_hidden_states
        out_h = [None] * nb
        if rows:
            if len(rows) == nb:
                outs = ctx.run_transformer_blocks()
            elif ctx.run_transformer_blocks_rows is not None:
                outs = ctx.run_transformer_blocks_rows(rows)
            else:  # extractor cannot subset: run everything, keep only the rows that asked for it
                full = ctx.run_transformer_blocks()
                outs = tuple(t[rows] for t in full)
            for j, i in enumerate(rows):
                h_i = outs[0][j:j + 1]
                states[i].previous_residual = (h_i - hidden[i:i + 1]).detach()
                if len(outs) > 1 and enc is not None:
                    states[i].previous_residual_encoder = (outs[1][j:j + 1] - enc[i:i + 1]).detach()
                out_h[i] = h_i
        for i in range(nb):
            if out_h[i] is None:
                out_h[i] = hidden[i:i + 1] + states[i].previous_residual
            states[i].previous_modulated_input = mod[i:i + 1].detach()
            states[i].cnt += 1
        self._forward_cnt += nb
        return ctx.postprocess(torch.cat(out_h, dim=0))

    def reset_state(self, module: torch.nn.Module) -> torch.nn.Module:
        self.state_manager.reset()
        self._forward_cnt = 0
        self.decisions = []
        return module


def apply_teacache_hook(module: torch.nn.Module, config: TeaCacheConfig) -> None:
    """Register a TeaCacheHook on ``module`` (hook.py:249-272)."""
    HookRegistry.get_or_create(module).register_hook(TeaCacheHook._HOOK_NAME, TeaCacheHook(config))
