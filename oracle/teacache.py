"""Oracle restatement of TeaCache's skip/compute logic (test infrastructure only).

Reference: ``vllm_omni/diffusion/cache/teacache/hook.py`` (``hook.py`` below), ``config.py``, ``state.py``.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from . import ops

# cache/teacache/config.py:9-40
COEFFICIENTS = {
    "FluxTransformer2DModel": [4.98651651e02, -2.83781631e02, 5.58554382e01, -3.82021401e00, 2.64230861e-01],
    "QwenImageTransformer2DModel": [-4.50000000e02, 2.80000000e02, -4.50000000e01, 3.20000000e00, -2.00000000e-02],
}


@dataclass
class BranchState:
    """state.py:13-38."""

    cnt: int = 0
    acc: float = 0.0
    prev_mod: torch.Tensor | None = None
    prev_res: torch.Tensor | None = None
    prev_res_enc: torch.Tensor | None = None


def decide(state: BranchState, rel: float | None, coeffs, thresh: float) -> bool:
    """hook.py:185-232 with the rel-L1 scalar already computed (None when there is no previous
    input): first call computes; otherwise acc += |poly(rel)|; acc < thresh -> skip; else reset + compute."""
    if state.cnt == 0:
        state.acc = 0.0
        return True
    if rel is None:
        return True
    state.acc += abs(float(np.poly1d(coeffs)(rel)))
    if state.acc < thresh:
        return False
    state.acc = 0.0
    return True


@dataclass
class TeaCacheOracle:
    """Sequential-CFG TeaCache around caller-supplied closures, one call per (step, branch):
    hook.py:87-183. ``branch`` alternates positive/negative by call parity when do_true_cfg."""

    coeffs: list[float]
    thresh: float
    do_true_cfg: bool = True
    states: dict[str, BranchState] = field(default_factory=dict)
    forward_cnt: int = 0
    log: list[dict] = field(default_factory=list)

    def __call__(self, mod_inp, hidden, enc, run_blocks, postprocess):
        branch = "negative" if (self.do_true_cfg and self.forward_cnt % 2 == 1) else "positive"
        st = self.states.setdefault(branch, BranchState())
        rel = None
        if st.cnt > 0 and st.prev_mod is not None:
            rel = ops.rel_l1(mod_inp, st.prev_mod)
        compute = decide(st, rel, self.coeffs, self.thresh)
        self.log.append({"branch": branch, "rel": rel, "acc": st.acc, "compute": compute})
        if not compute and st.prev_res is not None:
            hidden = hidden + st.prev_res
            if st.prev_res_enc is not None and enc is not None:
                enc = enc + st.prev_res_enc
        else:
            h0 = hidden.clone()
            e0 = enc.clone() if enc is not None else None
            outs = run_blocks()
            hidden = outs[0]
            if len(outs) > 1 and enc is not None:
                enc = outs[1]
            st.prev_res = (hidden - h0).detach()
            if e0 is not None:
                st.prev_res_enc = (enc - e0).detach()
        st.prev_mod = mod_inp.detach()
        st.cnt += 1
        self.forward_cnt += 1
        return postprocess(hidden)
