"""Checkpoint-name handling shared by the transformers of this package.

The reference fuses separately stored q/k/v projections into one ``to_qkv`` / ``add_kv_proj``
parameter while loading (vLLM's QKVParallelLinear ``weight_loader`` with shard ids "q", "k", "v":
models/qwen_image/qwen_image_transformer.py:1073-1113, models/flux/flux_transformer.py:588-628,
models/wan2_2/wan2_2_transformer.py:907-990) and renames a few diffusers keys. Here the fused
parameter is a plain ``nn.Linear`` weight whose rows are [q; k; v], so a shard is a row range.
"""

from __future__ import annotations

from collections.abc import Iterable

import torch
import torch.nn as nn

_SHARD_INDEX = {"q": 0, "k": 1, "v": 2}


def load_stacked_weights(module: nn.Module, weights: Iterable[tuple[str, torch.Tensor]],
                         stacked_params_mapping: list[tuple[str, str, str]],
                         substring_renames: tuple[tuple[str, str], ...] = (),
                         exact_renames: dict[str, str] | None = None,
                         skip_unknown: bool = False) -> set[str]:
    """Copy ``(name, tensor)`` pairs into ``module``'s parameters.

    stacked_params_mapping: (fused_param_fragment, stored_fragment, shard_id) triples; a stored name
      containing ``stored_fragment`` goes to rows [i*n, (i+1)*n) of the fused parameter, n = rows / 3.
    substring_renames: (old, new) applied to names the mapping above did not claim, only when the
      name as stored is not a parameter of ``module``.
    exact_renames: whole-name renames applied first.
    Returns the set of stored and resolved names that were loaded, like the reference's loaders.
    """
    params = dict(module.named_parameters())
    loaded: set[str] = set()
    with torch.no_grad():
        for name, tensor in weights:
            name = (exact_renames or {}).get(name, name)
            original = lookup = name
            for fused, stored, shard_id in stacked_params_mapping:
                if stored not in original:
                    continue
                lookup = original.replace(stored, fused)
                if lookup not in params:
                    raise KeyError(f"{original}: fused parameter {lookup} does not exist")
                p = params[lookup]
                n = p.shape[0] // 3
                if tensor.shape[0] != n or tuple(tensor.shape[1:]) != tuple(p.shape[1:]):
                    raise ValueError(f"{original}: shard of shape {tuple(tensor.shape)} does not fit a third of "
                                     f"{lookup} {tuple(p.shape)}")
                i = _SHARD_INDEX[shard_id]
                p[i * n:(i + 1) * n].copy_(tensor.to(device=p.device, dtype=p.dtype))
                break
            else:
                if lookup not in params:
                    for old, new in substring_renames:
                        if old in lookup:
                            lookup = lookup.replace(old, new)
                if lookup not in params:
                    if skip_unknown:
                        continue
                    raise KeyError(f"{original}: no parameter named {lookup}")
                p = params[lookup]
                if tuple(tensor.shape) != tuple(p.shape):
                    raise ValueError(f"{original}: shape {tuple(tensor.shape)} does not match {lookup} {tuple(p.shape)}")
                p.copy_(tensor.to(device=p.device, dtype=p.dtype))
            loaded.add(original)
            loaded.add(lookup)
    return loaded


QKV_JOINT_MAPPING = [
    (".to_qkv", ".to_q", "q"), (".to_qkv", ".to_k", "k"), (".to_qkv", ".to_v", "v"),
    (".add_kv_proj", ".add_q_proj", "q"), (".add_kv_proj", ".add_k_proj", "k"), (".add_kv_proj", ".add_v_proj", "v"),
]
