"""Trainer-side helpers around the ArcticMoE layer, with the reference's names and behaviour
(arctic_training/model/moe/utils.py:61-72, 425-543; moe.py:465-509).  Pure host logic: which
parameters are expert parameters, how an optimizer's parameter groups are split for them,
the per-rank expert checkpoint file name, and the per-phase timing report.  Nothing here
depends on DeepSpeed being importable; objects are duck-typed where the reference passes
DeepSpeed engines.
"""
import os
from collections import defaultdict
from typing import Any, Callable, Dict, List, Sequence, Set, Tuple, Union

import torch

from .moe import ArcticMoE
from .remap import detect_if_moe_model  # noqa: F401  (same module in the reference)

# router_gate and the shared-expert parameters are ordinary data-parallel parameters
EXPERT_PARAM_NAMES = ("expert_gate_up", "expert_down")


def amoe_install_deepspeed_timers(model, model_unwrapped) -> None:
    """Switch the phase timers of every ArcticMoE on when the engine profiles wall-clock time
    (utils.py:61-68).  `model` only needs a `wall_clock_breakdown()` method."""
    if not model.wall_clock_breakdown():
        return
    for module in model_unwrapped.modules():
        if isinstance(module, ArcticMoE):
            module.enable_wall_clock_breakdown()


def identify_expert_params(model, ep_size: int) -> List[Callable[[], int]]:
    """Tag the expert parameters of every ArcticMoE the way DeepSpeed's ZeRO-2 MoE support
    expects (`allreduce = False`, `group_name = "ep_size_<n>"`) and return their `data_ptr`
    bound methods, by which an optimizer's nameless parameter groups are later split
    (utils.py:425-464)."""
    group_name = f"ep_size_{ep_size}"
    found = []
    for module in model.modules():
        if not isinstance(module, ArcticMoE):
            continue
        for name, param in module.named_parameters():
            if name.split(":")[-1] in EXPERT_PARAM_NAMES:
                param.allreduce = False
                param.group_name = group_name
                found.append(param.data_ptr)
    print(f"Found {len(found)} MoE params")
    return found


def is_expert_param(param: torch.Tensor, expert_param_data_ptrs: Sequence) -> bool:
    """utils.py:467-474: membership of the bound `data_ptr` method plus the group tag."""
    return param.data_ptr in expert_param_data_ptrs and hasattr(param, "group_name")


def split_params_into_different_moe_groups_for_optimizer(
    param_groups: Union[Dict[str, Any], Tuple[Dict[str, Any], ...], List[Dict[str, Any]]],
    expert_param_data_ptrs: Sequence,
) -> List[Dict[str, Any]]:
    """Move the expert parameters out of each parameter group into a new group per
    (original group, expert-parallel group name), marked `moe=True`, appended after the
    original groups (utils.py:477-538).  The input groups are modified in place."""
    if isinstance(param_groups, tuple):
        param_groups = list(param_groups)
    elif isinstance(param_groups, dict):
        param_groups = [param_groups]
    elif not isinstance(param_groups, list):
        raise ValueError(f"Unknown param group type of {type(param_groups)}")

    ep_names: Set[str] = set()
    for group in param_groups:
        for param in group["params"]:
            if is_expert_param(param, expert_param_data_ptrs):
                ep_names.add(param.group_name)

    # one empty MoE group per (source group, ep group), hyper-parameters inherited from the source
    moe_groups: Dict[str, Dict[str, Dict[str, Any]]] = defaultdict(dict)
    for group in param_groups:
        for ep_name in ep_names:
            moe_groups[group["name"]][ep_name] = {**group, "name": ep_name, "moe": True, "params": []}

    for group in param_groups:
        kept = []
        for param in group["params"]:
            if is_expert_param(param, expert_param_data_ptrs):
                moe_groups[group["name"]][param.group_name]["params"].append(param)
            else:
                kept.append(param)
        group["params"] = kept

    for per_source in moe_groups.values():
        param_groups.extend(per_source.values())
    return param_groups


def get_expert_ckpt_name(save_dir, tag, ep_rank, moe_layer_id) -> str:
    """utils.py:541-543."""
    return os.path.join(save_dir, tag, f"ep_rank_{ep_rank}_moe_layer_{moe_layer_id}_model_states.pt")


def print_forward_breakdown(self, fwd_time=None, printer: Callable[[str], None] = print) -> None:
    """Report the per-phase times and token counts the ArcticMoE layers of `self` (any
    nn.Module) gathered, per layer and aggregated (moe.py:465-509; the reference patches it
    over deepspeed.runtime.engine's method of the same name)."""
    layers = [m for m in self.modules() if isinstance(m, ArcticMoE)]
    if not layers:
        return
    keys = list(layers[0].timers.times.keys())
    width = max((len(k) for k in keys), default=0) + 1
    total_time: Dict[str, float] = defaultdict(float)
    total_tokens: Dict[str, int] = defaultdict(int)
    for i, layer in enumerate(layers):
        for k, v in layer.timers.times.items():
            total_time[k] += v
            printer(f"layer={i} time  : {k:{width}}: {v:5.2f}ms")
        for k, v in layer.timers.token_counts.items():
            total_tokens[k] += v
            printer(f"layer={i} tokens: {k}: {v/1e3:6.2f}K")
        printer("")
    printer("all layers aggregate time (ms): " + " | ".join(f"{k}: {v:.2f}" for k, v in total_time.items()))
    printer("all layers aggregate token counts (K): " + " | ".join(f"{k}: {v/1e3:.2f}" for k, v in total_tokens.items()))
