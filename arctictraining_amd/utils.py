"""Trainer-side helpers around the ArcticMoE layer, with the reference's names and behaviour
(arctic_training/model/moe/utils.py:61-72, 425-543; moe.py:465-509).  Pure host logic: which
parameters are expert parameters, how an optimizer's parameter groups are split for them,
the per-rank expert checkpoint file name, and the per-phase timing report.  Nothing here
depends on DeepSpeed being importable; objects are duck-typed where the reference passes
DeepSpeed engines.

The two checkpoint routines are written against the attributes of a DeepSpeed engine they
touch (utils.py:546-666), so any object offering those works; `monkey_patch_ds_moe` binds them,
and the timing report, onto DeepSpeed's engine class when DeepSpeed is importable.
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


class TorchFileCheckpointEngine:
    """What the checkpoint routines need of a DeepSpeed checkpoint engine: torch.save / torch.load
    of one file (the role of deepspeed.runtime.checkpoint_engine.TorchCheckpointEngine, the default
    of utils.py:646)."""

    def preserves_storage_sharing(self) -> bool:
        return True

    def save(self, state_dict, path: str) -> None:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        torch.save(state_dict, path)

    def load(self, path: str, map_location=None):
        return torch.load(path, map_location=map_location, weights_only=True)


def _detached_copies(obj):
    """torch.save writes a tensor's whole storage: views (and the parameters of a flat buffer) are
    cloned first so that each file holds only its own tensors (the job of DeepSpeed's
    clone_tensors_for_torch_save, utils.py:572-573)."""
    if isinstance(obj, torch.Tensor):
        return obj.detach().clone()
    if isinstance(obj, dict):
        return type(obj)((k, _detached_copies(v)) for k, v in obj.items())
    if isinstance(obj, (list, tuple)):
        return type(obj)(_detached_copies(v) for v in obj)
    return obj


def _saveable(engine, state):
    return _detached_copies(state) if engine.checkpoint_engine.preserves_storage_sharing() else state


def amoe_save_checkpoint(self, save_dir, tag, client_state=None, exclude_frozen_parameters=False):
    """Checkpoint of an engine whose model holds ArcticMoE layers (utils.py:546-630): one file per
    ArcticMoE layer and expert-parallel rank with that layer's whole state dict under its full
    module path, one optimizer file per expert-parallel rank, and -- from expert-parallel rank 0 --
    the engine's main file holding every parameter that is neither an expert's nor a router's.

    `self` is the engine: `module`, `optimizer`, `lr_scheduler`, `checkpoint_engine`,
    `_get_ckpt_name`, `_get_optimizer_ckpt_name`, `zero_optimization()`, `module_state_dict()` and
    the bookkeeping counters are read from it."""
    print(f"AMoE Checkpoint saving into {save_dir}/{tag}")
    save_path = self._get_ckpt_name(save_dir, tag)
    ep_rank = 0
    moe_layer_id = 0
    for n_module, module in self.module.named_modules():
        if not isinstance(module, ArcticMoE):
            continue
        ep_rank = module.ep_rank  # also names the optimizer file below
        moe_state_dict = {n_module + "." + n: p for n, p in module.state_dict().items()}
        self.checkpoint_engine.save(_saveable(self, moe_state_dict), get_expert_ckpt_name(save_dir, tag, ep_rank, moe_layer_id))
        moe_layer_id += 1
    self._curr_ckpt_path = os.path.join(save_dir, tag)

    # optimizer states differ between expert-parallel ranks
    optimizer_state = {
        "optimizer": self.optimizer.state_dict() if self.optimizer and not self.zero_optimization() else None
    }
    self.checkpoint_engine.save(_saveable(self, optimizer_state), self._get_optimizer_ckpt_name(save_dir, tag, ep_rank))

    if ep_rank != 0:
        return
    full_state_dict = self.module_state_dict(exclude_frozen_parameters=exclude_frozen_parameters)
    non_moe_state_dict = {k: v for k, v in full_state_dict.items() if not ("expert" in k or "router_gate" in k)}
    loader = getattr(self, "training_dataloader", None)
    curriculum = getattr(self, "curriculum_learning_enabled", lambda: False)()
    random_ltd = getattr(self, "random_ltd_enabled", lambda: False)()
    state = dict(
        module=non_moe_state_dict,
        lr_scheduler=self.lr_scheduler.state_dict() if self.lr_scheduler is not None else None,
        data_sampler=loader.data_sampler.state_dict() if (loader is not None and curriculum) else None,
        random_ltd=self.random_ltd_scheduler.state_dict() if random_ltd else None,
        sparse_tensor_module_names=getattr(self, "sparse_tensor_module_names", None),
        skipped_steps=self.skipped_steps,
        global_steps=self.global_steps,
        global_samples=self.global_samples,
        dp_world_size=self.dp_world_size,
        mp_world_size=self.mp_world_size,
        num_experts=self.num_experts,
    )
    state.update(client_state or {})
    self.checkpoint_engine.save(_saveable(self, state), save_path)


def amoe_load_state_dict(
    checkpoint_path, tag, state_dict, old_moe_load, model=None, mpu=None, num_experts=1, checkpoint_engine=None, device=None
):
    """Add the per-layer ArcticMoE files of this rank to `state_dict` (in place), which already
    holds the non-MoE parameters of the main file (utils.py:638-666).  `old_moe_load`, `mpu` and
    `num_experts` are part of DeepSpeed's signature and are not used."""
    if checkpoint_engine is None:
        checkpoint_engine = TorchFileCheckpointEngine()
    if device is None:
        device = torch.device(f"cuda:{int(os.getenv('LOCAL_RANK', 0))}")
    moe_layer_id = 0
    for _, module in model.named_modules():
        if isinstance(module, ArcticMoE):
            path = get_expert_ckpt_name(checkpoint_path, tag, module.ep_rank, moe_layer_id)
            state_dict.update(checkpoint_engine.load(path, map_location=device))
            moe_layer_id += 1


def monkey_patch_ds_moe() -> None:
    """Bind the timing report and the two checkpoint routines onto DeepSpeed's engine class
    (utils.py:47-58).  Needs DeepSpeed; everything else in this module does not."""
    try:
        from deepspeed.runtime.engine import DeepSpeedEngine
    except ImportError as e:
        raise ImportError("monkey_patch_ds_moe patches deepspeed.runtime.engine.DeepSpeedEngine: install DeepSpeed") from e
    DeepSpeedEngine.print_forward_breakdown = print_forward_breakdown
    DeepSpeedEngine._save_moe_checkpoint = amoe_save_checkpoint
    DeepSpeedEngine.load_moe_state_dict = staticmethod(amoe_load_state_dict)


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
