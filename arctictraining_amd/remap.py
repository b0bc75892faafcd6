"""Original MoE block <-> ArcticMoE parameter layout, and the install / restore hooks.

Mirrors arctic_training/model/moe/utils.py:75-327 (`remap_orig_moe_mlp_params_to_arctic_moe`)
and :330-422 (`remap_arctic_moe_to_orig_moe_mlp_params`) for one GPU (ep_size == 1): every
`layer.mlp` that owns `experts` is replaced by an `ArcticMoE` whose parameters are filled from
the original block, and the original (emptied) block is stashed in `_hide` so that the model
can be restored for saving a checkpoint in the original format.

The weight re-layout itself -- transposing each expert's nn.Linear weights and interleaving
gate / up on the last dimension -- runs in the HIP kernels of csrc/remap.hip through the C ABI
(`amoe_remap_pack`, `amoe_remap_unpack`); there is no torch or CPU fallback for it.

Three storage formats of the original experts are understood:
  * a ModuleList of per-expert MLPs with `gate_proj`, `up_proj`, `down_proj` nn.Linear modules
    (what the reference reads, utils.py:232-254);
  * fused tensors `experts.gate_up_proj [E, 2I, H]` (gate rows, then up rows) and
    `experts.down_proj [E, H, I]` (the Qwen3-MoE experts of transformers >= 5);
  * the gpt-oss experts (the reference's non-list branch, utils.py:291-299): `gate_up_proj` holds
    gate and up INTERLEAVED, either as [E, 2I, H] (the reference transposes it) or already as
    [E, H, 2I]; `down_proj [E, H, I]`.  Which fused format a model uses is decided by its
    architecture (`fused_gate_up_interleaved` of the derived config).  The orientation of an
    interleaved `gate_up_proj` is taken from `fused_gate_up_transposed` of the model's config when it
    is set (True: stored [E, 2I, H] and transposed on install, as the reference does); without it
    the shape decides when it can (H != 2I), and a square tensor raises instead of being guessed.
"""
import copy
import re
from types import SimpleNamespace

import torch
import torch.nn.functional as F

from . import ops
from .moe import ArcticMoE


def detect_if_moe_model(model) -> bool:
    """utils.py:71-72."""
    return any(k for k in model.config.__dict__.keys() if re.search("experts", k))


def arctic_moe_config_from_hf(config, dtype, ep_size=1, enable_routing_replay=False) -> SimpleNamespace:
    """The ArcticMoE hyper-parameters the reference derives from a HF config (utils.py:107-171)."""
    if ep_size != 1:
        raise NotImplementedError("this build runs one GPU: ep_size must be 1")
    ns = SimpleNamespace(
        model_dim=config.hidden_size,
        input_dtype=dtype,
        top_k=config.num_experts_per_tok,
        normalize_topk_scores=getattr(config, "norm_topk_prob", False),
        loss_coeff=config.router_aux_loss_coef,
    )
    arch = (getattr(config, "architectures", None) or [""])[0] or ""
    if "GptOssForCausalLM" in arch:
        ns.act_fn = lambda x: x * torch.sigmoid(x * 1.702)
    elif config.hidden_act in ("relu", "gelu", "silu"):
        ns.act_fn = getattr(F, config.hidden_act)
    else:
        raise ValueError(f"Unsupported activation {config.hidden_act}")
    ns.intermediate_dim = getattr(config, "moe_intermediate_size", None) or config.intermediate_size
    if hasattr(config, "num_local_experts"):
        ns.num_experts = config.num_local_experts
    elif hasattr(config, "num_experts"):
        ns.num_experts = config.num_experts
    else:
        raise ValueError(
            "Can't find an entry for number of experts in model's config. The config object has the following keys:"
            f" {config.__dict__.keys()}"
        )
    ns.use_shared_expert = hasattr(config, "shared_expert_intermediate_size")
    ns.return_router_scores = arch in ("GptOssForCausalLM",)
    ns.fused_gate_up_interleaved = "GptOss" in arch  # layout of a fused experts.gate_up_proj tensor
    ns.fused_gate_up_transposed = getattr(config, "fused_gate_up_transposed", None)  # None: decided by the shape
    ns.use_triton = False
    ns.is_gated = True
    ns.use_custom_moe_kernel = False
    ns.enable_routing_replay = enable_routing_replay
    ns.ep_size, ns.ep_rank, ns.ep_group = 1, 0, None
    return ns


def _interleaved_is_transposed(cfg, shape, H: int, I2: int) -> bool:
    """Whether an interleaved fused gate_up_proj of `shape` is stored [E, 2I, H] (True: transposed on
    install, what the reference always does, utils.py:296) or already [E, H, 2I] (False)."""
    flag = getattr(cfg, "fused_gate_up_transposed", None)
    last = tuple(shape[-2:])
    if flag is not None:
        want = (I2, H) if flag else (H, I2)
        if last != want:
            raise ValueError(f"gate_up_proj of shape {tuple(shape)}: fused_gate_up_transposed={bool(flag)} means [E, {want[0]}, {want[1]}]")
        return bool(flag)
    if H == I2:
        raise ValueError(
            f"gate_up_proj of shape {tuple(shape)} is square (hidden == 2 * intermediate): set fused_gate_up_transposed "
            "in the model's config (True: stored [E, 2I, H], the layout the reference transposes; False: [E, H, 2I])"
        )
    if last == (I2, H):
        return True
    if last == (H, I2):
        return False
    raise ValueError(f"gate_up_proj of shape {tuple(shape)} is neither [E, {I2}, {H}] nor [E, {H}, {I2}]")


def _experts_is_a_list(experts) -> bool:
    return isinstance(experts, torch.nn.ModuleList)


def _stacked_linear_weights(experts, name: str, device) -> torch.Tensor:
    """[E, out, in] stack of the nn.Linear weights `name` of a ModuleList of experts."""
    return torch.stack([getattr(ex, name).weight.detach().to(device) for ex in experts]).contiguous()


@torch.no_grad()
def fill_arctic_moe_from_orig_mlp(arctic_moe: ArcticMoE, orig_mlp, device) -> None:
    """Copy the parameters of one original MoE block into an ArcticMoE (utils.py:206-300)."""
    experts = orig_mlp.experts
    arctic_moe.router_gate.copy_(orig_mlp.gate.weight.detach().to(device))
    if _experts_is_a_list(experts):
        gate = _stacked_linear_weights(experts, "gate_proj", device)  # [E, I, H]
        up = _stacked_linear_weights(experts, "up_proj", device)
        down = _stacked_linear_weights(experts, "down_proj", device)  # [E, H, I]
    else:
        fused = experts.gate_up_proj.detach().to(device)
        down = experts.down_proj.detach().to(device).contiguous()
        H, I2 = arctic_moe.model_dim, 2 * arctic_moe.intermediate_dim
        if getattr(arctic_moe._config, "fused_gate_up_interleaved", False):
            # gpt-oss: gate / up already interleaved; at most a batched transpose is needed
            if _interleaved_is_transposed(arctic_moe._config, fused.shape, H, I2):
                arctic_moe.expert_gate_up.copy_(ops.remap_pack(fused.contiguous()))
            else:
                arctic_moe.expert_gate_up.copy_(fused)
            arctic_moe.expert_down.copy_(ops.remap_pack(down))
            return
        if tuple(fused.shape[-2:]) != (I2, H):
            raise ValueError(
                f"fused gate_up_proj of shape {tuple(fused.shape)}: expected [E, {I2}, {H}] (gate rows, then up rows); "
                "a tensor that interleaves gate and up (gpt-oss) needs fused_gate_up_interleaved=True in the config"
            )
        inter = fused.shape[1] // 2
        gate, up = fused[:, :inter, :], fused[:, inter:, :]
    arctic_moe.expert_gate_up.copy_(ops.remap_pack(gate, up))
    arctic_moe.expert_down.copy_(ops.remap_pack(down))
    if arctic_moe._config.use_shared_expert:
        sh = orig_mlp.shared_expert
        g = sh.gate_proj.weight.detach().to(device)[None].contiguous()
        u = sh.up_proj.weight.detach().to(device)[None].contiguous()
        arctic_moe.shared_expert_gate_up.copy_(ops.remap_pack(g, u)[0])
        arctic_moe.shared_expert_down.copy_(ops.remap_pack(sh.down_proj.weight.detach().to(device)[None].contiguous())[0])
        arctic_moe.shared_expert_output_gate.copy_(orig_mlp.shared_expert_gate.weight.detach().to(device).t())


@torch.no_grad()
def fill_orig_mlp_from_arctic_moe(orig_mlp, arctic_moe: ArcticMoE) -> None:
    """The inverse copy (utils.py:357-413); `orig_mlp` must hold allocated parameters."""
    experts = orig_mlp.experts
    orig_mlp.gate.weight.copy_(arctic_moe.router_gate)
    gate_up = arctic_moe.expert_gate_up.detach().contiguous()
    down = ops.remap_unpack(arctic_moe.expert_down.detach().contiguous(), two=False)  # [E, H, I]
    if _experts_is_a_list(experts):
        gate, up = ops.remap_unpack(gate_up, two=True)
        for i, ex in enumerate(experts):
            ex.gate_proj.weight.copy_(gate[i])
            ex.up_proj.weight.copy_(up[i])
            ex.down_proj.weight.copy_(down[i])
    elif getattr(arctic_moe._config, "fused_gate_up_interleaved", False):
        fused = experts.gate_up_proj
        H, I2 = arctic_moe.model_dim, 2 * arctic_moe.intermediate_dim
        if _interleaved_is_transposed(arctic_moe._config, fused.shape, H, I2):
            fused.copy_(ops.remap_unpack(gate_up, two=False))
        else:
            fused.copy_(gate_up)
        experts.down_proj.copy_(down)
    else:
        fused = experts.gate_up_proj
        inter = fused.shape[1] // 2
        if fused.is_cuda and fused.is_contiguous() and fused.dtype == gate_up.dtype:
            ops.remap_unpack(gate_up, two=True, out0=fused.data[:, :inter, :], out1=fused.data[:, inter:, :])
        else:
            gate, up = ops.remap_unpack(gate_up, two=True)
            fused.copy_(torch.cat((gate, up), dim=1))
        experts.down_proj.copy_(down)
    if arctic_moe._config.use_shared_expert:
        sh = orig_mlp.shared_expert
        g, u = ops.remap_unpack(arctic_moe.shared_expert_gate_up.detach()[None].contiguous(), two=True)
        sh.gate_proj.weight.copy_(g[0])
        sh.up_proj.weight.copy_(u[0])
        sh.down_proj.weight.copy_(ops.remap_unpack(arctic_moe.shared_expert_down.detach()[None].contiguous(), two=False)[0])
        orig_mlp.shared_expert_gate.weight.copy_(arctic_moe.shared_expert_output_gate.t())


@torch.no_grad()
def remap_orig_moe_mlp_params_to_arctic_moe(
    model, ep_size=1, is_resume=False, enable_custom_moe_kernel=False, enable_routing_replay=False, device=None
):
    """Replace every MoE `layer.mlp` of `model` by an ArcticMoE with the same weights
    (utils.py:75-327).  `is_resume` skips the weight copy (a checkpoint fills them later);
    `enable_custom_moe_kernel` is accepted and ignored: the HIP kernels are the only path."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    cfg = arctic_moe_config_from_hf(model.config, model.dtype, ep_size, enable_routing_replay)
    meta = torch.device("meta")
    for layer_module in model.model.layers:
        if not hasattr(layer_module.mlp, "experts"):
            continue  # some models don't have moe in every layer
        with meta:
            arctic_moe = ArcticMoE(cfg)
        arctic_moe.to_empty(device=device)
        if not is_resume:
            fill_arctic_moe_from_orig_mlp(arctic_moe, layer_module.mlp, device)
        layer_module.mlp.to(meta)
        # a dict hides the original block from nn.Module's registration (utils.py:311-313)
        arctic_moe._hide = dict(orig_mlp=layer_module.mlp)
        layer_module.mlp = arctic_moe
    return model


@torch.no_grad()
def remap_arctic_moe_to_orig_moe_mlp_params(model):
    """Undo remap_orig_moe_mlp_params_to_arctic_moe: every ArcticMoE `layer.mlp` becomes the
    original block again, filled from the ArcticMoE's current weights (utils.py:330-422)."""
    for layer_module in model.model.layers:
        if not isinstance(layer_module.mlp, ArcticMoE):
            continue
        arctic_moe = layer_module.mlp
        device = arctic_moe.router_gate.device
        # leave the stashed original intact in case this is an interim save and not an exit
        orig_mlp = copy.deepcopy(arctic_moe._hide["orig_mlp"])
        orig_mlp.to_empty(device=device)
        fill_orig_mlp_from_arctic_moe(orig_mlp, arctic_moe)
        layer_module.mlp = orig_mlp
    return model
