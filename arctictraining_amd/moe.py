"""MI355X-native ArcticMoE layer: the reference's module surface
(arctic_training/model/moe/moe.py:33-51 `MoEConfig`, :63-323 `ArcticMoE`) over hand-written
HIP kernels reached through the C ABI of libarctic_moe_hip.so.

Same constructor argument, parameter names / shapes / layouts (they are checkpoint keys,
arctic_training/model/moe/utils.py:563-566), forward signature and return type as the
reference, so the trainer's `layer.mlp = ArcticMoE(config)` (utils.py:320) works unchanged.
The whole routed-expert computation is one torch.autograd.Function whose forward and
backward call the kernels stage by stage with no host synchronisation.
"""
import time
from collections import defaultdict
from dataclasses import dataclass
from typing import Any, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops


@dataclass(kw_only=True)
class MoEConfig:
    """Field for field the reference's MoEConfig (moe.py:33-51)."""

    act_fn: object
    ep_group: Any = None
    ep_size: int = 1
    ep_rank: int = 0
    input_dtype: torch.dtype
    intermediate_dim: int
    is_gated: bool = True
    loss_coeff: float = 0.01
    model_dim: int
    normalize_topk_scores: bool
    num_experts: int
    return_router_scores: bool = False
    top_k: int
    use_triton: bool = True  # accepted for compatibility; the HIP kernels are always used
    use_shared_expert: bool = False
    use_custom_moe_kernel: bool = False  # accepted for compatibility
    enable_routing_replay: bool = False


def classify_activation(act_fn) -> int:
    """Map the callable the reference config carries (utils.py:118-127) to the kernel's
    activation code by evaluating it on a few points."""
    if isinstance(act_fn, int):
        return act_fn
    if isinstance(act_fn, str):
        return {"silu": ops.ACT_SILU, "gelu": ops.ACT_GELU, "relu": ops.ACT_RELU, "gpt_oss": ops.ACT_GPT_OSS}[act_fn]
    probe = torch.tensor([-2.0, -0.5, 0.3, 1.7], dtype=torch.float32, device="cpu")  # also under a meta-device context
    got = act_fn(probe)
    candidates = {
        ops.ACT_SILU: F.silu(probe),
        ops.ACT_GELU: F.gelu(probe),
        ops.ACT_RELU: F.relu(probe),
        ops.ACT_GPT_OSS: probe * torch.sigmoid(probe * 1.702),
    }
    for code, ref in candidates.items():
        if torch.allclose(got, ref, atol=1e-6):
            return code
    raise ValueError("unsupported activation: expected silu, gelu, relu or x*sigmoid(1.702x)")


class PhaseTimers:
    """The attributes of the reference's SynchronizedWallClockTimerSimple that its callers
    touch (arctic_training/model/moe/timers.py:44-72): start/stop/elapsed, `times`,
    `token_counts`, and the `wall_clock_breakdown` switch.  A no-op unless switched on."""

    def __init__(self, wall_clock_breakdown: bool = False):
        self.wall_clock_breakdown = wall_clock_breakdown
        self.times = defaultdict(float)
        self.token_counts = defaultdict(int)
        self._t0 = {}

    def start(self, name):
        if self.wall_clock_breakdown:
            torch.cuda.synchronize()
            self._t0[name] = time.perf_counter()

    def stop(self, name):
        if self.wall_clock_breakdown:
            torch.cuda.synchronize()
            self.times[name] = (time.perf_counter() - self._t0.pop(name, time.perf_counter())) * 1000.0
        else:
            self.times[name] = 0

    def elapsed(self, name):
        return self.times[name]


_SPLIT_OFFSETS = {}


def _router_weight_grad(d_logits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """dW_router [E,H] = d_logits^T [E,T] @ x [T,H] (autograd of moe.py:233).

    The product is skinny (E rows) and deep (T): the library GEMM leaves most of the chip idle on
    it.  For bf16 it is run as a split-K on the grouped weight-gradient kernel instead -- the
    tokens are cut into chunks that play the role of experts, C[s] = d_logits[chunk s]^T @
    x[chunk s] -- and the partial products are summed in float32."""
    T, E = d_logits.shape
    splits = 16
    if x.dtype != torch.bfloat16 or E % 8 or T % (splits * 32):
        return torch.matmul(d_logits.t(), x)
    key = (T, splits, x.device)
    offs = _SPLIT_OFFSETS.get(key)
    if offs is None:
        offs = torch.arange(0, T + 1, T // splits, dtype=torch.int32, device=x.device)
        _SPLIT_OFFSETS[key] = offs
    part = ops.grouped_gemm_wgrad(d_logits, x, offs, splits, tile_cfg=1)  # [splits, E, H], 128x128 tiles
    return part.sum(dim=0, dtype=torch.float32).to(x.dtype)


class _ExpertLayerFn(torch.autograd.Function):
    """router top-k -> permutation -> grouped gated FFN -> weighted combine, and the
    gradients of all of it (the autograd of moe.py:231-233, 340-411, 176-193, 450-461 plus
    the load-balance hook :393-406)."""

    @staticmethod
    def forward(ctx, x, router_gate, w_gate_up, w_down, replay, opts):
        T, H = x.shape
        E, K = opts["num_experts"], opts["top_k"]
        timers: PhaseTimers = opts["timers"]

        timers.start("router")
        logits = torch.matmul(x, router_gate.t())  # plain library GEMM, moe.py:233
        probs, topk_idx, scores = ops.router_topk_fwd(logits, K, opts["normalize"])
        assign = topk_idx if replay is None else replay.to(torch.int32).contiguous()
        counts, offsets, token_of, slot_of, row_of, scores_perm = ops.permute_plan(assign, E, scores)
        timers.stop("router")

        # The gather x[token_of] (moe.py:356) happens inside the GEMMs' A loads: the routed copy
        # of the activations is never written.  The score of a routed row multiplies the expert's intermediate activation (epilogue of
        # the gate_up GEMM) instead of its output: the down projection is linear, so
        # (s * inter) @ W_down == s * (inter @ W_down), and the combine becomes a plain sum.
        timers.start("groupGeMM")
        cfg = opts["tile_cfg"]
        gate_up, inter_s = ops.grouped_gemm_gateup_act_fwd(
            x, w_gate_up, offsets, opts["act"], a_row_map=token_of, n_rows=T * K, tile_cfg=cfg, row_scale=scores_perm
        )
        out_s = ops.grouped_gemm_nn(inter_s, w_down, offsets, tile_cfg=cfg)
        timers.stop("groupGeMM")

        timers.start("moe-combine")
        y = ops.combine_fwd(out_s, row_of, None)
        timers.stop("moe-combine")

        ctx.opts = opts
        ctx.save_for_backward(
            x, router_gate, w_gate_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, slot_of, scores_perm,
            gate_up, inter_s,
        )
        # scores in routed-row order, in the model dtype, as the reference returns them
        scores_out = scores_perm.to(x.dtype)
        ctx.mark_non_differentiable(scores_out)
        cap = opts.get("capture")
        if cap is not None:
            cap.update(logits=logits, probs=probs, topk_idx=topk_idx, scores=scores, counts=counts, offsets=offsets,
                       token_of=token_of, slot_of=slot_of, row_of=row_of)
        return y, scores_out

    @staticmethod
    def backward(ctx, dy, _ds_perm):
        (x, router_gate, w_gate_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, slot_of, scores_perm,
         gate_up, inter_s) = ctx.saved_tensors
        opts = ctx.opts
        E, K = opts["num_experts"], opts["top_k"]
        T = x.shape[0]
        R = T * K
        cfg = opts["tile_cfg"]
        dy = dy.contiguous()

        # d(out_s)[r] = dy[token_of[r]]: the rows of dy are gathered inside the GEMMs' loads
        d_inter_s = ops.grouped_gemm_nt(dy, w_down, offsets, a_row_map=token_of, n_rows=R, tile_cfg=cfg)
        d_w_down = None
        if ctx.needs_input_grad[3]:
            d_w_down = ops.grouped_gemm_wgrad(inter_s, dy, offsets, E, tile_cfg=cfg, b_row_map=token_of)
        # gated-activation backward, with the score multiply: also yields d_scores [T,K]
        d_gate_up, d_scores = ops.gated_act_bwd(
            gate_up, d_inter_s, opts["act"], row_scale=scores_perm, slot_of=slot_of, tk=(T, K)
        )
        d_w_gate_up = None
        if ctx.needs_input_grad[2]:
            d_w_gate_up = ops.grouped_gemm_wgrad(x, d_gate_up, offsets, E, tile_cfg=cfg, a_row_map=token_of)

        d_logits = ops.router_bwd(
            d_scores, probs, topk_idx, counts, x.dtype, opts["normalize"], opts["loss_coeff"] / T / opts["ep_size"]
        )
        d_router_gate = _router_weight_grad(d_logits, x) if ctx.needs_input_grad[1] else None
        dx = None
        if ctx.needs_input_grad[0]:
            d_xp = ops.grouped_gemm_nt(d_gate_up, w_gate_up, offsets, tile_cfg=cfg)
            dx_router = torch.matmul(d_logits, router_gate)
            dx = ops.gather_rows_bwd(d_xp, row_of, addend=dx_router)
        return dx, d_router_gate, d_w_gate_up, d_w_down, None, None


class ArcticMoE(nn.Module):
    """Mixture-of-experts layer with the reference's surface (moe.py:63-323).

    Args:
        config: MoEConfig (or any object with the same attributes; the reference passes a
                SimpleNamespace, utils.py:107-161)
    """

    def __init__(self, config):
        super().__init__()
        self._config = config
        self.act_fn = config.act_fn
        self.ep_group = getattr(config, "ep_group", None)
        self.ep_rank = getattr(config, "ep_rank", 0)
        self.ep_size = getattr(config, "ep_size", 1)
        self.input_dtype = config.input_dtype
        self.intermediate_dim = config.intermediate_dim
        self.model_dim = config.model_dim
        self.num_experts = config.num_experts
        self.top_k = config.top_k
        self.use_custom_kernel = getattr(config, "use_custom_moe_kernel", False)
        if self.ep_size != 1:
            raise NotImplementedError("this build runs the expert layer on one GPU (ep_size must be 1)")
        if not getattr(config, "is_gated", True):
            raise NotImplementedError("only gated expert FFNs are supported (is_gated=True)")
        self._act_code = classify_activation(config.act_fn)

        self.timers = PhaseTimers()
        self.wall_clock_breakdown = False
        self.gate_time = 0.0
        self.num_local_experts = self.num_experts // self.ep_size
        self.tile_cfg = 0  # 0 = library default tile shape; other values are for tuning
        self.capture = None  # set to a dict to receive the routing intermediates of each forward

        dt = self.input_dtype
        self.router_gate = nn.Parameter(torch.empty((self.num_experts, self.model_dim), dtype=dt))
        self.expert_gate_up = nn.Parameter(
            torch.empty((self.num_local_experts, self.model_dim, 2 * self.intermediate_dim), dtype=dt)
        )
        self.gate_scale = 1.0
        self.up_scale = 0.0
        self.expert_down = nn.Parameter(torch.empty((self.num_local_experts, self.intermediate_dim, self.model_dim), dtype=dt))
        if getattr(config, "use_shared_expert", False):
            self.shared_expert_gate_up = nn.Parameter(torch.empty((self.model_dim, 2 * self.intermediate_dim), dtype=dt))
            self.shared_expert_down = nn.Parameter(torch.empty((self.intermediate_dim, self.model_dim), dtype=dt))
            self.shared_expert_output_gate = nn.Parameter(torch.empty(self.model_dim, 1, dtype=dt))
        self.enable_routing_replay = getattr(config, "enable_routing_replay", False)

    def enable_wall_clock_breakdown(self):
        """activate the phase timers (moe.py:153-156)"""
        self.wall_clock_breakdown = True
        self.timers.wall_clock_breakdown = True

    def extra_repr(self):
        lines = [
            f"(router_gate): Parameter({tuple(self.router_gate.shape)})",
            f"(expert_gate_up): Parameter({tuple(self.expert_gate_up.shape)})",
            f"(expert_down): Parameter({tuple(self.expert_down.shape)})",
        ]
        if getattr(self._config, "use_shared_expert", False):
            lines += [
                f"(shared_expert_gate_up): Parameter({tuple(self.shared_expert_gate_up.shape)})",
                f"(shared_expert_down): Parameter({tuple(self.shared_expert_down.shape)})",
                f"(shared_expert_output_gate): Parameter({tuple(self.shared_expert_output_gate.shape)})",
            ]
        return "\n".join(lines)

    def forward(self, hidden_states, routing_replay_assignments: Optional[torch.Tensor] = None):
        if self.enable_routing_replay:
            assert (
                routing_replay_assignments is not None
            ), "Routing replay assignments must be provided when routing replay is enabled"
        self.timers.start("amoe e2e")
        orig_shape = hidden_states.shape
        x = hidden_states.reshape(-1, hidden_states.shape[-1]).contiguous()
        opts = dict(
            num_experts=self.num_experts,
            top_k=self.top_k,
            normalize=bool(self._config.normalize_topk_scores),
            loss_coeff=float(getattr(self._config, "loss_coeff", 0.01)),
            ep_size=self.ep_size,
            act=self._act_code,
            tile_cfg=self.tile_cfg,
            timers=self.timers,
            capture=self.capture,
        )
        replay = routing_replay_assignments if self.enable_routing_replay else None
        output, scores = _ExpertLayerFn.apply(
            x, self.router_gate, self.expert_gate_up, self.expert_down, replay, opts
        )
        if getattr(self._config, "use_shared_expert", False):
            # dense shared expert with a sigmoid output gate (moe.py:305-314): library GEMMs
            self.timers.start("shared-expert")
            s_inter = torch.matmul(x, self.shared_expert_gate_up)
            s_gate, s_up = s_inter[..., 0::2], s_inter[..., 1::2]
            s_inter = s_up * self.act_fn(s_gate)
            s_out = torch.matmul(s_inter, self.shared_expert_down)
            s_out_gate = torch.matmul(x, self.shared_expert_output_gate)
            output = output + s_out * torch.sigmoid(s_out_gate)
            self.timers.stop("shared-expert")
        output = output.reshape(orig_shape)
        self.timers.stop("amoe e2e")
        return (output, scores) if getattr(self._config, "return_router_scores", False) else output
