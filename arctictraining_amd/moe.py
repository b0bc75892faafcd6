"""MI355X-native ArcticMoE layer: the reference's module surface
(arctic_training/model/moe/moe.py:33-51 `MoEConfig`, :63-323 `ArcticMoE`) over hand-written
HIP kernels reached through the C ABI of libarctic_moe_hip.so.

Same constructor argument, parameter names / shapes / layouts (they are checkpoint keys,
arctic_training/model/moe/utils.py:563-566), forward signature and return type as the
reference, so the trainer's `layer.mlp = ArcticMoE(config)` (utils.py:320) works unchanged.
The whole routed-expert computation is one torch.autograd.Function whose forward and
backward call the kernels stage by stage with no host synchronisation.
"""
import contextlib
import time
from collections import OrderedDict, defaultdict
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
    # accepted for compatibility and IGNORED: the reference's capacity-padded custom-kernel path (moe.py:140-149,
    # 413-448) differs from its default path by design (atomic row order, no load-balance gradient, scores
    # normalised inside the gather); this layer always computes the default path and warns once when the flag is set
    use_custom_moe_kernel: bool = False
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


class _SmallTensorCache:
    """A few small index tensors keyed by (size, kind, device), least recently used evicted first:
    the token count changes from step to step with packed variable-length batches, so the cache
    must not grow with the number of distinct sizes seen.  Nothing is stored while a HIP graph is
    being captured (a tensor created there lives in the graph's private pool and only holds its
    values after a replay)."""

    def __init__(self, max_entries: int = 8):
        self.max_entries = max_entries
        self._d = OrderedDict()

    def get(self, key, make):
        t = self._d.get(key)
        if t is not None:
            self._d.move_to_end(key)
            return t
        t = make()
        if not (t.is_cuda and torch.cuda.is_current_stream_capturing()):
            self._d[key] = t
            while len(self._d) > self.max_entries:
                self._d.popitem(last=False)
        return t

    def __len__(self):
        return len(self._d)


_INDEX_CACHE = _SmallTensorCache()


_side_streams: dict = {}


def _side_stream(device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority) for the expert weight gradients of the
    backward pass: they feed nothing else in the layer, and every grouped GEMM here is one
    workgroup per compute unit that ends with part of the chip idle -- launched from a second
    stream, the next kernel's workgroups start on the compute units as the previous kernel's leave."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    st = _side_streams.get(idx)
    if st is None:
        st = _side_streams[idx] = torch.cuda.Stream(device=idx)
    return st


def _token_offsets(T: int, parts: int, device) -> torch.Tensor:
    """int32 [parts + 1]: the T tokens cut into `parts` nearly equal consecutive chunks."""
    return _INDEX_CACHE.get(
        (T, parts, str(device)),
        lambda: (torch.arange(parts + 1, dtype=torch.int64, device=device) * T // parts).to(torch.int32),
    )


def _token_ids(T: int, device) -> torch.Tensor:
    return _INDEX_CACHE.get((T, "ids", str(device)), lambda: torch.arange(T, dtype=torch.int32, device=device))


def _dense_weight_grad(a: torch.Tensor, b: torch.Tensor, tile_cfg: int = 0, tile: int = 256) -> torch.Tensor:
    """C [Kd,N] = a^T [Kd,T] @ b [T,N]: the weight gradient of a dense (not routed) linear map.

    Few output tiles and a deep reduction over the tokens: run as a split-K on the grouped
    weight-gradient kernel -- the tokens are cut into chunks that play the role of experts,
    C[s] = a[chunk s]^T @ b[chunk s].  The kernel accumulates each partial product in float32 and
    stores it in the operands' 16-bit type; the (at most 16) partials are then added in float32
    and the sum is rounded once more."""
    T, Kd = a.shape
    N = b.shape[1]
    tiles = -(-Kd // tile) * -(-N // tile)
    splits = max(1, min(16, 512 // tiles, T // 256)) if a.dtype != torch.float32 else 1
    part = ops.grouped_gemm_wgrad(a, b, _token_offsets(T, splits, a.device), splits, tile_cfg=tile_cfg)
    if splits == 1:
        return part[0]
    return part.sum(dim=0, dtype=torch.float32).to(a.dtype)


def _router_weight_grad(d_logits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """dW_router [E,H] = d_logits^T [E,T] @ x [T,H] (autograd of moe.py:233): skinny (E rows) and
    deep (T), the library GEMM leaves most of the chip idle on it."""
    T, E = d_logits.shape
    if x.dtype == torch.float32 or E % 8 or T < 16 * 32:
        return torch.matmul(d_logits.t(), x)
    return _dense_weight_grad(d_logits, x, tile_cfg=1, tile=128)  # 128x128 tiles


def _route(x, router_gate, replay, opts):
    """Router linear map, softmax / top-k, and the permutation plan with the tile map of the
    row-grouped GEMMs (moe.py:231-233, 359-382).  Returns logits, probs, topk_idx, scores [T,K],
    the GEMM workspace that holds the tile map, and the plan (counts, offsets, token_of, slot_of,
    row_of, scores_perm)."""
    T = x.shape[0]
    E, K = opts["num_experts"], opts["top_k"]
    timers: PhaseTimers = opts["timers"]
    timers.start("router")
    logits = torch.matmul(x, router_gate.t())  # plain library GEMM, moe.py:233
    probs, topk_idx, scores = ops.router_topk_fwd(logits, K, opts["normalize"])
    assign = topk_idx
    if replay is not None:
        assign = replay.to(torch.int32).contiguous()
        if opts.get("check_replay", True) and not torch.cuda.is_current_stream_capturing():
            # The reference's one_hot(..., num_classes=E) raises on an expert id outside [0, E)
            # (moe.py:374).  The same error here, at the price of one host synchronisation per replayed
            # forward; `ArcticMoE.check_replay = False` (and a HIP graph capture, which cannot
            # synchronise) skips it, the permutation kernels then clamp such ids for memory safety.
            bad = ((assign < 0) | (assign >= E)).any()
            if bool(bad):
                raise RuntimeError(f"routing_replay_assignments holds expert ids outside [0, {E})")
    # the row-grouped GEMMs of a step share one tile map: the permutation plan builds it (its
    # scan kernel holds the offsets), the workspace is kept for backward
    ws = ops.gemm_workspace(T * K, E, x.device)
    plan = ops.permute_plan(assign, E, scores, gemm_workspace=ws, gemm_dtype=x.dtype, tile_cfg=opts["tile_cfg"])
    timers.stop("router")
    return logits, probs, topk_idx, scores, ws, plan


class _ExpertLayerFn(torch.autograd.Function):
    """router top-k -> permutation -> grouped gated FFN -> weighted combine, and the
    gradients of all of it (the autograd of moe.py:231-233, 340-411, 176-193, 450-461 plus
    the load-balance hook :393-406)."""

    @staticmethod
    def forward(ctx, x, router_gate, w_gate_up, w_down, sh_gate_up, sh_down, sh_out_gate, replay, opts):
        T, H = x.shape
        E, K = opts["num_experts"], opts["top_k"]
        timers: PhaseTimers = opts["timers"]
        cfg = opts["tile_cfg"]
        logits, probs, topk_idx, scores, ws, (counts, offsets, token_of, slot_of, row_of, scores_perm) = _route(
            x, router_gate, replay, opts
        )

        # The gather x[token_of] (moe.py:356) happens inside the GEMMs' A loads: the routed copy
        # of the activations is never written.  The score of a routed row multiplies the expert's intermediate activation (epilogue of
        # the gate_up GEMM) instead of its output: the down projection is linear, so
        # (s * inter) @ W_down == s * (inter @ W_down), and the combine becomes a plain sum.
        timers.start("groupGeMM")
        gate_up, inter_s = ops.grouped_gemm_gateup_act_fwd(
            x, w_gate_up, offsets, opts["act"], a_row_map=token_of, n_rows=T * K, tile_cfg=cfg, row_scale=scores_perm,
            workspace=ws, map_ready=True,
        )
        out_s = ops.grouped_gemm_nn(inter_s, w_down, offsets, tile_cfg=cfg, workspace=ws, map_ready=True)
        timers.stop("groupGeMM")

        # Shared expert (moe.py:305-314): a dense gated FFN over all T tokens, its output scaled per
        # token by sigmoid(x @ w_out_gate).  It runs through the same kernels as one more expert that
        # owns every token, the sigmoid in the role of the routing score; its output joins the
        # combine as the addend of the per-token sum.
        shared = sh_gate_up is not None
        sh_gu = sh_inter_s = sh_sig = sh_out = None
        if shared:
            timers.start("shared-expert")
            all_rows = _token_offsets(T, 1, x.device)
            sh_sig = torch.sigmoid(torch.matmul(x, sh_out_gate)).float().reshape(T)
            sh_gu, sh_inter_s = ops.grouped_gemm_gateup_act_fwd(
                x, sh_gate_up.unsqueeze(0), all_rows, opts["act"], tile_cfg=cfg, row_scale=sh_sig
            )
            sh_out = ops.grouped_gemm_nn(sh_inter_s, sh_down.unsqueeze(0), all_rows, tile_cfg=cfg)
            timers.stop("shared-expert")

        timers.start("moe-combine")
        # y[t] = sum_k out_s[row_of[t,k]] (+ the shared expert's row t)
        y = ops.gather_rows_bwd(out_s, row_of, addend=sh_out) if shared else ops.combine_fwd(out_s, row_of, None)
        timers.stop("moe-combine")

        ctx.opts = opts
        ctx.shared = shared
        ctx.gemm_ws = ws
        ctx.save_for_backward(
            x, router_gate, w_gate_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, slot_of, scores_perm,
            gate_up, inter_s, sh_gate_up, sh_down, sh_out_gate, sh_gu, sh_inter_s, sh_sig,
        )
        # scores in routed-row order, in the model dtype, as the reference returns them (moe.py:323,
        # only when return_router_scores); they stay attached to the graph like the reference's
        if opts["want_scores"]:
            scores_out = scores_perm.to(x.dtype)
        else:
            scores_out = scores_perm.new_empty(0)
            ctx.mark_non_differentiable(scores_out)
        ctx.set_materialize_grads(False)  # no zero-filled gradient for an output the loss does not use
        cap = opts.get("capture")
        if cap is not None:
            cap.update(logits=logits, probs=probs, topk_idx=topk_idx, scores=scores, counts=counts, offsets=offsets,
                       token_of=token_of, slot_of=slot_of, row_of=row_of)
        return y, scores_out

    @staticmethod
    def backward(ctx, dy, ds_perm):
        (x, router_gate, w_gate_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, slot_of, scores_perm,
         gate_up, inter_s, sh_gate_up, sh_down, sh_out_gate, sh_gu, sh_inter_s, sh_sig) = ctx.saved_tensors
        opts = ctx.opts
        E, K = opts["num_experts"], opts["top_k"]
        T = x.shape[0]
        R = T * K
        cfg = opts["tile_cfg"]
        if dy is None and ds_perm is None:  # neither output took part in the loss
            return (None,) * 9
        dy = torch.zeros_like(x) if dy is None else dy.contiguous()

        # The two expert weight gradients run on a second stream beside the chain of data gradients.
        # Fork: the side stream sees everything the main stream has queued so far (dy, the saved
        # tensors); join (below): the main stream waits for it before this function returns, so the
        # tensors either stream reads outlive the kernels that read them.
        main = side = None
        if x.is_cuda and opts.get("overlap_weight_grads", True):
            main, side = torch.cuda.current_stream(), _side_stream(x.device)
            side.wait_stream(main)

        def on_side(fn):
            if side is None:
                return fn()
            with torch.cuda.stream(side):
                out = fn()
            if not torch.cuda.is_current_stream_capturing():
                out.record_stream(main)   # allocated from the side stream's pool, consumed on the main stream
            return out

        # d(out_s)[r] = dy[token_of[r]]: the rows of dy are gathered inside the GEMMs' loads
        ws = ctx.gemm_ws  # still holds the forward's tile map
        fused = x.dtype != torch.float32 and cfg in (0, 1, 2)
        if fused:
            # data gradient of the down projection with the gated-activation backward as its
            # epilogue: d_inter is never written; the score gradients come back as per-N-tile row sums
            d_gate_up, parts = ops.grouped_gemm_nt_gated_bwd(
                dy, w_down, offsets, gate_up, opts["act"], row_scale=scores_perm, a_row_map=token_of, n_rows=R, tile_cfg=cfg,
                workspace=ws, map_ready=True,
            )
            if ds_perm is not None:  # gradient of the returned scores [R] (row order): one more partial
                parts = torch.cat((parts, ds_perm.float().reshape(1, R)))
                ds_perm = None
            d_scores = ops.score_grad_gather(parts, row_of)
        else:
            d_inter_s = ops.grouped_gemm_nt(dy, w_down, offsets, a_row_map=token_of, n_rows=R, tile_cfg=cfg, workspace=ws,
                                            map_ready=True)
            # gated-activation backward, with the score multiply: also yields d_scores [T,K]
            d_gate_up, d_scores = ops.gated_act_bwd(
                gate_up, d_inter_s, opts["act"], row_scale=scores_perm, slot_of=slot_of, tk=(T, K)
            )
        # (queued after the data gradient above, which it does not depend on: its workgroups take the
        # compute units as that kernel's last tiles finish)
        d_w_down = None
        if ctx.needs_input_grad[3]:
            d_w_down = on_side(lambda: ops.grouped_gemm_wgrad(inter_s, dy, offsets, E, tile_cfg=cfg, b_row_map=token_of))
        d_w_gate_up = None
        if ctx.needs_input_grad[2]:
            if side is not None:
                side.wait_stream(main)   # d_gate_up
            d_w_gate_up = on_side(lambda: ops.grouped_gemm_wgrad(x, d_gate_up, offsets, E, tile_cfg=cfg, a_row_map=token_of))
        if ds_perm is not None:
            # gradient of the returned scores [R] (row order), taken back to the slots [T,K]
            d_scores = d_scores + ds_perm.float()[row_of.long()]

        d_logits = ops.router_bwd(
            d_scores, probs, topk_idx, counts, x.dtype, opts["normalize"], opts["loss_coeff"] / T / opts["ep_size"]
        )
        d_router_gate = _router_weight_grad(d_logits, x) if ctx.needs_input_grad[1] else None
        cap = opts.get("capture")
        if cap is not None:
            cap.update(d_scores=d_scores, d_logits=d_logits)

        d_sh_gate_up = d_sh_down = d_sh_out_gate = d_sh_gu = d_pre = None
        if ctx.shared:
            # the same chain for the expert that owns every token; the "score" gradient comes
            # back per token and goes on through the sigmoid
            all_rows = _token_offsets(T, 1, x.device)
            d_sh_inter_s = ops.grouped_gemm_nt(dy, sh_down.unsqueeze(0), all_rows, tile_cfg=cfg)
            if ctx.needs_input_grad[5]:
                d_sh_down = _dense_weight_grad(sh_inter_s, dy, tile_cfg=cfg)
            d_sh_gu, d_sig = ops.gated_act_bwd(
                sh_gu, d_sh_inter_s, opts["act"], row_scale=sh_sig, slot_of=_token_ids(T, x.device), tk=(T, 1)
            )
            if ctx.needs_input_grad[4]:
                d_sh_gate_up = _dense_weight_grad(x, d_sh_gu, tile_cfg=cfg)
            d_pre = (d_sig.reshape(T) * sh_sig * (1.0 - sh_sig)).to(x.dtype).unsqueeze(1)  # [T,1]
            if ctx.needs_input_grad[6]:
                d_sh_out_gate = torch.matmul(x.t(), d_pre)

        dx = None
        if ctx.needs_input_grad[0]:
            d_xp = ops.grouped_gemm_nt(d_gate_up, w_gate_up, offsets, tile_cfg=cfg, workspace=ws, map_ready=True)
            dx_dense = torch.matmul(d_logits, router_gate)
            if ctx.shared:
                dx_dense.addmm_(d_pre, sh_out_gate.t())
                dx_dense += ops.grouped_gemm_nt(d_sh_gu, sh_gate_up.unsqueeze(0), all_rows, tile_cfg=cfg)
            dx = ops.gather_rows_bwd(d_xp, row_of, addend=dx_dense)
        if side is not None:
            main.wait_stream(side)
        return dx, d_router_gate, d_w_gate_up, d_w_down, d_sh_gate_up, d_sh_down, d_sh_out_gate, None, None


class _UngatedExpertLayerFn(torch.autograd.Function):
    """The layer with is_gated=False (moe.py:101-106, 188-191, 306-311): an expert is two plain
    linear maps, out = (x @ W_up[e]) @ W_down[e] with W_up [E,H,I] -- the reference applies its
    activation only inside the gated branch -- and the routing scores weight the combine
    (moe.py:450-461).  Same routing, permutation, load-balance hook and gradients as the gated
    layer; the grouped GEMMs run without an activation epilogue."""

    @staticmethod
    def forward(ctx, x, router_gate, w_up, w_down, sh_up, sh_down, sh_out_gate, replay, opts):
        T, H = x.shape
        K = opts["top_k"]
        timers: PhaseTimers = opts["timers"]
        cfg = opts["tile_cfg"]
        logits, probs, topk_idx, scores, ws, (counts, offsets, token_of, slot_of, row_of, scores_perm) = _route(
            x, router_gate, replay, opts
        )
        timers.start("groupGeMM")
        inter = ops.grouped_gemm_nn(x, w_up, offsets, a_row_map=token_of, n_rows=T * K, tile_cfg=cfg, workspace=ws,
                                    map_ready=True)
        out = ops.grouped_gemm_nn(inter, w_down, offsets, tile_cfg=cfg, workspace=ws, map_ready=True)
        timers.stop("groupGeMM")
        timers.start("moe-combine")
        y = ops.combine_fwd(out, row_of, scores)
        timers.stop("moe-combine")

        shared = sh_up is not None
        sh_inter = sh_out = sh_sig = None
        if shared:
            # dense linear maps over all T tokens: plain library GEMMs, like the reference's
            timers.start("shared-expert")
            sh_inter = torch.matmul(x, sh_up)
            sh_out = torch.matmul(sh_inter, sh_down)
            sh_sig = torch.sigmoid(torch.matmul(x, sh_out_gate))  # [T,1]
            y = y + sh_out * sh_sig
            timers.stop("shared-expert")

        ctx.opts = opts
        ctx.shared = shared
        ctx.gemm_ws = ws
        ctx.save_for_backward(x, router_gate, w_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, scores,
                              inter, out, sh_up, sh_down, sh_out_gate, sh_inter, sh_out, sh_sig)
        if opts["want_scores"]:
            scores_out = scores_perm.to(x.dtype)
        else:
            scores_out = scores_perm.new_empty(0)
            ctx.mark_non_differentiable(scores_out)
        ctx.set_materialize_grads(False)
        cap = opts.get("capture")
        if cap is not None:
            cap.update(logits=logits, probs=probs, topk_idx=topk_idx, scores=scores, counts=counts, offsets=offsets,
                       token_of=token_of, slot_of=slot_of, row_of=row_of)
        return y, scores_out

    @staticmethod
    def backward(ctx, dy, ds_perm):
        (x, router_gate, w_up, w_down, probs, topk_idx, counts, offsets, row_of, token_of, scores,
         inter, out, sh_up, sh_down, sh_out_gate, sh_inter, sh_out, sh_sig) = ctx.saved_tensors
        opts = ctx.opts
        E, K = opts["num_experts"], opts["top_k"]
        T = x.shape[0]
        cfg = opts["tile_cfg"]
        if dy is None and ds_perm is None:
            return (None,) * 9
        dy = torch.zeros_like(x) if dy is None else dy.contiguous()
        ws = ctx.gemm_ws  # still holds the forward's tile map

        # d_out[r] = s_r * dy[token_of[r]],  d_scores[t,k] = <dy[t], out[row_of[t,k]]>
        d_out, d_scores = ops.combine_bwd(dy, out, row_of, scores)
        if ds_perm is not None:
            d_scores = d_scores + ds_perm.float()[row_of.long()]
        d_inter = ops.grouped_gemm_nt(d_out, w_down, offsets, tile_cfg=cfg, workspace=ws, map_ready=True)
        d_w_down = ops.grouped_gemm_wgrad(inter, d_out, offsets, E, tile_cfg=cfg) if ctx.needs_input_grad[3] else None
        d_w_up = None
        if ctx.needs_input_grad[2]:
            d_w_up = ops.grouped_gemm_wgrad(x, d_inter, offsets, E, tile_cfg=cfg, a_row_map=token_of)

        d_logits = ops.router_bwd(
            d_scores, probs, topk_idx, counts, x.dtype, opts["normalize"], opts["loss_coeff"] / T / opts["ep_size"]
        )
        d_router_gate = _router_weight_grad(d_logits, x) if ctx.needs_input_grad[1] else None
        cap = opts.get("capture")
        if cap is not None:
            cap.update(d_scores=d_scores, d_logits=d_logits)

        d_sh_up = d_sh_down = d_sh_out_gate = d_sh_inter = d_pre = None
        if ctx.shared:
            d_sh_out = dy * sh_sig
            d_sig = (dy.float() * sh_out.float()).sum(dim=1, keepdim=True)
            sig = sh_sig.float()
            d_pre = (d_sig * sig * (1.0 - sig)).to(x.dtype)  # [T,1]
            d_sh_inter = torch.matmul(d_sh_out, sh_down.t())
            if ctx.needs_input_grad[5]:
                d_sh_down = torch.matmul(sh_inter.t(), d_sh_out)
            if ctx.needs_input_grad[4]:
                d_sh_up = torch.matmul(x.t(), d_sh_inter)
            if ctx.needs_input_grad[6]:
                d_sh_out_gate = torch.matmul(x.t(), d_pre)

        dx = None
        if ctx.needs_input_grad[0]:
            d_xp = ops.grouped_gemm_nt(d_inter, w_up, offsets, tile_cfg=cfg, workspace=ws, map_ready=True)
            dx_dense = torch.matmul(d_logits, router_gate)
            if ctx.shared:
                dx_dense.addmm_(d_pre, sh_out_gate.t())
                dx_dense.addmm_(d_sh_inter, sh_up.t())
            dx = ops.gather_rows_bwd(d_xp, row_of, addend=dx_dense)
        return dx, d_router_gate, d_w_up, d_w_down, d_sh_up, d_sh_down, d_sh_out_gate, None, None


class ArcticMoE(nn.Module):
    """Mixture-of-experts layer with the reference's surface (moe.py:63-323).

    Args:
        config: MoEConfig (or any object with the same attributes; the reference passes a
                SimpleNamespace, utils.py:107-161)

    Attributes beyond the reference's, all optional:
        tile_cfg: tile shape of the grouped GEMMs (0 = the library's default; 1, 2, 3, 5 for tuning)
        check_replay: raise on a replayed expert id outside [0, E), as the reference's one_hot does
                (one host synchronisation per replayed forward; skipped under graph capture)
        overlap_weight_grads: run the two expert weight gradients of the backward on a second stream
        capture: a dict that receives the routing intermediates of each forward (tests)
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
        if self.use_custom_kernel:
            import warnings

            warnings.warn(
                "ArcticMoE: use_custom_moe_kernel=True is ignored -- the layer computes the reference's default path "
                "(ragged rows, load-balance gradient, scores normalised in the gate), not its capacity-padded one",
                stacklevel=2,
            )
        if self.ep_size != 1:
            raise NotImplementedError("this build runs the expert layer on one GPU (ep_size must be 1)")
        self.is_gated = bool(getattr(config, "is_gated", True))
        self._act_code = classify_activation(config.act_fn)

        self.timers = PhaseTimers()
        self.wall_clock_breakdown = False
        self.gate_time = 0.0
        self.num_local_experts = self.num_experts // self.ep_size
        self.tile_cfg = 0  # 0 = library default tile shape; other values are for tuning
        # replayed expert ids outside [0, E) raise like the reference's one_hot (one host synchronisation per
        # replayed forward); False: no check, the permutation kernels clamp them
        self.check_replay = True
        self.capture = None  # set to a dict to receive the routing intermediates of each forward

        dt = self.input_dtype
        # gate and up projection interleaved when gated, one plain projection otherwise (moe.py:101-106)
        up_cols = (2 if self.is_gated else 1) * self.intermediate_dim
        self.router_gate = nn.Parameter(torch.empty((self.num_experts, self.model_dim), dtype=dt))
        self.expert_gate_up = nn.Parameter(
            torch.empty((self.num_local_experts, self.model_dim, up_cols), dtype=dt)
        )
        self.gate_scale = 1.0
        self.up_scale = 0.0
        self.expert_down = nn.Parameter(torch.empty((self.num_local_experts, self.intermediate_dim, self.model_dim), dtype=dt))
        if getattr(config, "use_shared_expert", False):
            self.shared_expert_gate_up = nn.Parameter(torch.empty((self.model_dim, up_cols), dtype=dt))
            self.shared_expert_down = nn.Parameter(torch.empty((self.intermediate_dim, self.model_dim), dtype=dt))
            self.shared_expert_output_gate = nn.Parameter(torch.empty(self.model_dim, 1, dtype=dt))
        self.enable_routing_replay = getattr(config, "enable_routing_replay", False)
        # backward: the two expert weight gradients on a second stream (see _side_stream)
        self.overlap_weight_grads = True

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
            check_replay=self.check_replay,
            overlap_weight_grads=self.overlap_weight_grads,
            want_scores=bool(getattr(self._config, "return_router_scores", False)),
            timers=self.timers,
            capture=self.capture,
        )
        replay = routing_replay_assignments if self.enable_routing_replay else None
        if self.tile_cfg == 3 and x.dtype == torch.float16:
            # (the row-grouped products are not built for that combination; the default shape is)
            raise RuntimeError("ArcticMoE: tile_cfg 3 is not available for float16 layers")
        if x.shape[0] == 0:
            # no tokens (the reference returns an empty tensor from the same code path): nothing to
            # launch; the result still hangs off every parameter so that their gradients are zeros
            output = (x + sum(p.sum() for p in self.parameters()) * 0).reshape(orig_shape)
            self.timers.stop("amoe e2e")
            return (output, x.new_zeros(0)) if getattr(self._config, "return_router_scores", False) else output
        shared = (None, None, None)
        if getattr(self._config, "use_shared_expert", False):
            shared = (self.shared_expert_gate_up, self.shared_expert_down, self.shared_expert_output_gate)
        # the kernels are launched on the current device's current stream: make x's device current
        with torch.cuda.device(x.device) if x.is_cuda else contextlib.nullcontext():
            layer_fn = _ExpertLayerFn if self.is_gated else _UngatedExpertLayerFn
            output, scores = layer_fn.apply(
                x, self.router_gate, self.expert_gate_up, self.expert_down, *shared, replay, opts
            )
        output = output.reshape(orig_shape)
        self.timers.stop("amoe e2e")
        return (output, scores) if getattr(self._config, "return_router_scores", False) else output
