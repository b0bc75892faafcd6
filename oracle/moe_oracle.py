"""CPU oracle for the ArcticMoE expert layer (TEST INFRASTRUCTURE ONLY).

This module is a checker.  It restates, on the CPU with torch/numpy, the
algorithm of the reference's default (non-Triton, non-custom-kernel, EP=1)
ArcticMoE path.  Nothing in the shipped package imports it: only the test
suite, the smoke check and the CPU-baseline leg of the benchmark do, and they
use it as the thing results are compared to, never as the thing measured or
shipped.

Each function cites the reference lines it follows (paths relative to the
reference tree):

  router linear        arctic_training/model/moe/moe.py:231-233
  softmax / top-k      arctic_training/model/moe/moe.py:359-366
  tie rule             arctic_training/kernels/moe_ops/top_k_gating/top_k_gating_cuda.cu:113-128
                       (value descending, lowest expert index wins a tie;
                       torch.topk itself leaves tie order unspecified)
  permutation / counts arctic_training/model/moe/moe.py:367-382
  load-balance hook    arctic_training/model/moe/moe.py:383-409
  row gather           arctic_training/model/moe/moe.py:353-357
  grouped GEMM         arctic_training/model/moe/moe.py:54-60
  gated expert FFN     arctic_training/model/moe/moe.py:176-193 (scale constants :110-111)
  expert FFN, no gate  arctic_training/model/moe/moe.py:101-106, 188-191 (is_gated=False: no activation)
  weighted combine     arctic_training/model/moe/moe.py:450-461
  shared expert        arctic_training/model/moe/moe.py:305-314 (parameters :116-130)
  weight layout        arctic_training/model/moe/utils.py:249-266

Parity pins (all in tests/test_oracle_pins.py; the reference holds no golden
vector for this path, so every function is pinned by mathematics or by the
installed third-party HF block instead):

  softmax_probs         closed forms on 2/3-element rows + library identity
  topk_canonical        brute-force full sort, torch.topk on tie-free rows,
                        hand-built tied rows
  normalize_and_cast    closed form, sum-to-one invariant
  permutation           literal one_hot/where/cat formulation vs. stable
                        counting sort, exhaustively for T<=4, E<=3, K<=2, plus
                        the invariants and a worked example
  grouped_gemm          per-expert fp64 matmul on the same row ranges; empty
                        groups leave zero rows
  expert_ffn            de-interleaved chunk formulation; silu closed form;
                        is_gated=False: token-major dense closed form of the
                        whole layer (two products, no activation)
  combine               dense token-major sum
  shared_expert         the installed transformers Qwen2MoeSparseMoeBlock
                        (shared MLP + sigmoid gate) after weight-layout mapping,
                        forward and all gradients; closed form on a 1x1 case
  load-balance hook     closed form d/dprobs of coeff * sum_e freq_e * mean_t p
  forward (autograd)    torch.autograd.gradcheck in fp64
  analytic_backward     equality with autograd of forward
  whole layer           the installed transformers Qwen3MoeSparseMoeBlock after
                        weight-layout mapping (forward and all gradients)
"""

from dataclasses import dataclass
from typing import Callable, Dict, Optional

import numpy as np
import torch
import torch.nn.functional as F


@dataclass
class OracleConfig:
    """The MoEConfig fields that are live on the default path
    (arctic_training/model/moe/moe.py:33-51, values installed at utils.py:107-161)."""

    model_dim: int
    intermediate_dim: int
    num_experts: int
    top_k: int
    normalize_topk_scores: bool = True
    loss_coeff: float = 0.01
    ep_size: int = 1
    act: str = "silu"
    is_gated: bool = True


def activation(name: str) -> Callable[[torch.Tensor], torch.Tensor]:
    """utils.py:118-127: silu / gelu / relu from torch.nn.functional, or the
    gpt-oss variant x * sigmoid(1.702 x)."""
    if name == "silu":
        return F.silu
    if name == "gelu":
        return F.gelu
    if name == "relu":
        return F.relu
    if name == "gpt_oss":
        return lambda x: x * torch.sigmoid(x * 1.702)
    raise ValueError(f"unsupported activation {name}")


# --------------------------------------------------------------------------
# routing
# --------------------------------------------------------------------------


def router_linear(x2d: torch.Tensor, router_gate: torch.Tensor) -> torch.Tensor:
    """moe.py:233 -- logits = F.linear(hidden_states, router_gate); result in the
    dtype of the operands (bf16 logits are rounded to bf16)."""
    return F.linear(x2d, router_gate)


def softmax_probs(logits: torch.Tensor) -> torch.Tensor:
    """moe.py:361 -- softmax over experts evaluated in float32 whatever the
    logits dtype (float64 logits stay float64 so that the exact-arithmetic mode
    of the oracle is not degraded)."""
    dt = torch.float64 if logits.dtype == torch.float64 else torch.float32
    return F.softmax(logits, dim=-1, dtype=dt)


def topk_canonical(values: torch.Tensor, k: int):
    """moe.py:363 with the tie rule of top_k_gating_cuda.cu:113-128: the k
    largest entries of each row in descending order; among equal values the
    lowest expert index comes first.  Returns (top values, int64 indices)."""
    v = values.detach().cpu().numpy()
    # a stable sort of the negated values keeps ascending index inside a tie
    order = np.argsort(-v.astype(np.float64), axis=-1, kind="stable")[:, :k]
    idx = torch.from_numpy(np.ascontiguousarray(order)).to(torch.int64)
    return torch.gather(values, -1, idx), idx


def normalize_and_cast(topk_scores: torch.Tensor, normalize: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """moe.py:364-366."""
    if normalize:
        topk_scores = topk_scores / torch.sum(topk_scores, dim=-1, keepdim=True)
    return topk_scores.to(out_dtype)


def permutation(expert_idx_tk: torch.Tensor, num_experts: int):
    """moe.py:367-382 -- the order of the routed rows.

    `expert_idx_tk` is [T, K].  The flat position of slot (t, k) is
    f = k * T + t (k-major, from `.t().reshape(-1)`).  Rows are grouped by
    expert in ascending expert id and, inside an expert, in ascending f:
    exactly what concatenating `where(one_hot[:, e])` over e yields.

    Returns (perm [R] flat positions, token_ids [R] = perm % T,
    counts [E]) as int64 tensors.
    """
    T, K = expert_idx_tk.shape
    flat = expert_idx_tk.t().reshape(-1).cpu().numpy().astype(np.int64)
    perm_parts = [np.nonzero(flat == e)[0] for e in range(num_experts)]
    perm = np.concatenate(perm_parts) if perm_parts else np.zeros(0, np.int64)
    counts = np.array([p.size for p in perm_parts], dtype=np.int64)
    token_ids = perm % T
    return (
        torch.from_numpy(perm.astype(np.int64)),
        torch.from_numpy(token_ids.astype(np.int64)),
        torch.from_numpy(counts),
    )


def inverse_row_map(perm: torch.Tensor, T: int, K: int) -> torch.Tensor:
    """row_of[t, k] = the routed row that holds slot (t, k): the inverse of
    `perm` re-indexed token-major.  (The reference never builds this map on its
    default path -- its index_add_ scatters instead -- but the inverse of a
    permutation is unique, so it is pinned by perm.)"""
    R = perm.numel()
    inv = torch.empty(R, dtype=torch.int64)
    inv[perm] = torch.arange(R, dtype=torch.int64)
    return inv.view(K, T).t().contiguous()


def gate(
    logits: torch.Tensor,
    cfg: OracleConfig,
    score_dtype: torch.dtype,
    select_values: Optional[torch.Tensor] = None,
    replay_assignments: Optional[torch.Tensor] = None,
):
    """moe.py:359-411 without the (identity at EP=1) count exchange.

    `select_values`, when given, supplies the numbers the top-k *selection*
    looks at (e.g. logits produced by the device under test) while the
    probabilities and their gradient still come from `logits`; selection on
    logits and on their float32 softmax agree unless two distinct logits round
    to one probability, which `selection_agrees` reports.

    Returns a dict with probs, topk_idx [T,K], scores_tk [T,K] (score_dtype),
    perm, token_ids, counts, scores_perm [R], expert_freq.
    """
    E = cfg.num_experts
    logits = logits.view(-1, E)
    probs = softmax_probs(logits)
    sel = probs if select_values is None else select_values.view(-1, E).to(torch.float64)
    _, topk_idx = topk_canonical(sel, cfg.top_k)
    topk_p = torch.gather(probs, -1, topk_idx)
    scores_tk = normalize_and_cast(topk_p, cfg.normalize_topk_scores, score_dtype)
    assign = topk_idx if replay_assignments is None else replay_assignments.to(torch.int64)
    perm, token_ids, counts = permutation(assign, E)
    scores_perm = scores_tk.t().reshape(-1)[perm]
    total = counts.sum()
    expert_freq = counts.to(probs.dtype) / total.to(probs.dtype)
    return dict(
        probs=probs,
        topk_idx=topk_idx,
        assign_idx=assign,
        scores_tk=scores_tk,
        perm=perm,
        token_ids=token_ids,
        counts=counts,
        scores_perm=scores_perm,
        expert_freq=expert_freq,
    )


def selection_agrees(logits: torch.Tensor, k: int) -> bool:
    """True when choosing the top-k on the logits and on their float32 softmax
    gives the same indices in the same order for every row."""
    _, a = topk_canonical(logits.to(torch.float64), k)
    _, b = topk_canonical(softmax_probs(logits), k)
    return bool(torch.equal(a, b))


# --------------------------------------------------------------------------
# experts
# --------------------------------------------------------------------------


def grouped_gemm(A: torch.Tensor, B: torch.Tensor, rows_cumsum: torch.Tensor) -> torch.Tensor:
    """moe.py:54-60 -- C[rows of expert e] = A[rows of expert e] @ B[e], output
    zero-initialised, rows taken from the inclusive cumulative counts."""
    total = int(rows_cumsum[-1]) if rows_cumsum.numel() else 0
    out = torch.zeros((total, B.shape[-1]), dtype=A.dtype)
    for e in range(rows_cumsum.numel()):
        start = 0 if e == 0 else int(rows_cumsum[e - 1])
        end = int(rows_cumsum[e])
        out[start:end, :] = torch.matmul(A[start:end, :], B[e])
    return out


def expert_ffn(xp: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, rows_cumsum, act: str,
               is_gated: bool = True):
    """moe.py:176-193 -- gate in the even, up in the odd columns of the first
    GEMM's output; inter = (up + 0.0) * act(gate * 1.0); second GEMM.
    Returns (gate_up, inter, out).  With is_gated=False (w_gate_up [E,H,I], moe.py:101-106) the
    first GEMM's output goes to the second as it is: the activation sits inside the gated branch
    only (moe.py:188-191)."""
    fn = activation(act)
    gu = grouped_gemm(xp, w_gate_up, rows_cumsum)
    if not is_gated:
        return gu, gu, grouped_gemm(gu, w_down, rows_cumsum)
    g, u = gu[..., 0::2], gu[..., 1::2]
    inter = (u + 0.0) * fn(g * 1.0)
    out = grouped_gemm(inter, w_down, rows_cumsum)
    return gu, inter, out


def combine(moe_out: torch.Tensor, token_ids: torch.Tensor, scores_perm: torch.Tensor, top_k: int) -> torch.Tensor:
    """moe.py:450-461 -- y = 0; y[token_ids[r]] += moe_out[r] * scores[r]."""
    T = moe_out.shape[0] // top_k
    y = torch.zeros((T, moe_out.shape[1]), dtype=moe_out.dtype)
    return y.index_add(0, token_ids, moe_out * scores_perm[:, None])


def shared_expert(x2d: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, w_out_gate: torch.Tensor, act: str,
                  is_gated: bool = True):
    """moe.py:305-314 -- a dense gated FFN every token goes through, scaled per token by a
    sigmoid gate: (up * act(gate)) @ W_down * sigmoid(x @ w_out_gate).  w_gate_up [H, 2I] has the
    gate in the even and the up projection in the odd columns, w_down is [I, H], w_out_gate [H, 1]."""
    fn = activation(act)
    s_inter = torch.matmul(x2d, w_gate_up)
    if is_gated:  # moe.py:308-310; without the gate the first product feeds the second unchanged
        s_gate, s_up = s_inter[..., 0::2], s_inter[..., 1::2]
        s_inter = s_up * fn(s_gate)
    s_out = torch.matmul(s_inter, w_down)
    s_out_gate = torch.matmul(x2d, w_out_gate)
    return s_out * torch.sigmoid(s_out_gate)


# --------------------------------------------------------------------------
# whole layer
# --------------------------------------------------------------------------


def forward(
    x: torch.Tensor,
    router_gate: torch.Tensor,
    expert_gate_up: torch.Tensor,
    expert_down: torch.Tensor,
    cfg: OracleConfig,
    compute_dtype: Optional[torch.dtype] = None,
    logits_for_selection: Optional[torch.Tensor] = None,
    replay_assignments: Optional[torch.Tensor] = None,
    model_dtype: Optional[torch.dtype] = None,
    shared=None,
) -> Dict[str, torch.Tensor]:
    """moe.py:219-323 on the default path at EP=1, differentiable with autograd.
    `shared` = (shared_expert_gate_up, shared_expert_down, shared_expert_output_gate) adds the
    shared expert (use_shared_expert=True).

    compute_dtype=None runs every op in the dtype of the inputs, with the
    reference's rounding after each op ("reference rounding" mode: what the
    reference computes on a CPU).  compute_dtype=float32/float64 up-casts the
    (already rounded) inputs once and keeps every intermediate in that type
    ("exact" mode); the logits are then still rounded through the model dtype
    (`model_dtype`, by default the dtype of x), because that rounding decides
    the routing.
    """
    in_dtype = model_dtype if model_dtype is not None else x.dtype
    orig_shape = x.shape
    x2d = x.reshape(-1, x.shape[-1])
    if compute_dtype is not None and compute_dtype != in_dtype:
        x2d, router_gate, expert_gate_up, expert_down = (
            t.to(compute_dtype) for t in (x2d, router_gate, expert_gate_up, expert_down)
        )
        if shared is not None:
            shared = tuple(t.to(compute_dtype) for t in shared)
        logits = router_linear(x2d, router_gate)
        # straight-through rounding of the logits to the model dtype
        logits = logits + (logits.detach().to(in_dtype).to(compute_dtype) - logits.detach())
        score_dtype = compute_dtype
    else:
        logits = router_linear(x2d, router_gate)
        score_dtype = in_dtype

    g = gate(logits, cfg, score_dtype, select_values=logits_for_selection, replay_assignments=replay_assignments)
    probs = g["probs"]
    T = probs.shape[0]
    if probs.requires_grad:
        freq = g["expert_freq"]
        coeff = cfg.loss_coeff / T / 1

        def _lb_hook(grad):
            # moe.py:393-406
            if grad is None:  # autograd may probe with an undefined gradient
                return None
            return grad + freq.unsqueeze(0).to(grad.dtype) * coeff / cfg.ep_size

        probs.register_hook(_lb_hook)

    xp = x2d[g["token_ids"]]
    cumsum = g["counts"].cumsum(0)
    gu, inter, out = expert_ffn(xp, expert_gate_up, expert_down, cumsum, cfg.act, cfg.is_gated)
    y = combine(out, g["token_ids"], g["scores_perm"], cfg.top_k)
    if shared is not None:
        y = y + shared_expert(x2d, *shared, cfg.act, cfg.is_gated)
    res = dict(g)
    res.update(logits=logits, xp=xp, gate_up=gu, inter=inter, moe_out=out, y=y.reshape(orig_shape), cumsum=cumsum)
    return res


def forward_backward(x, router_gate, expert_gate_up, expert_down, dy, cfg, **kw):
    """forward + autograd backward with upstream gradient dy.  Gradients are
    returned in the compute dtype (no rounding back to the input dtype)."""
    model_dtype = x.dtype
    leaf_dtype = kw.get("compute_dtype") or model_dtype
    leaves = [
        t.detach().to(leaf_dtype).clone().requires_grad_(True) for t in (x, router_gate, expert_gate_up, expert_down)
    ]
    shared = kw.pop("shared", None)
    d_scores_perm = kw.pop("d_scores_perm", None)  # upstream gradient of the returned scores (moe.py:323)
    if shared is not None:
        shared = tuple(t.detach().to(leaf_dtype).clone().requires_grad_(True) for t in shared)
    res = forward(*leaves, cfg, model_dtype=model_dtype, shared=shared, **kw)
    y = res["y"]
    if d_scores_perm is None:
        y.backward(dy.to(y.dtype).reshape(y.shape))
    else:
        sp = res["scores_perm"]
        torch.autograd.backward([y, sp], [dy.to(y.dtype).reshape(y.shape), d_scores_perm.to(sp.dtype)])
    res["dx"], res["d_router_gate"], res["d_expert_gate_up"], res["d_expert_down"] = (t.grad for t in leaves)
    if shared is not None:
        res["d_shared_expert_gate_up"], res["d_shared_expert_down"], res["d_shared_expert_output_gate"] = (
            t.grad for t in shared
        )
    return res


def silu_grad(g: torch.Tensor) -> torch.Tensor:
    s = torch.sigmoid(g)
    return s * (1 + g * (1 - s))


def router_backward(d_s_tk, probs, topk_idx, expert_freq, cfg, T):
    """Gradient of the router from d(scores) [T,K] back to the logits: the derivative of the
    normalisation and gather of moe.py:363-365, the load-balance hook moe.py:393-406 and the
    softmax of moe.py:361.  Returns (d_probs, d_logits), both [T,E] in the dtype of probs."""
    p_top = torch.gather(probs, -1, topk_idx)
    if cfg.normalize_topk_scores:
        S = p_top.sum(-1, keepdim=True)
        sn = p_top / S
        d_ptop = (d_s_tk - (d_s_tk * sn).sum(-1, keepdim=True)) / S
    else:
        d_ptop = d_s_tk
    d_probs = torch.zeros_like(probs).scatter_add(-1, topk_idx, d_ptop)
    d_probs = d_probs + expert_freq[None, :] * (cfg.loss_coeff / T) / cfg.ep_size
    d_logits = probs * (d_probs - (probs * d_probs).sum(-1, keepdim=True))
    return d_probs, d_logits


def analytic_backward(res: Dict[str, torch.Tensor], x2d, router_gate, expert_gate_up, expert_down, dy2d, cfg):
    """Stage-by-stage backward written out by hand (no autograd), so that each
    device backward kernel has a stage-level reference.  `res` is the result of
    `forward` in an exact mode (float32/float64); the formulas are the
    derivatives of moe.py:233, :361-366, :356, :187-192, :460 and the hook at
    :393-406.  SiLU only."""
    assert cfg.act == "silu" and cfg.is_gated
    dt = res["y"].dtype
    x2d, router_gate, expert_gate_up, expert_down, dy2d = (
        t.detach().to(dt) for t in (x2d, router_gate, expert_gate_up, expert_down, dy2d)
    )
    T, K, E = x2d.shape[0], cfg.top_k, cfg.num_experts
    tok, perm, counts = res["token_ids"], res["perm"], res["counts"]
    s_perm = res["scores_perm"].detach()
    out, inter, gu = res["moe_out"].detach(), res["inter"].detach(), res["gate_up"].detach()
    xp = res["xp"].detach()
    offs = torch.cat([torch.zeros(1, dtype=torch.int64), counts.cumsum(0)])

    # combine backward
    dy_rows = dy2d[tok]
    d_out = dy_rows * s_perm[:, None]
    d_s_perm = (dy_rows * out).sum(-1)
    # down projection
    d_inter = torch.zeros_like(inter)
    d_wd = torch.zeros_like(expert_down)
    for e in range(E):
        a, b = int(offs[e]), int(offs[e + 1])
        d_inter[a:b] = d_out[a:b] @ expert_down[e].t()
        d_wd[e] = inter[a:b].t() @ d_out[a:b]
    # gated activation
    gte, up = gu[:, 0::2], gu[:, 1::2]
    d_up = d_inter * F.silu(gte)
    d_gate = d_inter * up * silu_grad(gte)
    d_gu = torch.stack((d_gate, d_up), dim=-1).reshape(gu.shape)
    # gate_up projection
    d_xp = torch.zeros_like(xp)
    d_wgu = torch.zeros_like(expert_gate_up)
    for e in range(E):
        a, b = int(offs[e]), int(offs[e + 1])
        d_xp[a:b] = d_gu[a:b] @ expert_gate_up[e].t()
        d_wgu[e] = xp[a:b].t() @ d_gu[a:b]
    dx = torch.zeros_like(x2d).index_add(0, tok, d_xp)
    # scores back to [T, K]
    d_s_flat = torch.zeros(T * K, dtype=dt)
    d_s_flat[perm] = d_s_perm
    d_s_tk = d_s_flat.view(K, T).t()
    d_probs, d_logits = router_backward(d_s_tk, res["probs"].detach().to(dt), res["topk_idx"], res["expert_freq"].to(dt),
                                        cfg, T)
    d_wr = d_logits.t() @ x2d
    dx = dx + d_logits @ router_gate
    return dict(
        d_out=d_out,
        d_scores_perm=d_s_perm,
        d_scores_tk=d_s_tk,
        d_inter=d_inter,
        d_gate_up=d_gu,
        d_xp=d_xp,
        d_probs=d_probs,
        d_logits=d_logits,
        dx=dx,
        d_router_gate=d_wr,
        d_expert_gate_up=d_wgu,
        d_expert_down=d_wd,
    )


# --------------------------------------------------------------------------
# synthetic inputs shared by tests, fixtures and the benchmark
# --------------------------------------------------------------------------


def make_inputs(T, H, E, K, I, dtype, seed, bias_hot=None, n_hot=0, n_dead=0):
    """Seeded inputs generated on the CPU in float32 then cast: x, dy ~ N(0,1);
    every weight ~ N(0, 0.02).  With n_hot/n_dead set, a constant input channel
    (x[:, H-1] = 1) and per-expert entries of router_gate[:, H-1] bias the first
    n_hot experts up by `bias_hot` and push the last n_dead experts to zero
    traffic."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    wr = torch.randn(E, H, generator=g) * 0.02
    wgu = torch.randn(E, H, 2 * I, generator=g) * 0.02
    wd = torch.randn(E, I, H, generator=g) * 0.02
    dy = torch.randn(T, H, generator=g)
    if n_hot or n_dead:
        x[:, H - 1] = 1.0
        wr[:, H - 1] = 0.0
        if n_hot:
            wr[:n_hot, H - 1] = float(bias_hot)
        if n_dead:
            wr[E - n_dead :, H - 1] = -1.0e4
    return tuple(t.to(dtype) for t in (x, wr, wgu, wd, dy))


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.detach().to(torch.float64).flatten()
    b = b.detach().to(torch.float64).flatten()
    den = float(torch.linalg.vector_norm(b))
    num = float(torch.linalg.vector_norm(a - b))
    return num / den if den > 0 else num
