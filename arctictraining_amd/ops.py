"""Thin tensor-level wrappers over the C ABI: allocate outputs with torch, pass raw device
pointers and the current HIP stream, raise on error.  One function per stage of the
expert layer, in the order the reference's forward runs them
(arctic_training/model/moe/moe.py:219-323).
"""
from typing import Optional, Tuple

import torch

from . import _lib

F32, BF16, F16 = 0, 1, 2
_DTYPE_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
ACT_SILU, ACT_GELU, ACT_RELU, ACT_GPT_OSS = 0, 1, 2, 3
TILE_MAP_READY = 0x100  # AMOE_TILE_MAP_READY


def _dtype_code(t) -> int:
    """dtype code of the C ABI for a tensor or a torch dtype"""
    dt = t.dtype if isinstance(t, torch.Tensor) else t
    code = _DTYPE_CODES.get(dt)
    if code is None:
        raise RuntimeError(f"the expert-layer kernels support float32, bfloat16 and float16, not {dt}")
    return code


def _chk(t: torch.Tensor, name: str, dtype=None) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (the HIP kernels have no CPU fallback)")
    if t.device.index != torch.cuda.current_device():
        # kernels are launched on the current device's current stream
        raise RuntimeError(f"{name} lives on {t.device} but the current device is cuda:{torch.cuda.current_device()}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")
    return t


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def router_topk_fwd(logits: torch.Tensor, top_k: int, normalize: bool):
    """logits [T,E] -> probs [T,E] f32, topk_idx [T,K] i32, scores [T,K] f32."""
    lib = _lib.load()
    _chk(logits, "logits")
    T, E = logits.shape
    probs = torch.empty((T, E), dtype=torch.float32, device=logits.device)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    scores = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    rc = lib.amoe_router_topk_fwd(
        logits.data_ptr(), _dtype_code(logits), T, E, top_k, int(normalize), probs.data_ptr(), idx.data_ptr(),
        scores.data_ptr(), _stream()
    )
    _lib.check(rc, "amoe_router_topk_fwd")
    return probs, idx, scores


def router_bwd(d_scores, probs, topk_idx, counts, out_dtype, normalize: bool, lb_coeff: float) -> torch.Tensor:
    lib = _lib.load()
    _chk(d_scores, "d_scores", torch.float32)
    _chk(probs, "probs", torch.float32)
    _chk(topk_idx, "topk_idx", torch.int32)
    _chk(counts, "counts", torch.int32)
    T, E = probs.shape
    K = topk_idx.shape[1]
    d_logits = torch.empty((T, E), dtype=out_dtype, device=probs.device)
    rc = lib.amoe_router_bwd(
        d_scores.data_ptr(), probs.data_ptr(), topk_idx.data_ptr(), counts.data_ptr(), _dtype_code(d_logits), T, E, K,
        int(normalize), float(lb_coeff), d_logits.data_ptr(), _stream()
    )
    _lib.check(rc, "amoe_router_bwd")
    return d_logits


def permute_plan(assign: torch.Tensor, num_experts: int, scores: Optional[torch.Tensor] = None,
                 gemm_workspace: Optional[torch.Tensor] = None, gemm_dtype: Optional[torch.dtype] = None, tile_cfg: int = 0):
    """assign [T,K] i32 -> counts [E], offsets [E+1], token_of [R], slot_of [R], row_of [T,K] (all i32) and,
    when scores [T,K] f32 is given, scores_perm [R] f32 (else None).  With gemm_workspace (and the
    dtype / tile_cfg of the row-grouped GEMMs that will use it) the plan also builds their tile map
    there, so that each of them can be called with map_ready=True."""
    lib = _lib.load()
    _chk(assign, "assign", torch.int32)
    T, K = assign.shape
    R, E, dev = T * K, num_experts, assign.device
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    token_of = torch.empty(R, dtype=torch.int32, device=dev)
    slot_of = torch.empty(R, dtype=torch.int32, device=dev)
    row_of = torch.empty((T, K), dtype=torch.int32, device=dev)
    scores_perm = None
    if scores is not None:
        _chk(scores, "scores", torch.float32)
        scores_perm = torch.empty(R, dtype=torch.float32, device=dev)
    ws_bytes = lib.amoe_permute_workspace_bytes(R, E)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    if gemm_workspace is not None:
        _chk(gemm_workspace, "gemm_workspace", torch.uint8)
        rc = lib.amoe_permute_plan_tiled(
            assign.data_ptr(), _ptr(scores), T, K, E, counts.data_ptr(), offsets.data_ptr(), token_of.data_ptr(),
            slot_of.data_ptr(), row_of.data_ptr(), _ptr(scores_perm), ws.data_ptr(), ws.numel(), gemm_workspace.data_ptr(),
            gemm_workspace.numel(), _dtype_code(gemm_dtype), tile_cfg, _stream()
        )
        _lib.check(rc, "amoe_permute_plan_tiled")
        return counts, offsets, token_of, slot_of, row_of, scores_perm
    rc = lib.amoe_permute_plan(
        assign.data_ptr(), _ptr(scores), T, K, E, counts.data_ptr(), offsets.data_ptr(), token_of.data_ptr(),
        slot_of.data_ptr(), row_of.data_ptr(), _ptr(scores_perm), ws.data_ptr(), ws.numel(), _stream()
    )
    _lib.check(rc, "amoe_permute_plan")
    return counts, offsets, token_of, slot_of, row_of, scores_perm


def permute_plan_static(assign: torch.Tensor, num_experts: int, scores: Optional[torch.Tensor] = None, out=None):
    """permute_plan through the entry point that allocates nothing: its counters live in a fixed
    array inside the library (ceil(T*K/512)*E <= 2^20).  `out` = (counts, offsets, token_of, slot_of,
    row_of, scores_perm) preallocated by the caller makes the call itself allocation-free."""
    lib = _lib.load()
    _chk(assign, "assign", torch.int32)
    T, K = assign.shape
    R, E, dev = T * K, num_experts, assign.device
    if out is None:
        i32 = dict(dtype=torch.int32, device=dev)
        out = (torch.empty(E, **i32), torch.empty(E + 1, **i32), torch.empty(R, **i32), torch.empty(R, **i32),
               torch.empty((T, K), **i32), torch.empty(R, dtype=torch.float32, device=dev) if scores is not None else None)
    counts, offsets, token_of, slot_of, row_of, scores_perm = out
    if scores is not None:
        _chk(scores, "scores", torch.float32)
    rc = lib.amoe_permute_plan_static(
        assign.data_ptr(), _ptr(scores), T, K, E, counts.data_ptr(), offsets.data_ptr(), token_of.data_ptr(),
        slot_of.data_ptr(), row_of.data_ptr(), _ptr(scores_perm) if scores is not None else None, _stream()
    )
    _lib.check(rc, "amoe_permute_plan_static")
    return counts, offsets, token_of, slot_of, row_of, (scores_perm if scores is not None else None)


def gather_rows_fwd(x: torch.Tensor, token_of: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    _chk(x, "x")
    _chk(token_of, "token_of", torch.int32)
    R, H = token_of.numel(), x.shape[1]
    xp = torch.empty((R, H), dtype=x.dtype, device=x.device)
    rc = lib.amoe_gather_rows_fwd(x.data_ptr(), token_of.data_ptr(), xp.data_ptr(), _dtype_code(x), R, H, _stream())
    _lib.check(rc, "amoe_gather_rows_fwd")
    return xp


def gather_rows_bwd(d_xp: torch.Tensor, row_of: torch.Tensor, addend: Optional[torch.Tensor] = None) -> torch.Tensor:
    lib = _lib.load()
    _chk(d_xp, "d_xp")
    _chk(row_of, "row_of", torch.int32)
    if addend is not None:
        _chk(addend, "addend", d_xp.dtype)
    T, K = row_of.shape
    H = d_xp.shape[1]
    dx = torch.empty((T, H), dtype=d_xp.dtype, device=d_xp.device)
    rc = lib.amoe_gather_rows_bwd(
        d_xp.data_ptr(), row_of.data_ptr(), _ptr(addend), dx.data_ptr(), _dtype_code(d_xp), T, K, H, _stream()
    )
    _lib.check(rc, "amoe_gather_rows_bwd")
    return dx


def combine_fwd(moe_out: torch.Tensor, row_of: torch.Tensor, scores: Optional[torch.Tensor]) -> torch.Tensor:
    """y[t] = sum_k scores[t,k] * moe_out[row_of[t,k]]; scores None = unweighted."""
    lib = _lib.load()
    _chk(moe_out, "moe_out")
    _chk(row_of, "row_of", torch.int32)
    if scores is not None:
        _chk(scores, "scores", torch.float32)
    T, K = row_of.shape
    H = moe_out.shape[1]
    y = torch.empty((T, H), dtype=moe_out.dtype, device=moe_out.device)
    rc = lib.amoe_combine_fwd(
        moe_out.data_ptr(), row_of.data_ptr(), _ptr(scores), y.data_ptr(), _dtype_code(moe_out), T, K, H, _stream()
    )
    _lib.check(rc, "amoe_combine_fwd")
    return y


def combine_bwd(dy, moe_out, row_of, scores, need_d_out: bool = True) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    lib = _lib.load()
    _chk(dy, "dy", moe_out.dtype)
    _chk(moe_out, "moe_out")
    _chk(row_of, "row_of", torch.int32)
    _chk(scores, "scores", torch.float32)
    T, K = row_of.shape
    H = moe_out.shape[1]
    d_out = torch.empty_like(moe_out) if need_d_out else None
    d_scores = torch.empty((T, K), dtype=torch.float32, device=dy.device)
    rc = lib.amoe_combine_bwd(
        dy.data_ptr(), moe_out.data_ptr(), row_of.data_ptr(), scores.data_ptr(), _ptr(d_out), d_scores.data_ptr(),
        _dtype_code(dy), T, K, H, _stream()
    )
    _lib.check(rc, "amoe_combine_bwd")
    return d_out, d_scores


def gemm_workspace(R: int, E: int, device) -> torch.Tensor:
    """Workspace of the row-grouped GEMMs (holds the tile map built from `offsets`).  Calls that
    share R, E, offsets, dtype and tile shape may share one workspace; all but the first can then
    pass map_ready=True and skip rebuilding the map."""
    n = _lib.load().amoe_grouped_gemm_workspace_bytes(R, E)
    return torch.empty(max(n, 16), dtype=torch.uint8, device=device)


def _ws_and_cfg(R, E, device, tile_cfg, workspace, map_ready):
    if workspace is None:
        if map_ready:
            raise RuntimeError("map_ready needs the workspace that holds the map")
        workspace = gemm_workspace(R, E, device)
    return workspace, (tile_cfg | TILE_MAP_READY) if map_ready else tile_cfg


def grouped_gemm_gateup_act_fwd(
    xp: torch.Tensor,
    w_gate_up: torch.Tensor,
    offsets: torch.Tensor,
    act: int = ACT_SILU,
    a_row_map: Optional[torch.Tensor] = None,
    n_rows: Optional[int] = None,
    tile_cfg: int = 0,
    want_gate_up: bool = True,
    row_scale: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    map_ready: bool = False,
):
    """gate_up [R,2I], inter [R,I] (times row_scale [R] when given) from xp [R,H] (or x [T,H] with
    a_row_map [R]) and w [E,H,2I]."""
    lib = _lib.load()
    _chk(xp, "xp")
    _chk(w_gate_up, "w_gate_up", xp.dtype)
    _chk(offsets, "offsets", torch.int32)
    if a_row_map is not None:
        _chk(a_row_map, "a_row_map", torch.int32)
    if row_scale is not None:
        _chk(row_scale, "row_scale", torch.float32)
    E, H, I2 = w_gate_up.shape
    R = int(n_rows if n_rows is not None else (a_row_map.numel() if a_row_map is not None else xp.shape[0]))
    I = I2 // 2
    gate_up = torch.empty((R, I2), dtype=xp.dtype, device=xp.device) if want_gate_up else None
    inter = torch.empty((R, I), dtype=xp.dtype, device=xp.device)
    ws, tile_cfg = _ws_and_cfg(R, E, xp.device, tile_cfg, workspace, map_ready)
    rc = lib.amoe_grouped_gemm_gateup_act_fwd(
        xp.data_ptr(), _ptr(a_row_map), w_gate_up.data_ptr(), offsets.data_ptr(), _ptr(row_scale), _ptr(gate_up),
        inter.data_ptr(),
        _dtype_code(xp), R, E, H, I, act, ws.data_ptr(), ws.numel(), tile_cfg, _stream()
    )
    _lib.check(rc, "amoe_grouped_gemm_gateup_act_fwd")
    return gate_up, inter


def grouped_gemm_nn(A, B, offsets, a_row_map=None, n_rows=None, tile_cfg: int = 0, workspace=None,
                    map_ready: bool = False) -> torch.Tensor:
    """C[rows_e,:] = A[rows_e,:] @ B[e];  A [R,Kd], B [E,Kd,N] -> C [R,N]."""
    lib = _lib.load()
    _chk(A, "A")
    _chk(B, "B", A.dtype)
    _chk(offsets, "offsets", torch.int32)
    E, Kd, N = B.shape
    R = int(n_rows if n_rows is not None else (a_row_map.numel() if a_row_map is not None else A.shape[0]))
    C = torch.empty((R, N), dtype=A.dtype, device=A.device)
    ws, tile_cfg = _ws_and_cfg(R, E, A.device, tile_cfg, workspace, map_ready)
    rc = lib.amoe_grouped_gemm_nn(
        A.data_ptr(), _ptr(a_row_map), B.data_ptr(), offsets.data_ptr(), C.data_ptr(), _dtype_code(A), R, E, Kd, N,
        ws.data_ptr(), ws.numel(), tile_cfg, _stream()
    )
    _lib.check(rc, "amoe_grouped_gemm_nn")
    return C


def grouped_gemm_nt(A, B, offsets, a_row_map=None, n_rows=None, tile_cfg: int = 0, workspace=None,
                    map_ready: bool = False) -> torch.Tensor:
    """C[rows_e,:] = A[rows_e,:] @ B[e]^T;  A [R,N], B [E,Kd,N] -> C [R,Kd]."""
    lib = _lib.load()
    _chk(A, "A")
    _chk(B, "B", A.dtype)
    _chk(offsets, "offsets", torch.int32)
    E, Kd, N = B.shape
    R = int(n_rows if n_rows is not None else (a_row_map.numel() if a_row_map is not None else A.shape[0]))
    C = torch.empty((R, Kd), dtype=A.dtype, device=A.device)
    ws, tile_cfg = _ws_and_cfg(R, E, A.device, tile_cfg, workspace, map_ready)
    rc = lib.amoe_grouped_gemm_nt(
        A.data_ptr(), _ptr(a_row_map), B.data_ptr(), offsets.data_ptr(), C.data_ptr(), _dtype_code(A), R, E, Kd, N,
        ws.data_ptr(), ws.numel(), tile_cfg, _stream()
    )
    _lib.check(rc, "amoe_grouped_gemm_nt")
    return C


def grouped_gemm_nt_gated_bwd(dy, w_down, offsets, gate_up, act: int = ACT_SILU, row_scale=None, a_row_map=None,
                              n_rows=None, want_score_parts: bool = True, tile_cfg: int = 0, workspace=None,
                              map_ready: bool = False):
    """d_gate_up [R,2I] and score partials [n_parts,R] f32 (None unless wanted) from dy rows [.,H]
    (gathered through a_row_map), w_down [E,I,H] and the forward's gate_up [R,2I]: the data gradient
    of the down projection with the gated-activation backward as its epilogue (bfloat16 or float16)."""
    lib = _lib.load()
    if dy.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("grouped_gemm_nt_gated_bwd: bfloat16 or float16 operands only")
    _chk(dy, "dy")
    _chk(w_down, "w_down", dy.dtype)
    _chk(gate_up, "gate_up", dy.dtype)
    _chk(offsets, "offsets", torch.int32)
    if a_row_map is not None:
        _chk(a_row_map, "a_row_map", torch.int32)
    if row_scale is not None:
        _chk(row_scale, "row_scale", torch.float32)
    E, I, H = w_down.shape
    R = int(n_rows if n_rows is not None else (a_row_map.numel() if a_row_map is not None else dy.shape[0]))
    if gate_up.shape != (R, 2 * I):
        raise RuntimeError(f"gate_up must be [{R}, {2 * I}], got {tuple(gate_up.shape)}")
    d_gate_up = torch.empty_like(gate_up)
    parts = None
    if want_score_parts:
        parts = torch.empty((lib.amoe_gated_bwd_score_parts(I, tile_cfg), R), dtype=torch.float32, device=dy.device)
    ws, tile_cfg = _ws_and_cfg(R, E, dy.device, tile_cfg, workspace, map_ready)
    rc = lib.amoe_grouped_gemm_nt_gated_bwd(
        dy.data_ptr(), _ptr(a_row_map), w_down.data_ptr(), offsets.data_ptr(), gate_up.data_ptr(), _ptr(row_scale),
        d_gate_up.data_ptr(), _ptr(parts), _dtype_code(dy), R, E, I, H, act, ws.data_ptr(), ws.numel(), tile_cfg, _stream()
    )
    _lib.check(rc, "amoe_grouped_gemm_nt_gated_bwd")
    return d_gate_up, parts


def score_grad_gather(parts: torch.Tensor, row_of: torch.Tensor) -> torch.Tensor:
    """d_scores [T,K] f32 = sum over the partials [n_parts, T*K] of the entry at row_of[t,k]."""
    lib = _lib.load()
    _chk(parts, "parts", torch.float32)
    _chk(row_of, "row_of", torch.int32)
    T, K = row_of.shape
    if parts.dim() != 2 or parts.shape[1] != T * K:
        raise RuntimeError(f"parts must be [n_parts, {T * K}], got {tuple(parts.shape)}")
    d_scores = torch.empty((T, K), dtype=torch.float32, device=parts.device)
    rc = lib.amoe_score_grad_gather(parts.data_ptr(), parts.shape[0], row_of.data_ptr(), d_scores.data_ptr(), T, K, _stream())
    _lib.check(rc, "amoe_score_grad_gather")
    return d_scores


def grouped_gemm_wgrad(A, B, offsets, num_experts: int, tile_cfg: int = 0, a_row_map=None, b_row_map=None) -> torch.Tensor:
    """C[e] = A[rows_e,:]^T @ B[rows_e,:];  A [R,Kd], B [R,N] -> C [E,Kd,N].  With a_row_map [R] (or
    b_row_map [R]) the rows of A (or B) are gathered from a smaller matrix inside the kernel."""
    lib = _lib.load()
    _chk(A, "A")
    _chk(B, "B", A.dtype)
    _chk(offsets, "offsets", torch.int32)
    if a_row_map is not None:
        _chk(a_row_map, "a_row_map", torch.int32)
    if b_row_map is not None:
        _chk(b_row_map, "b_row_map", torch.int32)
    R = a_row_map.numel() if a_row_map is not None else A.shape[0]
    if b_row_map is None and a_row_map is not None and B.shape[0] != R:
        raise RuntimeError("B must have one row per routed row")
    Kd = A.shape[1]
    N = B.shape[1]
    C = torch.empty((num_experts, Kd, N), dtype=A.dtype, device=A.device)
    rc = lib.amoe_grouped_gemm_wgrad(
        A.data_ptr(), _ptr(a_row_map), B.data_ptr(), _ptr(b_row_map), offsets.data_ptr(), C.data_ptr(), _dtype_code(A), R,
        num_experts, Kd, N, tile_cfg, _stream()
    )
    _lib.check(rc, "amoe_grouped_gemm_wgrad")
    return C


def gated_act_bwd(
    gate_up: torch.Tensor,
    d_inter: torch.Tensor,
    act: int = ACT_SILU,
    row_scale: Optional[torch.Tensor] = None,
    slot_of: Optional[torch.Tensor] = None,
    tk: Optional[Tuple[int, int]] = None,
):
    """d_gate_up [R,2I]; with row_scale [R], slot_of [R] and tk=(T,K) also d_row_scale [T,K] f32."""
    lib = _lib.load()
    _chk(gate_up, "gate_up")
    _chk(d_inter, "d_inter", gate_up.dtype)
    R, I = d_inter.shape
    d_gu = torch.empty_like(gate_up)
    d_scale = None
    T = K = 0
    if row_scale is not None:
        _chk(row_scale, "row_scale", torch.float32)
    if slot_of is not None:
        _chk(slot_of, "slot_of", torch.int32)
        T, K = tk
        d_scale = torch.empty((T, K), dtype=torch.float32, device=gate_up.device)
    rc = lib.amoe_gated_act_bwd(
        gate_up.data_ptr(), d_inter.data_ptr(), _ptr(row_scale), _ptr(slot_of), d_gu.data_ptr(), _ptr(d_scale),
        _dtype_code(gate_up), R, I, T, K, act, _stream()
    )
    _lib.check(rc, "amoe_gated_act_bwd")
    return d_gu if slot_of is None else (d_gu, d_scale)


def _expert_view(t: torch.Tensor, name: str):
    """[E, I, H] tensor whose experts may be strided (a slice of a fused tensor) but whose
    [I, H] matrices are dense; returns (E, I, H, expert stride in elements)."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (the HIP kernels have no CPU fallback)")
    if t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2]:
        raise RuntimeError(f"{name} must be [E, I, H] with dense [I, H] matrices, got strides {t.stride()}")
    return t.shape[0], t.shape[1], t.shape[2], (t.stride(0) if t.shape[0] > 1 else t.shape[1] * t.shape[2])


def remap_pack(in0: torch.Tensor, in1: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[e][h][G*i+g] = in_g[e][i][h]: gate/up nn.Linear weights [E,I,H] -> interleaved
    expert_gate_up [E,H,2I] (in1 given), or a batched transpose [E,I,H] -> [E,H,I] (in1 None)."""
    lib = _lib.load()
    E, I, H, es = _expert_view(in0, "in0")
    if in1 is not None:
        if _expert_view(in1, "in1") != (E, I, H, es) or in1.dtype != in0.dtype:
            raise RuntimeError("in1 must match in0 in shape, strides and dtype")
    out = torch.empty((E, H, (2 if in1 is not None else 1) * I), dtype=in0.dtype, device=in0.device)
    rc = lib.amoe_remap_pack(in0.data_ptr(), _ptr(in1), out.data_ptr(), _dtype_code(in0), E, I, H, es, _stream())
    _lib.check(rc, "amoe_remap_pack")
    return out


def remap_unpack(joint: torch.Tensor, two: bool, out0: Optional[torch.Tensor] = None, out1: Optional[torch.Tensor] = None):
    """The inverse of remap_pack: joint [E,H,G*I] -> out_g [E,I,H] (G = 2 if `two`).  out0 / out1
    may be given (e.g. the halves of a fused [E,2I,H] tensor); returns out0 or (out0, out1)."""
    lib = _lib.load()
    _chk(joint, "joint")
    E, H, GI = joint.shape
    G = 2 if two else 1
    if GI % G:
        raise RuntimeError("the last dimension of an interleaved gate_up tensor must be even")
    I = GI // G
    if out0 is None:
        out0 = torch.empty((E, I, H), dtype=joint.dtype, device=joint.device)
        out1 = torch.empty((E, I, H), dtype=joint.dtype, device=joint.device) if two else None
    shape = _expert_view(out0, "out0")
    if shape[:3] != (E, I, H) or out0.dtype != joint.dtype:
        raise RuntimeError("out0 must be [E, I, H] of the input's dtype")
    if two and (out1 is None or _expert_view(out1, "out1") != shape or out1.dtype != joint.dtype):
        raise RuntimeError("out1 must match out0")
    rc = lib.amoe_remap_unpack(joint.data_ptr(), out0.data_ptr(), _ptr(out1) if two else None, _dtype_code(joint), E, I, H,
                               shape[3], _stream())
    _lib.check(rc, "amoe_remap_unpack")
    return (out0, out1) if two else out0
