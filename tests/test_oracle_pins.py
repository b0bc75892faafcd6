"""Pins for the CPU oracle: every function of oracle/moe_oracle.py is checked
against something that is not a re-typing of its own formula -- closed forms,
brute force, library routines, invariants, torch.autograd, and the installed
transformers Qwen3-MoE block (third-party code, the same baseline the
reference's own MoE test compares losses with, tests/trainer/test_moe.py:218-223).
"""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def test_softmax_closed_forms():
    # two logits: p0 = sigmoid(a - b)
    a, b = 0.3, -1.1
    p = O.softmax_probs(torch.tensor([[a, b]]))
    assert p.dtype == torch.float32
    assert abs(float(p[0, 0]) - 1 / (1 + math.exp(b - a))) < 1e-7
    # equal logits: uniform
    p = O.softmax_probs(torch.zeros(2, 5, dtype=torch.bfloat16))
    assert p.dtype == torch.float32 and torch.allclose(p, torch.full((2, 5), 0.2))
    # shift invariance and log-ratio
    l = torch.tensor([[1.0, 2.0, 4.0]])
    p = O.softmax_probs(l)
    p2 = O.softmax_probs(l + 7.0)
    assert torch.allclose(p, p2, atol=1e-7)
    assert abs(math.log(float(p[0, 2] / p[0, 0])) - 3.0) < 1e-5
    # the library call the reference itself makes (moe.py:361)
    l = torch.randn(16, 33).to(torch.bfloat16)
    assert torch.equal(O.softmax_probs(l), F.softmax(l, dim=-1, dtype=torch.float32))


def _brute_topk(row, k):
    order = sorted(range(len(row)), key=lambda i: (-row[i], i))
    return order[:k]


def test_topk_brute_force_and_ties():
    g = torch.Generator().manual_seed(1)
    v = torch.rand(64, 9, generator=g)
    _, idx = O.topk_canonical(v, 3)
    for r in range(v.shape[0]):
        assert idx[r].tolist() == _brute_topk(v[r].tolist(), 3)
    # tie-free rows: must equal torch.topk exactly (indices and values)
    tv, ti = torch.topk(v, 3, dim=-1)
    ov, oi = O.topk_canonical(v, 3)
    assert torch.equal(ti, oi) and torch.equal(tv, ov)
    # hand-built ties: lowest index first, also across the k / k+1 boundary
    row = torch.tensor([[0.1, 0.4, 0.4, 0.05, 0.4, 0.1]])
    _, idx = O.topk_canonical(row, 2)
    assert idx.tolist() == [[1, 2]]
    _, idx = O.topk_canonical(row, 4)
    assert idx.tolist() == [[1, 2, 4, 0]]
    # heavily tied random rows (few distinct values)
    q = torch.randint(0, 4, (200, 16), generator=g).float()
    _, idx = O.topk_canonical(q, 8)
    for r in range(q.shape[0]):
        assert idx[r].tolist() == _brute_topk(q[r].tolist(), 8)


def test_normalize_and_cast():
    s = torch.tensor([[0.5, 0.25], [0.1, 0.3]])
    n = O.normalize_and_cast(s, True, torch.float32)
    assert torch.allclose(n, torch.tensor([[2 / 3, 1 / 3], [0.25, 0.75]]))
    assert torch.allclose(n.sum(-1), torch.ones(2))
    assert torch.equal(O.normalize_and_cast(s, False, torch.float32), s)
    assert O.normalize_and_cast(s, True, torch.bfloat16).dtype == torch.bfloat16


def _literal_permutation(idx_tk, E):
    """the reference's own sequence of library calls, moe.py:367-382"""
    T = idx_tk.shape[0]
    flat = idx_tk.t().reshape(-1)
    mask = F.one_hot(flat, num_classes=E).t()
    slots = torch.cat([torch.where(mask[i])[0] for i in range(mask.shape[0])])
    return slots, slots % T, mask.sum(dim=-1)


def test_permutation_worked_example():
    idx = torch.tensor([[1, 0], [0, 1], [1, 0]])
    perm, tok, counts = O.permutation(idx, 2)
    assert perm.tolist() == [1, 3, 5, 0, 2, 4]
    assert tok.tolist() == [1, 0, 2, 0, 2, 1]
    assert counts.tolist() == [3, 3]
    assert (perm // 3).tolist() == [0, 1, 1, 0, 0, 1]
    row_of = O.inverse_row_map(perm, 3, 2)
    assert row_of.tolist() == [[3, 1], [0, 5], [4, 2]]


def test_permutation_exhaustive_small():
    for T in range(1, 5):
        for E in range(1, 4):
            for K in range(1, min(E, 2) + 1):
                choices = list(itertools.permutations(range(E), K))
                for combo in itertools.product(choices, repeat=T):
                    idx = torch.tensor(combo, dtype=torch.int64).view(T, K)
                    perm, tok, counts = O.permutation(idx, E)
                    lp, lt, lc = _literal_permutation(idx, E)
                    assert torch.equal(perm, lp) and torch.equal(tok, lt) and torch.equal(counts, lc)
                    flat = idx.t().reshape(-1).numpy()
                    assert np.array_equal(perm.numpy(), np.argsort(flat, kind="stable"))


def test_permutation_invariants_random():
    g = torch.Generator().manual_seed(5)
    T, E, K = 257, 13, 4
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    perm, tok, counts = O.permutation(idx, E)
    R = T * K
    assert sorted(perm.tolist()) == list(range(R))
    assert int(counts.sum()) == R
    assert torch.equal(tok, perm % T)
    flat = idx.t().reshape(-1)
    offs = [0] + counts.cumsum(0).tolist()
    for e in range(E):
        seg = perm[offs[e] : offs[e + 1]]
        assert bool((flat[seg] == e).all())
        assert bool((seg[1:] > seg[:-1]).all())
    lp, lt, lc = _literal_permutation(idx, E)
    assert torch.equal(perm, lp) and torch.equal(counts, lc)
    row_of = O.inverse_row_map(perm, T, K)
    for t in (0, 7, 256):
        for k in range(K):
            r = int(row_of[t, k])
            assert int(tok[r]) == t and int(perm[r]) == k * T + t


def test_grouped_gemm_and_empty_groups():
    g = torch.Generator().manual_seed(2)
    counts = torch.tensor([3, 0, 5, 0, 1])
    cs = counts.cumsum(0)
    A = torch.randn(9, 6, generator=g, dtype=torch.float64)
    B = torch.randn(5, 6, 4, generator=g, dtype=torch.float64)
    C = O.grouped_gemm(A, B, cs)
    ref = torch.zeros(9, 4, dtype=torch.float64)
    row_expert = [0, 0, 0, 2, 2, 2, 2, 2, 4]
    for r, e in enumerate(row_expert):
        for n in range(4):
            ref[r, n] = sum(float(A[r, k]) * float(B[e, k, n]) for k in range(6))
    assert torch.allclose(C, ref, atol=1e-12)
    # every group empty but the last
    cs = torch.tensor([0, 0, 9])
    C = O.grouped_gemm(A, B[:3], cs)
    assert torch.allclose(C, A @ B[2], atol=1e-12)


def test_expert_ffn_interleave_and_silu():
    g = torch.Generator().manual_seed(3)
    R, H, I, E = 7, 5, 3, 2
    cs = torch.tensor([4, 7])
    xp = torch.randn(R, H, generator=g, dtype=torch.float64)
    w_gate = torch.randn(E, H, I, generator=g, dtype=torch.float64)
    w_up = torch.randn(E, H, I, generator=g, dtype=torch.float64)
    wd = torch.randn(E, I, H, generator=g, dtype=torch.float64)
    # layout contract of utils.py:249-263: stack on a new last axis then flatten
    wgu = torch.stack((w_gate, w_up), dim=-1).view(E, H, 2 * I)
    gu, inter, out = O.expert_ffn(xp, wgu, wd, cs, "silu")
    for r in range(R):
        e = 0 if r < 4 else 1
        gt = xp[r] @ w_gate[e]
        up = xp[r] @ w_up[e]
        silu = gt / (1 + torch.exp(-gt))
        assert torch.allclose(inter[r], up * silu, atol=1e-12)
        assert torch.allclose(out[r], (up * silu) @ wd[e], atol=1e-12)
        assert torch.allclose(gu[r, 0::2], gt, atol=1e-12) and torch.allclose(gu[r, 1::2], up, atol=1e-12)


def test_combine_dense():
    g = torch.Generator().manual_seed(4)
    T, K, E, H = 6, 2, 4, 3
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    perm, tok, counts = O.permutation(idx, E)
    s_tk = torch.rand(T, K, generator=g, dtype=torch.float64)
    s_perm = s_tk.t().reshape(-1)[perm]
    out = torch.randn(T * K, H, generator=g, dtype=torch.float64)
    y = O.combine(out, tok, s_perm, K)
    row_of = O.inverse_row_map(perm, T, K)
    for t in range(T):
        ref = sum(s_tk[t, k] * out[row_of[t, k]] for k in range(K))
        assert torch.allclose(y[t], ref, atol=1e-12)


def _tiny(dtype=torch.float64, T=6, H=5, E=4, K=2, I=3, seed=0, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=dtype)
    wr = torch.randn(E, H, generator=g, dtype=dtype) * scale
    wgu = torch.randn(E, H, 2 * I, generator=g, dtype=dtype) * scale
    wd = torch.randn(E, I, H, generator=g, dtype=dtype) * scale
    dy = torch.randn(T, H, generator=g, dtype=dtype)
    cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.01)
    return x, wr, wgu, wd, dy, cfg


def test_gradcheck_fp64():
    x, wr, wgu, wd, dy, cfg = _tiny()
    cfg.loss_coeff = 0.0  # the hook is not the derivative of the forward value
    sel = O.router_linear(x, wr).detach()  # freeze the routing decisions

    def fn(x_, wr_, wgu_, wd_):
        return O.forward(x_, wr_, wgu_, wd_, cfg, logits_for_selection=sel)["y"]

    leaves = [t.clone().requires_grad_(True) for t in (x, wr, wgu, wd)]
    assert torch.autograd.gradcheck(fn, leaves, eps=1e-6, atol=1e-5)


@pytest.mark.parametrize("normalize", [True, False])
def test_analytic_backward_matches_autograd(normalize):
    x, wr, wgu, wd, dy, cfg = _tiny(T=9, H=6, E=5, K=3, I=4, seed=11)
    cfg.normalize_topk_scores = normalize
    cfg.loss_coeff = 0.37
    res = O.forward_backward(x, wr, wgu, wd, dy, cfg)
    ana = O.analytic_backward(res, x, wr, wgu, wd, dy, cfg)
    for k in ("dx", "d_router_gate", "d_expert_gate_up", "d_expert_down"):
        assert torch.allclose(ana[k], res[k], atol=1e-10), k


def test_load_balance_hook_closed_form():
    """moe.py:393-406: the hook adds d/dprobs of coeff * sum_e freq_e * mean_t probs[t,e]
    with freq detached, i.e. coeff * freq_e / T on every row."""
    x, wr, wgu, wd, dy, cfg = _tiny(T=8, E=4, K=2, seed=21)
    cfg.loss_coeff = 0.5
    res1 = O.forward_backward(x, wr, wgu, wd, dy, cfg)
    cfg0 = O.OracleConfig(**{**cfg.__dict__, "loss_coeff": 0.0})
    res0 = O.forward_backward(x, wr, wgu, wd, dy, cfg0)
    # explicit auxiliary loss differentiated by autograd
    wr_ = wr.clone().requires_grad_(True)
    x_ = x.clone().requires_grad_(True)
    probs = F.softmax(F.linear(x_, wr_), dim=-1)
    freq = res1["counts"].to(torch.float64) / res1["counts"].sum()
    aux = 0.5 * (freq * probs.mean(0)).sum()
    aux.backward()
    assert torch.allclose(res1["d_router_gate"] - res0["d_router_gate"], wr_.grad, atol=1e-12)
    assert torch.allclose(res1["dx"] - res0["dx"], x_.grad, atol=1e-12)
    assert torch.allclose(res1["d_expert_down"], res0["d_expert_down"])


def _hf_block(T, H, E, K, I, norm, seed):
    from transformers import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

    c = Qwen3MoeConfig(
        hidden_size=H,
        moe_intermediate_size=I,
        intermediate_size=I,
        num_experts=E,
        num_experts_per_tok=K,
        norm_topk_prob=norm,
        hidden_act="silu",
        num_hidden_layers=1,
        num_attention_heads=1,
        num_key_value_heads=1,
        vocab_size=8,
    )
    blk = Qwen3MoeSparseMoeBlock(c).to(torch.float64)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        blk.gate.weight.copy_(torch.randn(E, H, generator=g, dtype=torch.float64) * 0.5)
        blk.experts.gate_up_proj.copy_(torch.randn(E, 2 * I, H, generator=g, dtype=torch.float64) * 0.3)
        blk.experts.down_proj.copy_(torch.randn(E, H, I, generator=g, dtype=torch.float64) * 0.3)
    return blk


@pytest.mark.parametrize("norm", [True, False])
def test_whole_layer_against_hf_block(norm):
    T, H, E, K, I = 24, 16, 6, 2, 12
    blk = _hf_block(T, H, E, K, I, norm, seed=7)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, T // 2, H, generator=g, dtype=torch.float64)
    dy = torch.randn(2, T // 2, H, generator=g, dtype=torch.float64)
    xh = x.clone().requires_grad_(True)
    yh = blk(xh)
    yh.backward(dy)
    # HF layout -> reference layout (utils.py:249-266): gate rows then up rows,
    # each [I, H], become interleaved columns of [H, 2I]; down [H, I] -> [I, H]
    gu = blk.experts.gate_up_proj.detach()
    w_gate, w_up = gu[:, :I, :].transpose(1, 2), gu[:, I:, :].transpose(1, 2)
    wgu = torch.stack((w_gate, w_up), dim=-1).reshape(E, H, 2 * I).contiguous()
    wd = blk.experts.down_proj.detach().transpose(1, 2).contiguous()
    wr = blk.gate.weight.detach()
    cfg = O.OracleConfig(
        model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, normalize_topk_scores=norm, loss_coeff=0.0
    )
    res = O.forward_backward(x, wr, wgu, wd, dy, cfg)
    # HF evaluates its softmax in float32 even for float64 inputs, so anything
    # downstream of the probabilities agrees to float32 rounding only
    assert torch.allclose(res["y"], yh.detach(), atol=5e-6)
    assert torch.allclose(res["dx"], xh.grad, atol=5e-6)
    assert torch.allclose(res["d_router_gate"], blk.gate.weight.grad, atol=5e-6)
    dgu_h = blk.experts.gate_up_proj.grad
    dgu = res["d_expert_gate_up"]
    assert torch.allclose(dgu[:, :, 0::2], dgu_h[:, :I, :].transpose(1, 2), atol=5e-6)
    assert torch.allclose(dgu[:, :, 1::2], dgu_h[:, I:, :].transpose(1, 2), atol=5e-6)
    assert torch.allclose(res["d_expert_down"], blk.experts.down_proj.grad.transpose(1, 2), atol=5e-6)
    ana = O.analytic_backward(res, x.reshape(-1, H), wr, wgu, wd, dy.reshape(-1, H), cfg)
    assert torch.allclose(ana["d_expert_gate_up"], dgu, atol=1e-12)


def test_shared_expert_closed_form():
    """H = I = 1: (x*wu) * silu(x*wg) * wd * sigmoid(x*wo), written out with math.exp."""
    import math

    x, wg, wu, wd, wo = 0.7, -1.3, 0.9, 1.7, 0.4
    got = O.shared_expert(
        torch.tensor([[x]], dtype=torch.float64),
        torch.tensor([[wg, wu]], dtype=torch.float64),  # gate in the even, up in the odd column
        torch.tensor([[wd]], dtype=torch.float64),
        torch.tensor([[wo]], dtype=torch.float64),
        "silu",
    )
    g = x * wg
    want = (x * wu) * (g / (1 + math.exp(-g))) * wd / (1 + math.exp(-x * wo))
    assert abs(float(got) - want) < 1e-15
    # swapping the two interleaved columns must change the result (gate and up are not symmetric)
    swapped = O.shared_expert(
        torch.tensor([[x]], dtype=torch.float64), torch.tensor([[wu, wg]], dtype=torch.float64),
        torch.tensor([[wd]], dtype=torch.float64), torch.tensor([[wo]], dtype=torch.float64), "silu",
    )
    assert abs(float(swapped) - want) > 1e-3


def test_layer_without_gate_closed_form():
    """is_gated=False (moe.py:101-106, 188-191, 306-311): the layer is linear in x between the
    router and the combine.  Checked against a token-major dense evaluation that shares only the
    routing decision (indices and scores) with the oracle:
    y[t] = sum_k s[t,k] * (x[t] @ W_up[e] @ W_down[e]) + (x[t] @ S_up @ S_down) * sigmoid(x[t] @ s_o).
    A stray activation, a de-interleave of the [E,H,I] projection or a missing score would fail it."""
    T, H, E, K, I = 23, 12, 5, 2, 7
    g = torch.Generator().manual_seed(5)
    x, wr = torch.randn(T, H, generator=g, dtype=torch.float64), torch.randn(E, H, generator=g, dtype=torch.float64)
    wup = torch.randn(E, H, I, generator=g, dtype=torch.float64)
    wd = torch.randn(E, I, H, generator=g, dtype=torch.float64)
    sh = (torch.randn(H, I, generator=g, dtype=torch.float64), torch.randn(I, H, generator=g, dtype=torch.float64),
          torch.randn(H, 1, generator=g, dtype=torch.float64))
    cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, is_gated=False)
    for shared in (None, sh):
        res = O.forward(x, wr, wup, wd, cfg, shared=shared)
        probs = torch.softmax(x @ wr.t(), dim=-1)
        s, idx = probs.topk(K, dim=-1)
        s = s / s.sum(-1, keepdim=True)
        want = torch.zeros(T, H, dtype=torch.float64)
        for t in range(T):
            for k in range(K):
                e = int(idx[t, k])
                want[t] += s[t, k] * (x[t] @ wup[e] @ wd[e])
            if shared is not None:
                want[t] += (x[t] @ sh[0] @ sh[1]) * torch.sigmoid(x[t] @ sh[2])
        assert torch.allclose(res["y"], want, atol=1e-12)
        assert res["inter"].shape == (T * K, I) and torch.equal(res["inter"], res["gate_up"])
    # the gated layer on the same shapes is a different function (the activation is really absent above)
    gated = O.forward(x, wr, torch.cat((wup, wup), dim=-1), wd, O.OracleConfig(H, I, E, K))
    assert not torch.allclose(gated["y"], O.forward(x, wr, wup, wd, cfg)["y"], atol=1e-3)


def test_whole_layer_with_shared_expert_against_hf_block():
    """The installed transformers Qwen2-MoE block = routed experts + shared MLP times a sigmoid
    gate (the block the reference's shared-expert parameters are filled from, utils.py:268-289)."""
    from transformers import Qwen2MoeConfig
    from transformers.models.qwen2_moe.modeling_qwen2_moe import Qwen2MoeSparseMoeBlock

    T, H, E, K, I = 24, 16, 6, 2, 12
    c = Qwen2MoeConfig(
        hidden_size=H, moe_intermediate_size=I, shared_expert_intermediate_size=I, intermediate_size=I, num_experts=E,
        num_experts_per_tok=K, norm_topk_prob=True, hidden_act="silu", num_hidden_layers=1, num_attention_heads=1,
        num_key_value_heads=1, vocab_size=8,
    )
    blk = Qwen2MoeSparseMoeBlock(c).to(torch.float64)
    g = torch.Generator().manual_seed(21)
    with torch.no_grad():
        blk.gate.weight.copy_(torch.randn(E, H, generator=g, dtype=torch.float64) * 0.5)
        blk.experts.gate_up_proj.copy_(torch.randn(E, 2 * I, H, generator=g, dtype=torch.float64) * 0.3)
        blk.experts.down_proj.copy_(torch.randn(E, H, I, generator=g, dtype=torch.float64) * 0.3)
        for lin in (blk.shared_expert.gate_proj, blk.shared_expert.up_proj, blk.shared_expert.down_proj, blk.shared_expert_gate):
            lin.weight.copy_(torch.randn(lin.weight.shape, generator=g, dtype=torch.float64) * 0.3)
    x = torch.randn(2, T // 2, H, generator=g, dtype=torch.float64)
    dy = torch.randn(2, T // 2, H, generator=g, dtype=torch.float64)
    xh = x.clone().requires_grad_(True)
    yh = blk(xh)
    yh.backward(dy)

    gu = blk.experts.gate_up_proj.detach()
    wgu = torch.stack((gu[:, :I, :].transpose(1, 2), gu[:, I:, :].transpose(1, 2)), dim=-1).reshape(E, H, 2 * I).contiguous()
    wd = blk.experts.down_proj.detach().transpose(1, 2).contiguous()
    sh = blk.shared_expert
    # utils.py:272-289: nn.Linear weights transposed; gate / up interleaved on the last dimension
    s_gu = torch.stack((sh.gate_proj.weight.detach().T, sh.up_proj.weight.detach().T), dim=-1).reshape(H, 2 * I).contiguous()
    s_d = sh.down_proj.weight.detach().T.contiguous()
    s_og = blk.shared_expert_gate.weight.detach().T.contiguous()
    cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, normalize_topk_scores=True, loss_coeff=0.0)
    res = O.forward_backward(x, blk.gate.weight.detach(), wgu, wd, dy, cfg, shared=(s_gu, s_d, s_og))
    # HF evaluates the router softmax in float32: agreement to float32 rounding downstream of it
    assert torch.allclose(res["y"], yh.detach(), atol=5e-6)
    assert torch.allclose(res["dx"], xh.grad, atol=5e-6)
    assert torch.allclose(res["d_shared_expert_gate_up"][:, 0::2], sh.gate_proj.weight.grad.T, atol=1e-12)
    assert torch.allclose(res["d_shared_expert_gate_up"][:, 1::2], sh.up_proj.weight.grad.T, atol=1e-12)
    assert torch.allclose(res["d_shared_expert_down"], sh.down_proj.weight.grad.T, atol=1e-12)
    assert torch.allclose(res["d_shared_expert_output_gate"], blk.shared_expert_gate.weight.grad.T, atol=1e-12)
    # the shared expert's share of y is what is left when the routed layer is taken away
    routed = O.forward(x, blk.gate.weight.detach(), wgu, wd, cfg)
    assert torch.allclose(
        res["y"].detach() - routed["y"], O.shared_expert(x.reshape(-1, H), s_gu, s_d, s_og, "silu").reshape(x.shape), atol=1e-12
    )


def test_reference_rounding_mode_close_to_exact():
    """bf16 with the reference's per-op rounding stays within the bf16 bar of
    the exact evaluation from the same rounded inputs."""
    x, wr, wgu, wd, dy = O.make_inputs(64, 32, 8, 2, 48, torch.bfloat16, seed=3)
    cfg = O.OracleConfig(model_dim=32, intermediate_dim=48, num_experts=8, top_k=2, loss_coeff=0.001)
    ref = O.forward_backward(x, wr, wgu, wd, dy, cfg)
    sel = ref["logits"].detach()
    ex = O.forward_backward(x, wr, wgu, wd, dy, cfg, compute_dtype=torch.float64, logits_for_selection=sel)
    assert torch.equal(ref["topk_idx"], ex["topk_idx"])
    assert O.rel_l2(ref["y"], ex["y"]) < 1e-2
    for k in ("dx", "d_expert_gate_up", "d_expert_down"):
        assert O.rel_l2(ref[k], ex[k]) < 2e-2, k


def test_selection_on_logits_equals_selection_on_probs():
    x, wr, *_ = O.make_inputs(512, 64, 32, 4, 8, torch.bfloat16, seed=9)
    logits = O.router_linear(x, wr)
    assert O.selection_agrees(logits, 4)
    # a row made entirely of ties still agrees (index order)
    assert O.selection_agrees(torch.zeros(3, 8, dtype=torch.bfloat16), 4)
