"""The BASELINE configurations at their FULL sizes.

The float64 oracle cannot evaluate 3.7-17 TFLOP layers in seconds, so at full size the layer is
checked through what does not grow with the size:
  * routing -- top-k indices, counts, permutation maps -- bit-exact against the oracle on ALL
    tokens (integer work, cheap on the CPU);
  * y and dx of a handful of sampled tokens against the oracle run on just those tokens (with
    loss_coeff = 0 a token's output and input gradient depend on no other token);
  * sampled rows / columns of the expert weight gradients against their definition (the stage
    formulas of the backward: dW_down[e][i,:] = sum_r inter_s[r,i] dy[tok_r,:], dW_gate_up[e][:,c]
    = sum_r x[tok_r,:] d_gate_up[r,c]) evaluated in float64 over exactly the rows of that expert.
C4 has no router: its grouped GEMMs are checked on sampled rows and elements the same way.
C3 and C5 are additionally checked in FULL (test_full_size_every_row_and_expert): every row of y and
dx, every expert of both weight gradients, against the reference's formulas in float32 on the device.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O
from test_gpu_layer import build_layer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(gpu_device):
    from arctictraining_amd import ops as _ops

    return _ops


TOL = 1e-2  # rel-L2, bf16

# name: (T, H, E, K, I, bias_hot, n_hot, n_dead, oracle compute dtype)
FULL = {
    "c3_qwen3_30b": (16384, 2048, 128, 8, 768, None, 0, 0, torch.float64),
    "c5_stress": (32768, 2048, 64, 4, 1408, 1.6, 4, 8, torch.float64),
    "c2_mixtral": (8192, 4096, 8, 2, 14336, None, 0, 0, torch.float32),
}


def device_inputs(T, H, E, I, dev, seed, bias_hot=None, n_hot=0, n_dead=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    bf = torch.bfloat16
    x = torch.randn(T, H, device=dev, generator=g)
    wr = torch.randn(E, H, device=dev, generator=g) * 0.02
    if n_hot or n_dead:
        x[:, H - 1] = 1.0
        wr[:, H - 1] = 0.0
        wr[:n_hot, H - 1] = float(bias_hot)
        wr[E - n_dead:, H - 1] = -1.0e4
    x, wr = x.to(bf), wr.to(bf)
    wgu = torch.empty(E, H, 2 * I, device=dev, dtype=bf)
    wd = torch.empty(E, I, H, device=dev, dtype=bf)
    for e in range(E):  # expert by expert: no float32 copy of the whole weight
        wgu[e] = (torch.randn(H, 2 * I, device=dev, generator=g) * 0.02).to(bf)
        wd[e] = (torch.randn(I, H, device=dev, generator=g) * 0.02).to(bf)
    dy = torch.randn(T, H, device=dev, generator=g).to(bf)
    return x, wr, wgu, wd, dy


def bf16_round(t):
    return t.to(torch.bfloat16).to(t.dtype)


@pytest.mark.parametrize("name", list(FULL))
def test_full_size_layer(gpu_device, name):
    T, H, E, K, I, bias_hot, n_hot, n_dead, odt = FULL[name]
    print("full-size layer", name, flush=True)
    dev = gpu_device
    x, wr, wgu, wd, dy = device_inputs(T, H, E, I, dev, 4242, bias_hot, n_hot, n_dead)
    layer = build_layer(torch.bfloat16, H, E, K, I, dev, loss_coeff=0.0)
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    layer.capture = {}
    xg = x.clone().requires_grad_(True)
    y = layer(xg)
    y.backward(dy)
    torch.cuda.synchronize()
    cap = layer.capture

    # ---- routing, all tokens, bit-exact
    logits = cap["logits"].float().cpu()
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.0)
    g = O.gate(logits, ocfg, torch.bfloat16, select_values=logits)
    assert torch.equal(cap["topk_idx"].cpu().long(), g["topk_idx"]), "top-k indices"
    assert torch.equal(cap["counts"].cpu().long(), g["counts"]), "counts"
    assert torch.equal(cap["slot_of"].cpu().long(), g["perm"]), "permutation"
    assert torch.equal(cap["token_of"].cpu().long(), g["token_ids"]), "token ids"
    assert torch.equal(cap["row_of"].cpu().long(), O.inverse_row_map(g["perm"], T, K)), "inverse map"
    # scores are floating point: equal up to one rounding step of the model dtype (2^-8 relative)
    s_got, s_ref = cap["scores"].cpu().double(), g["scores_tk"].double()
    assert float(((s_got - s_ref).abs() / s_ref).max()) <= 2.0 ** -7, "scores"
    assert float((s_got != s_ref).double().mean()) < 0.01, "scores differ in more than 1% of the slots"
    if n_dead:
        assert int((g["counts"][-n_dead:] == 0).sum()) == n_dead
        assert 0.35 < float(g["counts"][:n_hot].sum()) / float(g["counts"].sum()) < 0.65
        assert bool((layer.expert_down.grad[-n_dead:] == 0).all()) and bool((layer.expert_gate_up.grad[-n_dead:] == 0).all())

    # ---- sampled tokens against the oracle run on those tokens only
    rng = np.random.default_rng(7)
    S = torch.from_numpy(np.sort(rng.choice(T, size=16, replace=False)))
    xs, dys = x[S.to(dev)].cpu(), dy[S.to(dev)].cpu()
    ref = O.forward_backward(xs, wr.cpu(), wgu.cpu(), wd.cpu(), dys, ocfg, compute_dtype=odt,
                             logits_for_selection=logits[S])
    assert torch.equal(ref["topk_idx"], g["topk_idx"][S])
    e_y = O.rel_l2(y.detach()[S.to(dev)].cpu(), ref["y"])
    e_dx = O.rel_l2(xg.grad[S.to(dev)].cpu(), ref["dx"])
    print(f"  sampled tokens: y {e_y:.2e} dx {e_dx:.2e}", flush=True)
    assert e_y <= TOL and e_dx <= TOL
    del ref

    # ---- sampled rows / columns of the expert weight gradients against their definition
    act, dact = O.activation("silu"), O.silu_grad
    offsets = cap["offsets"].long()
    token_of = cap["token_of"].long()
    s_perm = cap["scores"].t().reshape(-1)[cap["slot_of"].long()].double()
    counts = g["counts"]
    live = [int(e) for e in torch.nonzero(counts > 0).flatten()]
    experts = [live[0], live[len(live) // 2], live[-1]]
    for e in experts:
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        tok = token_of[r0:r1]
        Xe, DYe, se = x[tok].double(), dy[tok].double(), s_perm[r0:r1]
        for i in (0, I // 2 + 1, I - 1):
            gu = bf16_round(Xe @ wgu[e][:, 2 * i:2 * i + 2].double())           # stored in the model dtype
            gate, up = gu[:, 0], gu[:, 1]
            inter_s = bf16_round(se * up * act(gate))
            ref_row = inter_s @ DYe                                            # dW_down[e][i, :]
            err = O.rel_l2(layer.expert_down.grad[e, i].double(), ref_row)
            assert err <= TOL, f"dW_down[{e}][{i}]: {err:.3e}"
            d_inter = bf16_round(DYe @ wd[e][i].double())
            d_gate = bf16_round(se * d_inter * up * dact(gate))
            d_up = bf16_round(se * d_inter * act(gate))
            for c, dcol in ((2 * i, d_gate), (2 * i + 1, d_up)):
                ref_col = Xe.t() @ dcol                                        # dW_gate_up[e][:, c]
                err = O.rel_l2(layer.expert_gate_up.grad[e, :, c].double(), ref_col)
                assert err <= TOL, f"dW_gate_up[{e}][:, {c}]: {err:.3e}"


@pytest.mark.parametrize("name", ["c3_qwen3_30b", "c5_stress"])
def test_full_size_router_gradient(gpu_device, name):
    """The router's gradient path at full size with the load-balance term switched on
    (loss_coeff = 0.001): the score gradients of sampled tokens against their definition, the
    router backward kernel against the oracle's formula on ALL tokens, and d_router_gate (the
    16-way split of the token dimension on the weight-gradient kernel) against d_logits^T x in
    float64."""
    T, H, E, K, I, bias_hot, n_hot, n_dead, _ = FULL[name]
    print("full-size router gradient", name, flush=True)
    dev = gpu_device
    x, wr, wgu, wd, dy = device_inputs(T, H, E, I, dev, 777, bias_hot, n_hot, n_dead)
    layer = build_layer(torch.bfloat16, H, E, K, I, dev, loss_coeff=0.001)
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    layer.capture = {}
    xg = x.clone().requires_grad_(True)
    layer(xg).backward(dy)
    torch.cuda.synchronize()
    cap = layer.capture
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)

    # (a) score gradients of sampled tokens: d_s[t,k] = <dy[t], (up * act(gate)) @ W_down[e]>
    act = O.activation("silu")
    rng = np.random.default_rng(11)
    topk = cap["topk_idx"].long()
    S = np.sort(rng.choice(T, size=12, replace=False))
    ref_ds = torch.zeros(len(S), K, dtype=torch.float64, device=dev)
    for a, t in enumerate(S):
        for k in range(K):
            e = int(topk[t, k])
            gu = bf16_round(x[t].double() @ wgu[e].double())
            out = (gu[1::2] * act(gu[0::2])) @ wd[e].double()
            ref_ds[a, k] = (dy[t].double() * out).sum()
    err = O.rel_l2(cap["d_scores"][torch.from_numpy(S).to(dev)].cpu(), ref_ds.cpu())
    print(f"  d_scores (sampled tokens): {err:.2e}", flush=True)
    assert err <= TOL

    # (b) router backward on all tokens from the captured score gradients
    counts = cap["counts"].cpu().long()
    freq = counts.double() / counts.sum().double()
    _, ref_dl = O.router_backward(cap["d_scores"].cpu().double(), cap["probs"].cpu().double(), topk.cpu(), freq, ocfg, T)
    err = O.rel_l2(cap["d_logits"].cpu(), ref_dl)
    print(f"  d_logits (all tokens): {err:.2e}", flush=True)
    assert err <= TOL
    # (At this size the load-balance term, loss_coeff / T per entry and nearly uniform over the
    # experts, lies below the float32 rounding of the softmax backward it is added into -- in the
    # reference too; that it is applied is checked where it is visible, in
    # test_layer_load_balance_term and test_router_bwd.)

    # (c) d_router_gate = d_logits^T @ x, float64 on the device from the captured (bf16) d_logits
    ref_wr = cap["d_logits"].double().t() @ x.double()
    err = O.rel_l2(layer.router_gate.grad.cpu(), ref_wr.cpu())
    print(f"  d_router_gate: {err:.2e}", flush=True)
    assert err <= TOL


def _device_reference(x, wr, wgu, wd, dy, cap, K):
    """The default path of the reference (moe.py:54-60 grouped product as a per-expert matmul loop,
    :176-193 gated FFN, :340-357 gather, :450-461 combine) and the stage formulas of its backward, in
    float32 torch ops on the device, over the routing the layer captured (the routing itself is
    compared bit for bit elsewhere).  Intermediates the reference stores in the model dtype are
    rounded to it.  Returns y, the expert part of dx, both weight gradients and the score gradients."""
    bf = torch.bfloat16
    T, H = x.shape
    E, _, I2 = wgu.shape
    tok = cap["token_of"].long()
    offs = cap["offsets"].cpu().tolist()
    s_perm = cap["scores"].t().reshape(-1)[cap["slot_of"].long()].float()     # k-major flatten, row order
    xp = x[tok].float()
    R = tok.numel()
    gate_up = torch.empty(R, I2, device=x.device, dtype=bf)
    for e in range(E):
        if offs[e + 1] > offs[e]:
            gate_up[offs[e]:offs[e + 1]] = (xp[offs[e]:offs[e + 1]] @ wgu[e].float()).to(bf)
    gate, up = gate_up[:, 0::2].float(), gate_up[:, 1::2].float()
    inter = (up * F.silu(gate)).to(bf)
    out = torch.empty(R, H, device=x.device, dtype=bf)
    for e in range(E):
        if offs[e + 1] > offs[e]:
            out[offs[e]:offs[e + 1]] = (inter[offs[e]:offs[e + 1]].float() @ wd[e].float()).to(bf)
    y = torch.zeros(T, H, device=x.device).index_add_(0, tok, out.float() * s_perm[:, None])
    # backward
    dyp = dy[tok].float()
    d_s = (dyp * out.float()).sum(1)                                          # [R], row order
    d_out = dyp * s_perm[:, None]
    del dyp
    d_wd = torch.zeros(E, wd.shape[1], H, device=x.device)
    d_inter = torch.empty(R, wd.shape[1], device=x.device)
    for e in range(E):
        if offs[e + 1] > offs[e]:
            sl = slice(offs[e], offs[e + 1])
            d_inter[sl] = d_out[sl] @ wd[e].float().t()
            d_wd[e] = inter[sl].float().t() @ d_out[sl]
    del d_out
    sg = torch.sigmoid(gate)
    d_gu = torch.empty(R, I2, device=x.device)
    d_gu[:, 0::2] = d_inter * up * (sg * (1 + gate * (1 - sg)))
    d_gu[:, 1::2] = d_inter * (gate * sg)
    d_gu = d_gu.to(bf).float()                                                # stored in the model dtype
    del d_inter, sg
    d_wgu = torch.zeros(E, H, I2, device=x.device)
    d_xp = torch.empty(R, H, device=x.device)
    for e in range(E):
        if offs[e + 1] > offs[e]:
            sl = slice(offs[e], offs[e + 1])
            d_xp[sl] = d_gu[sl] @ wgu[e].float().t()
            d_wgu[e] = xp[sl].t() @ d_gu[sl]
    dx_experts = torch.zeros(T, H, device=x.device).index_add_(0, tok, d_xp.to(bf).float())
    d_scores = torch.zeros(T * K, device=x.device)
    d_scores[cap["slot_of"].long()] = d_s                                     # slot f = k*T + t
    return y, dx_experts, d_wgu, d_wd, d_scores.view(K, T).t().contiguous()


def _worst_row(got, ref):
    """largest per-row error relative to the RMS row norm of the reference (a tile written to the
    wrong place, or not at all, shows up here however small its share of the whole tensor)"""
    got, ref = got.float(), ref.float()
    rms = ref.norm(dim=-1).pow(2).mean().sqrt()
    return float(((got - ref).norm(dim=-1) / rms).max())


@pytest.mark.parametrize("name", ["c3_qwen3_30b", "c5_stress"])
def test_full_size_every_row_and_expert(gpu_device, name):
    """C3 and C5 in full: EVERY row of y and dx and EVERY expert of both expert weight gradients
    (and d_router_gate) against the reference's formulas evaluated in float32 torch ops on the device."""
    T, H, E, K, I, bias_hot, n_hot, n_dead, _ = FULL[name]
    print("full-size, every row and expert", name, flush=True)
    dev = gpu_device
    x, wr, wgu, wd, dy = device_inputs(T, H, E, I, dev, 90210, bias_hot, n_hot, n_dead)
    layer = build_layer(torch.bfloat16, H, E, K, I, dev, loss_coeff=0.0)
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    layer.capture = {}
    xg = x.clone().requires_grad_(True)
    y = layer(xg)
    y.backward(dy)
    torch.cuda.synchronize()
    cap = layer.capture
    y_ref, dx_exp, d_wgu, d_wd, d_scores = _device_reference(x, wr, wgu, wd, dy, cap, K)

    e_y, w_y = O.rel_l2(y.detach().float().cpu(), y_ref.cpu()), _worst_row(y.detach(), y_ref)
    print(f"  y: rel-L2 {e_y:.2e}, worst row {w_y:.2e}", flush=True)
    assert e_y <= TOL and w_y <= 5 * TOL
    # the router's share of dx from the reference's formulas (oracle, all tokens) on the reference's score gradients
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.0)
    counts = cap["counts"].cpu().long()
    freq = counts.double() / counts.sum().double()
    _, d_logits = O.router_backward(d_scores.cpu().double(), cap["probs"].cpu().double(), cap["topk_idx"].cpu().long(), freq, ocfg, T)
    d_logits = d_logits.to(torch.bfloat16).to(dev)
    dx_ref = dx_exp + d_logits.float() @ wr.float()
    e_dx, w_dx = O.rel_l2(xg.grad.float().cpu(), dx_ref.cpu()), _worst_row(xg.grad, dx_ref)
    print(f"  dx: rel-L2 {e_dx:.2e}, worst row {w_dx:.2e}", flush=True)
    assert e_dx <= TOL and w_dx <= 5 * TOL
    e_wr = O.rel_l2(layer.router_gate.grad.float().cpu(), (d_logits.float().t() @ x.float()).cpu())
    print(f"  d_router_gate: rel-L2 {e_wr:.2e}", flush=True)
    assert e_wr <= TOL
    worst = {"gate_up": 0.0, "down": 0.0}
    for e in range(E):
        for nm, got, ref in (("gate_up", layer.expert_gate_up.grad[e], d_wgu[e]), ("down", layer.expert_down.grad[e], d_wd[e])):
            if int(counts[e]) == 0:
                assert bool((got == 0).all()), f"d_{nm}[{e}] of an expert without rows"
                continue
            err = float((got.float() - ref).norm() / ref.norm())
            worst[nm] = max(worst[nm], err)
            assert err <= TOL, f"d_{nm}[{e}]: {err:.3e}"
            assert _worst_row(got, ref) <= 5 * TOL, f"d_{nm}[{e}]: a row is off"
    print(f"  weight gradients, worst expert: gate_up {worst['gate_up']:.2e} down {worst['down']:.2e}", flush=True)


def test_full_size_c4_grouped_gemms(ops, gpu_device):
    """C4: one EP rank's share of a DeepSeek-V3-like layer -- 65536 pre-assigned rows,
    32 local experts with Zipf(1.2) loads, H=7168, I=2048; forward and backward grouped GEMMs."""
    R, E, H, I = 65536, 32, 7168, 2048
    print("full-size c4", flush=True)
    dev = gpu_device
    rng = np.random.Generator(np.random.PCG64(44))
    p = np.arange(1, E + 1, dtype=np.float64) ** -1.2
    counts = rng.multinomial(R, p / p.sum())
    offs_cpu = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    offs = torch.from_numpy(offs_cpu).to(dev)
    g = torch.Generator(device=dev).manual_seed(44)
    bf = torch.bfloat16
    xp = torch.randn(R, H, device=dev, generator=g).to(bf)
    dout = torch.randn(R, H, device=dev, generator=g).to(bf)
    scores = torch.rand(R, device=dev, generator=g)
    wgu = torch.empty(E, H, 2 * I, device=dev, dtype=bf)
    wd = torch.empty(E, I, H, device=dev, dtype=bf)
    for e in range(E):
        wgu[e] = (torch.randn(H, 2 * I, device=dev, generator=g) * 0.02).to(bf)
        wd[e] = (torch.randn(I, H, device=dev, generator=g) * 0.02).to(bf)
    act, dact = O.activation("silu"), O.silu_grad

    gate_up, inter_s = ops.grouped_gemm_gateup_act_fwd(xp, wgu, offs, row_scale=scores)
    out = ops.grouped_gemm_nn(inter_s, wd, offs)
    d_inter = ops.grouped_gemm_nt(dout, wd, offs)
    d_wd = ops.grouped_gemm_wgrad(inter_s, dout, offs, E)
    # the layer and bench.py run the data gradient of down with the gated-activation backward as its
    # epilogue; the unfused pair (d_inter above, gated_act_bwd) is the cross-check
    d_gu, parts = ops.grouped_gemm_nt_gated_bwd(dout, wd, offs, gate_up, row_scale=scores)
    d_gu_unfused = ops.gated_act_bwd(gate_up, d_inter, row_scale=scores)
    d_xp = ops.grouped_gemm_nt(d_gu, wgu, offs)
    d_wgu = ops.grouped_gemm_wgrad(xp, d_gu, offs, E)
    torch.cuda.synchronize()

    expert_of = np.repeat(np.arange(E), counts)
    rows = np.unique(np.concatenate([offs_cpu[:-1][counts > 0], offs_cpu[1:][counts > 0] - 1, rng.choice(R, 12)]))
    for r in rows:
        e = int(expert_of[r])
        gu_ref = xp[r].double() @ wgu[e].double()
        assert O.rel_l2(gate_up[r].double(), gu_ref) <= TOL, f"gate_up row {r}"
        gu_b = gate_up[r].double()
        inter_ref = scores[r].double() * gu_b[1::2] * act(gu_b[0::2])
        assert O.rel_l2(inter_s[r].double(), inter_ref) <= TOL, f"inter row {r}"
        assert O.rel_l2(out[r].double(), inter_s[r].double() @ wd[e].double()) <= TOL, f"down row {r}"
        assert O.rel_l2(d_inter[r].double(), wd[e].double() @ dout[r].double()) <= TOL, f"d_inter row {r}"
        dg_ref = torch.empty(2 * I, dtype=torch.float64, device=dev)
        di = d_inter[r].double()
        dg_ref[0::2] = scores[r].double() * di * gu_b[1::2] * dact(gu_b[0::2])
        dg_ref[1::2] = scores[r].double() * di * act(gu_b[0::2])
        assert O.rel_l2(d_gu[r].double(), dg_ref) <= TOL, f"d_gate_up row {r}"
        assert O.rel_l2(d_xp[r].double(), wgu[e].double() @ d_gu[r].double()) <= TOL, f"d_xp row {r}"
    for e in (0, E // 2, E - 1):
        r0, r1 = int(offs_cpu[e]), int(offs_cpu[e + 1])
        for i in (0, I - 1):
            ref_row = inter_s[r0:r1, i].double() @ dout[r0:r1].double()
            assert O.rel_l2(d_wd[e, i].double(), ref_row) <= TOL, f"dW_down[{e}][{i}]"
        for c in (1, 2 * I - 2):
            ref_col = xp[r0:r1].double().t() @ d_gu[r0:r1, c].double()
            assert O.rel_l2(d_wgu[e, :, c].double(), ref_col) <= TOL, f"dW_gate_up[{e}][:, {c}]"
    # fused against unfused on ALL rows (the unfused pair rounds d_inter to the model dtype in between)
    err = O.rel_l2(d_gu.float().cpu(), d_gu_unfused.float().cpu())
    print(f"  fused vs unfused d_gate_up, all rows: {err:.2e}", flush=True)
    assert err <= TOL and _worst_row(d_gu, d_gu_unfused) <= 5 * TOL
    # the score-gradient row sums of the fused kernel: sum_i d_inter * up * act(gate), all rows
    gu_f = gate_up.float()
    ds_ref = (d_inter.float() * gu_f[:, 1::2] * F.silu(gu_f[:, 0::2])).sum(1)
    err = O.rel_l2(parts.sum(0).cpu(), ds_ref.cpu())
    print(f"  score-gradient row sums, all rows: {err:.2e}", flush=True)
    assert err <= TOL
    del gu_f, ds_ref, d_gu_unfused
    # rows are processed exactly once: every output row is written (no NaN / stale memory)
    for t in (gate_up, inter_s, out, d_inter, d_xp, d_wd, d_wgu):
        assert bool(torch.isfinite(t.float()).all())
