"""Whole-layer parity: the ArcticMoE module (HIP kernels through the C ABI, forward and
backward) against the CPU oracle on the same seeded inputs.

Routing (top-k indices, per-expert counts, permutation order) must be bit-exact given the
logits the layer itself computed; outputs and gradients must agree with the oracle
evaluated in float64 from the same rounded inputs to rel-L2 <= 1e-2 (bf16) / 2.5e-3 (float16, whose
mantissa is 3 bits longer) / 1e-5 (float32).
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 1e-2, torch.float16: 2.5e-3, torch.float32: 1e-5}

# name: (dtype, T, H, E, K, I, extra make_inputs kwargs)  -- the BASELINE configurations,
# the first at full size, the bf16 ones scaled down so the float64 oracle runs in seconds
CONFIGS = {
    "c1_full_fp32": (torch.float32, 2048, 512, 8, 2, 1024, {}),
    "c2_mixtral_scaled": (torch.bfloat16, 1024, 512, 8, 2, 1792, {}),
    "c3_qwen3_scaled": (torch.bfloat16, 2048, 256, 128, 8, 192, {}),
    "c5_stress_scaled": (torch.bfloat16, 4096, 256, 64, 4, 192, dict(bias_hot=0.55, n_hot=4, n_dead=8)),
    "tiny_fp32": (torch.float32, 37, 64, 5, 3, 32, {}),
    "tiny_bf16_k1": (torch.bfloat16, 130, 64, 4, 1, 64, {}),
    # the largest expert count and top-k the kernels take; most experts get a handful of rows, some none
    "widest_routing": (torch.bfloat16, 300, 128, 512, 16, 64, {}),
    # float16: the third type the reference's kernels dispatch (top_k_gating.cpp:56-59)
    "tiny_f16": (torch.float16, 130, 64, 4, 2, 64, {}),
    "c3_qwen3_scaled_f16": (torch.float16, 2048, 256, 128, 8, 192, {}),
}


def build_layer(dtype, H, E, K, I, device, normalize=True, loss_coeff=0.001, act=F.silu, **kw):
    from arctictraining_amd import ArcticMoE, MoEConfig

    cfg = MoEConfig(
        act_fn=act,
        input_dtype=dtype,
        intermediate_dim=I,
        model_dim=H,
        normalize_topk_scores=normalize,
        num_experts=E,
        top_k=K,
        loss_coeff=loss_coeff,
        **kw,
    )
    return ArcticMoE(cfg).to(device)


def run_layer(layer, x, wr, wgu, wd, dy, device, replay=None):
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    for p in layer.parameters():
        p.grad = None
    layer.capture = {}
    xg = x.to(device).requires_grad_(True)
    out = layer(xg, replay) if replay is not None else layer(xg)
    y = out[0] if isinstance(out, tuple) else out
    y.backward(dy.to(device))
    torch.cuda.synchronize()
    return dict(
        y=y.detach().cpu(),
        dx=xg.grad.cpu(),
        d_router_gate=layer.router_gate.grad.cpu(),
        d_expert_gate_up=layer.expert_gate_up.grad.cpu(),
        d_expert_down=layer.expert_down.grad.cpu(),
        cap={k: v.cpu() for k, v in layer.capture.items()},
        out=out,
    )


def check_against_oracle(got, x, wr, wgu, wd, dy, ocfg, dtype, replay=None):
    cap = got["cap"]
    ref = O.forward_backward(
        x, wr, wgu, wd, dy, ocfg, compute_dtype=torch.float64, logits_for_selection=cap["logits"],
        replay_assignments=replay,
    )
    T, K = cap["topk_idx"].shape
    # ---- bit-exact routing
    assert torch.equal(cap["topk_idx"].long(), ref["topk_idx"]), "top-k indices"
    assert torch.equal(cap["counts"].long(), ref["counts"]), "per-expert counts"
    assert torch.equal(cap["slot_of"].long(), ref["perm"]), "permutation order"
    assert torch.equal(cap["token_of"].long(), ref["token_ids"]), "token ids"
    assert torch.equal(cap["row_of"].long(), O.inverse_row_map(ref["perm"], T, K)), "inverse map"
    # the layer's logits are the oracle's up to the rounding of the model dtype
    assert O.rel_l2(cap["logits"], ref["logits"]) <= TOL[dtype]
    # ---- values
    tol = TOL[dtype]
    errs = {k: O.rel_l2(got[k], ref[k]) for k in ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down")}
    print("rel-L2:", {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: rel-L2 {v:.3e} > {tol}"
    return ref, errs


@pytest.mark.parametrize("name", list(CONFIGS))
def test_layer_matches_oracle(gpu_device, name):
    dtype, T, H, E, K, I, extra = CONFIGS[name]
    print("layer", name, flush=True)
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=1234, **extra)
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    got = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)
    ref, _ = check_against_oracle(got, x, wr, wgu, wd, dy, ocfg, dtype)
    if name == "c5_stress_scaled":
        counts = ref["counts"]
        assert int((counts[-8:] == 0).sum()) == 8, "the biased router must starve the last 8 experts"
        assert 0.35 < float(counts[:4].sum()) / float(counts.sum()) < 0.65
        assert bool((got["d_expert_gate_up"][-8:] == 0).all()) and bool((got["d_expert_down"][-8:] == 0).all())


def test_layer_end_to_end_without_logit_handover(gpu_device):
    """Same inputs -> same routing with nothing handed from the device to the oracle: x in {-1, 0, 1}
    with 16 non-zeros a row and router weights in {-1/8, 0, 1/8}, so every logit is a multiple of 1/8
    of magnitude at most 2: exact in any summation order and in bf16, and full of ties.  The oracle
    computes its own logits (float64) and must select, count and permute exactly as the layer did."""
    dtype, T, H, E, K, I = torch.bfloat16, 4096, 256, 64, 4, 128
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=77)
    g = torch.Generator().manual_seed(78)
    xs = torch.zeros(T, H)
    cols = torch.rand(T, H, generator=g).argsort(dim=1)[:, :16]
    xs.scatter_(1, cols, torch.randint(0, 2, (T, 16), generator=g).float() * 2 - 1)
    x = xs.to(dtype)
    wr = (torch.randint(-1, 2, (E, H), generator=g).float() / 8).to(dtype)
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    got = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)
    ref = O.forward_backward(x, wr, wgu, wd, dy, ocfg, compute_dtype=torch.float64)
    cap = got["cap"]
    assert torch.equal(cap["logits"].double(), ref["logits"].double()), "the logits are exact on both sides"
    # ties: most tokens have a repeated value among their top logits, so the order of equal values matters
    top = ref["logits"].double().topk(K + 1, dim=1).values
    assert float((top[:, :-1] == top[:, 1:]).any(dim=1).float().mean()) > 0.5
    assert torch.equal(cap["topk_idx"].long(), ref["topk_idx"]), "top-k indices"
    assert torch.equal(cap["counts"].long(), ref["counts"]), "per-expert counts"
    assert torch.equal(cap["slot_of"].long(), ref["perm"]), "permutation order"
    assert torch.equal(cap["token_of"].long(), ref["token_ids"]), "token ids"
    for k in ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down"):
        err = O.rel_l2(got[k], ref[k])
        assert err <= TOL[dtype], f"{k}: rel-L2 {err:.3e}"


def test_layer_3d_input_and_no_normalisation(gpu_device):
    dtype, T, H, E, K, I = torch.bfloat16, 512, 128, 16, 4, 64
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=5)
    layer = build_layer(dtype, H, E, K, I, gpu_device, normalize=False, loss_coeff=0.05)
    got = run_layer(layer, x.view(4, T // 4, H), wr, wgu, wd, dy.view(4, T // 4, H), gpu_device)
    assert got["y"].shape == (4, T // 4, H)
    ocfg = O.OracleConfig(
        model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.05, normalize_topk_scores=False
    )
    got["y"], got["dx"] = got["y"].view(T, H), got["dx"].view(T, H)
    check_against_oracle(got, x, wr, wgu, wd, dy, ocfg, dtype)


def test_layer_load_balance_term(gpu_device):
    """The load-balance gradient (moe.py:393-406) changes d_router_gate and dx only, by
    the amount the oracle predicts."""
    dtype, T, H, E, K, I = torch.float32, 256, 64, 8, 2, 64
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=6)
    res = {}
    for coeff in (0.0, 5.0):
        layer = build_layer(dtype, H, E, K, I, gpu_device, loss_coeff=coeff)
        res[coeff] = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
        ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=coeff)
        check_against_oracle(res[coeff], x, wr, wgu, wd, dy, ocfg, dtype)
    assert torch.equal(res[0.0]["d_expert_down"], res[5.0]["d_expert_down"])
    assert not torch.equal(res[0.0]["d_router_gate"], res[5.0]["d_router_gate"])


def test_layer_routing_replay_and_returned_scores(gpu_device):
    """With replay the rows go to the replayed experts while the scores stay those of the
    layer's own top-k (moe.py:363-372); return_router_scores returns them in row order."""
    dtype, T, H, E, K, I = torch.bfloat16, 300, 128, 8, 2, 64
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=8)
    g = torch.Generator().manual_seed(9)
    replay = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    layer = build_layer(
        dtype, H, E, K, I, gpu_device, enable_routing_replay=True, return_router_scores=True
    )
    got = run_layer(layer, x, wr, wgu, wd, dy, gpu_device, replay=replay.to(gpu_device))
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)
    ref, _ = check_against_oracle(got, x, wr, wgu, wd, dy, ocfg, dtype, replay=replay)
    y, scores = got["out"]
    assert scores.shape == (T * K,) and scores.dtype == dtype
    assert O.rel_l2(scores.cpu(), ref["scores_perm"]) <= 1e-2
    with pytest.raises(AssertionError):
        layer(x.to(gpu_device))
    # an expert id outside [0, E) raises like the reference's one_hot (moe.py:374); with the check switched
    # off the permutation kernels clamp it (no host sync on the hot path)
    bad = replay.clone()
    bad[5, 0] = E + 3
    with pytest.raises(RuntimeError, match="outside"):
        layer(x.to(gpu_device), bad.to(gpu_device))
    layer.check_replay = False
    layer(x.to(gpu_device), bad.to(gpu_device))
    torch.cuda.synchronize()
    layer.check_replay = True


@pytest.mark.parametrize(
    "dtype,T,H,E,K,I,act",
    [
        (torch.float32, 128, 64, 4, 2, 32, "silu"),
        (torch.bfloat16, 1024, 256, 16, 4, 128, "silu"),
        (torch.bfloat16, 2048 + 96, 512, 8, 2, 256, "gelu"),  # token count not a multiple of any tile
        (torch.float16, 1024, 256, 16, 4, 128, "silu"),
    ],
    ids=["fp32", "bf16", "bf16_ragged_gelu", "f16"],
)
def test_layer_shared_expert(gpu_device, dtype, T, H, E, K, I, act):
    """Shared expert with a sigmoid output gate (moe.py:305-314) on top of the routed path:
    output and every gradient, the shared expert's parameters included, against the oracle."""
    tol = TOL[dtype]
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=10)
    layer = build_layer(dtype, H, E, K, I, gpu_device, use_shared_expert=True, act=getattr(F, act))
    g = torch.Generator().manual_seed(11)
    sgu, sd, sg = ((torch.randn(s, generator=g) * 0.05).to(dtype) for s in ((H, 2 * I), (I, H), (H, 1)))
    with torch.no_grad():
        layer.shared_expert_gate_up.copy_(sgu)
        layer.shared_expert_down.copy_(sd)
        layer.shared_expert_output_gate.copy_(sg)
    got = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001, act=act)
    ref = O.forward_backward(
        x, wr, wgu, wd, dy, ocfg, compute_dtype=torch.float64, logits_for_selection=got["cap"]["logits"],
        shared=(sgu, sd, sg),
    )
    assert torch.equal(got["cap"]["topk_idx"].long(), ref["topk_idx"])
    for k in ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down"):
        assert O.rel_l2(got[k], ref[k]) <= tol, k
    for name in ("shared_expert_gate_up", "shared_expert_down", "shared_expert_output_gate"):
        grad = getattr(layer, name).grad
        assert grad is not None and grad.shape == getattr(layer, name).shape
        assert O.rel_l2(grad.cpu(), ref["d_" + name]) <= tol, name
    # the shared expert must matter in this test: without it the output is far away
    routed_only = O.forward(x, wr, wgu, wd, ocfg, compute_dtype=torch.float64, logits_for_selection=got["cap"]["logits"])
    assert O.rel_l2(got["y"], routed_only["y"]) > 10 * tol


@pytest.mark.parametrize(
    "dtype,T,H,E,K,I,shared",
    [
        (torch.float32, 200, 64, 4, 2, 96, False),
        (torch.bfloat16, 1500, 256, 16, 4, 384, False),
        (torch.bfloat16, 1024, 256, 8, 2, 128, True),
        (torch.float32, 128, 64, 4, 2, 32, True),
        (torch.float16, 1024, 256, 8, 2, 128, True),
    ],
    ids=["fp32", "bf16", "bf16_shared", "fp32_shared", "f16_shared"],
)
def test_layer_without_gate(gpu_device, dtype, T, H, E, K, I, shared):
    """is_gated=False (moe.py:101-106, 188-191, 306-311): expert_gate_up is [E,H,I] and an expert is
    (x @ W_up) @ W_down with nothing in between; the routing scores weight the combine.  Output,
    returned scores and every gradient (with a gradient flowing into the returned scores) against
    the oracle."""
    tol = TOL[dtype]
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=21)
    wup = wgu[:, :, :I].contiguous()   # a plain [E,H,I] projection
    layer = build_layer(dtype, H, E, K, I, gpu_device, is_gated=False, use_shared_expert=shared,
                        return_router_scores=True)
    assert tuple(layer.expert_gate_up.shape) == (E, H, I)
    sh = None
    if shared:
        assert tuple(layer.shared_expert_gate_up.shape) == (H, I)
        g = torch.Generator().manual_seed(22)
        sh = tuple((torch.randn(s, generator=g) * 0.05).to(dtype) for s in ((H, I), (I, H), (H, 1)))
        with torch.no_grad():
            layer.shared_expert_gate_up.copy_(sh[0])
            layer.shared_expert_down.copy_(sh[1])
            layer.shared_expert_output_gate.copy_(sh[2])
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wup)
        layer.expert_down.copy_(wd)
    layer.capture = {}
    g = torch.Generator().manual_seed(23)
    d_sp = torch.randn(T * K, generator=g)
    xg = x.to(gpu_device).requires_grad_(True)
    y, sp = layer(xg)
    torch.autograd.backward([y, sp], [dy.to(gpu_device), d_sp.to(dtype).to(gpu_device)])
    torch.cuda.synchronize()
    cap = {k: v.cpu() for k, v in layer.capture.items()}
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001, is_gated=False)
    ref = O.forward_backward(
        x, wr, wup, wd, dy, ocfg, compute_dtype=torch.float64, logits_for_selection=cap["logits"], shared=sh,
        d_scores_perm=d_sp.to(dtype),
    )
    assert torch.equal(cap["topk_idx"].long(), ref["topk_idx"])
    assert torch.equal(cap["slot_of"].long(), ref["perm"])
    got = dict(y=y.detach().cpu(), dx=xg.grad.cpu(), d_router_gate=layer.router_gate.grad.cpu(),
               d_expert_gate_up=layer.expert_gate_up.grad.cpu(), d_expert_down=layer.expert_down.grad.cpu())
    errs = {k: O.rel_l2(v, ref[k]) for k, v in got.items()}
    print("rel-L2:", {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: rel-L2 {v:.3e} > {tol}"
    assert O.rel_l2(sp.detach().float().cpu(), ref["scores_perm"]) <= tol
    if shared:
        for name in ("shared_expert_gate_up", "shared_expert_down", "shared_expert_output_gate"):
            assert O.rel_l2(getattr(layer, name).grad.cpu(), ref["d_" + name]) <= tol, name


def test_layer_is_deterministic(gpu_device):
    dtype, T, H, E, K, I = torch.bfloat16, 1024, 256, 32, 4, 128
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=13)
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    a = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
    b = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
    for k in ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down"):
        assert torch.equal(a[k], b[k]), f"{k} differs between two identical runs"


def test_weight_gradients_on_the_second_stream_match_the_serial_order(gpu_device):
    """The backward runs the two expert weight gradients on a second stream (layer.overlap_weight_grads,
    on by default).  Every gradient must be bit-identical to the run with everything on one stream, over
    several steps in a row (a missing wait between the streams shows up as a stale or half-written tensor)."""
    dtype, T, H, E, K, I = torch.bfloat16, 4096, 256, 32, 4, 384
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    assert layer.overlap_weight_grads is True
    keys = ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down")
    for seed in (21, 22, 23):
        x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=seed)
        layer.overlap_weight_grads = False
        serial = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
        layer.overlap_weight_grads = True
        for rep in range(3):
            both = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)
            for k in keys:
                assert torch.equal(serial[k], both[k]), f"{k}, seed {seed}, repetition {rep}"


def test_module_surface(gpu_device):
    """Names, shapes and attributes the reference's callers rely on (moe.py:91-130,
    utils.py:61-68, 350-369, 449-461)."""
    layer = build_layer(torch.bfloat16, 128, 8, 2, 64, gpu_device, use_shared_expert=True)
    names = dict(layer.named_parameters())
    assert set(names) == {
        "router_gate", "expert_gate_up", "expert_down", "shared_expert_gate_up", "shared_expert_down",
        "shared_expert_output_gate",
    }
    assert names["router_gate"].shape == (8, 128)
    assert names["expert_gate_up"].shape == (8, 128, 128)
    assert names["expert_down"].shape == (8, 64, 128)
    assert layer.num_local_experts == 8 and layer.ep_size == 1 and layer.ep_rank == 0
    assert layer._config.use_shared_expert
    layer.enable_wall_clock_breakdown()
    assert layer.timers.wall_clock_breakdown
    x = torch.randn(16, 128, device=gpu_device, dtype=torch.bfloat16)
    for p in layer.parameters():
        torch.nn.init.normal_(p, std=0.02)
    layer(x)
    assert layer.timers.elapsed("amoe e2e") > 0 and layer.timers.elapsed("groupGeMM") > 0
    assert "expert_gate_up" in repr(layer)


def test_layer_under_hip_graph_capture(gpu_device):
    """Forward + backward captured into one HIP graph (nothing in the layer synchronises with the
    host or allocates outside torch's capturable allocator): every replay, with eager work and
    synchronisations between the replays, must reproduce the eager result bit for bit."""
    dtype, T, H, E, K, I = torch.bfloat16, 1024, 256, 32, 4, 128
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    g = torch.Generator().manual_seed(77)
    with torch.no_grad():
        for p in layer.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.05).to(dtype))
    xs = [torch.randn(T, H, generator=g).to(dtype).to(gpu_device) for _ in range(3)]
    dys = [torch.randn(T, H, generator=g).to(dtype).to(gpu_device) for _ in range(3)]

    def eager(x, dy):
        for p in layer.parameters():
            p.grad = None
        xg = x.clone().requires_grad_(True)
        y = layer(xg)
        y.backward(dy)
        return [y.detach().clone(), xg.grad.clone()] + [p.grad.clone() for p in layer.parameters()]

    want = [eager(x, dy) for x, dy in zip(xs, dys)]

    x_st = xs[0].clone().requires_grad_(True)
    dy_st = dys[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up on the capture stream: allocator pools, cached offsets
            for p in layer.parameters():
                p.grad = None
            x_st.grad = None
            layer(x_st).backward(dy_st)
    torch.cuda.current_stream().wait_stream(side)
    for p in layer.parameters():
        p.grad = None
    x_st.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_st = layer(x_st)
        y_st.backward(dy_st)
    # the graph's outputs live in its private pool: keep them, the eager runs below rebind .grad
    got = [y_st.detach(), x_st.grad] + [p.grad for p in layer.parameters()]
    for r in (0, 1, 2, 1):
        with torch.no_grad():
            x_st.copy_(xs[r])
            dy_st.copy_(dys[r])
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(got, want[r]):
            assert torch.equal(a, b), f"replay of input {r} differs from the eager result"
        # eager work between replays
        _ = eager(xs[(r + 1) % 3], dys[(r + 1) % 3])
        for p in layer.parameters():
            p.grad = None
        torch.cuda.synchronize()


def test_layer_with_frozen_parameters_and_plain_inference(gpu_device):
    """Gradients are only produced for what asks for them: frozen expert weights and a frozen
    router get none, the rest equal a run in which everything is trainable; a forward under
    no_grad gives the same output."""
    dtype, T, H, E, K, I = torch.bfloat16, 512, 128, 8, 2, 64
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=21)
    layer = build_layer(dtype, H, E, K, I, gpu_device)
    full = run_layer(layer, x, wr, wgu, wd, dy, gpu_device)

    layer.expert_gate_up.requires_grad_(False)
    layer.router_gate.requires_grad_(False)
    for p in layer.parameters():
        p.grad = None
    xg = x.to(gpu_device).requires_grad_(True)
    y = layer(xg)
    y.backward(dy.to(gpu_device))
    assert layer.expert_gate_up.grad is None and layer.router_gate.grad is None
    assert torch.equal(y.detach().cpu(), full["y"])
    assert torch.equal(xg.grad.cpu(), full["dx"])
    assert torch.equal(layer.expert_down.grad.cpu(), full["d_expert_down"])

    # input that needs no gradient: only the parameter gradients are computed
    layer.expert_gate_up.requires_grad_(True)
    for p in layer.parameters():
        p.grad = None
    layer(x.to(gpu_device)).backward(dy.to(gpu_device))
    assert torch.equal(layer.expert_gate_up.grad.cpu(), full["d_expert_gate_up"])

    with torch.no_grad():
        y2 = layer(x.to(gpu_device))
    assert not y2.requires_grad and torch.equal(y2.cpu(), full["y"])
