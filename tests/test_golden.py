"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py):
the CPU oracle must keep reproducing them (CPU test) and the HIP layer must match them
(GPU test): routing bit-exact, values to rel-L2 1e-2 (bf16) / 1e-5 (float32)."""
import glob
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def _load(path):
    z = np.load(path, allow_pickle=False)
    dtype = torch.bfloat16 if int(z["is_bf16"]) else torch.float32
    t = {k: torch.from_numpy(z[k]) for k in z.files if z[k].ndim > 0}
    meta = {k: z[k].item() for k in z.files if z[k].ndim == 0}
    ins = [t[k].to(dtype) for k in ("x", "router_gate", "expert_gate_up", "expert_down", "dy")]
    cfg = O.OracleConfig(
        model_dim=meta["H"], intermediate_dim=meta["I"], num_experts=meta["E"], top_k=meta["K"],
        normalize_topk_scores=bool(meta["normalize"]), loss_coeff=meta["loss_coeff"],
    )
    return dtype, ins, cfg, t, meta


def test_fixtures_present():
    assert len(FIXTURES) >= 3


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_oracle_reproduces_fixture(path):
    dtype, (x, wr, wgu, wd, dy), cfg, t, meta = _load(path)
    ref = O.forward_backward(x, wr, wgu, wd, dy, cfg, compute_dtype=torch.float64)
    assert torch.equal(ref["topk_idx"].int(), t["topk_idx"])
    assert torch.equal(ref["counts"].int(), t["counts"])
    assert torch.equal(ref["perm"].int(), t["perm"])
    assert torch.equal(ref["token_ids"].int(), t["token_ids"])
    for k in ("y", "dx", "d_router_gate", "d_expert_gate_up", "d_expert_down"):
        assert O.rel_l2(ref[k], t[k]) < 1e-6, k
    # the reference-rounding mode (every op in the model dtype) routes identically here
    rr = O.forward(x, wr, wgu, wd, cfg)
    assert torch.equal(rr["topk_idx"].int(), t["topk_idx"])
    assert O.rel_l2(rr["y"], t["y"]) < (1e-2 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_hip_layer_matches_fixture(gpu_device, path):
    from arctictraining_amd import ArcticMoE, MoEConfig

    dtype, (x, wr, wgu, wd, dy), cfg, t, meta = _load(path)
    layer = ArcticMoE(
        MoEConfig(
            act_fn=F.silu, input_dtype=dtype, intermediate_dim=cfg.intermediate_dim, model_dim=cfg.model_dim,
            normalize_topk_scores=cfg.normalize_topk_scores, num_experts=cfg.num_experts, top_k=cfg.top_k,
            loss_coeff=cfg.loss_coeff,
        )
    ).to(gpu_device)
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    layer.capture = {}
    xg = x.to(gpu_device).requires_grad_(True)
    y = layer(xg)
    y.backward(dy.to(gpu_device))
    cap = layer.capture
    assert torch.equal(cap["topk_idx"].cpu(), t["topk_idx"]), "top-k indices"
    assert torch.equal(cap["counts"].cpu(), t["counts"]), "counts"
    assert torch.equal(cap["slot_of"].cpu(), t["perm"]), "permutation order"
    assert torch.equal(cap["token_of"].cpu(), t["token_ids"]), "token ids"
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    got = dict(
        y=y, dx=xg.grad, d_router_gate=layer.router_gate.grad, d_expert_gate_up=layer.expert_gate_up.grad,
        d_expert_down=layer.expert_down.grad,
    )
    for k, v in got.items():
        err = O.rel_l2(v.detach().cpu(), t[k])
        assert err <= tol, f"{k}: rel-L2 {err:.3e} > {tol}"
