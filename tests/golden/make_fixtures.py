"""Writes the golden fixtures of the expert layer: seeded inputs and the CPU oracle's
outputs (routing, output, every gradient) for a few tiny configurations.

    python tests/golden/make_fixtures.py

The reference holds no golden vector for this path (its only MoE test compares training
losses end to end), so these fixtures come from the oracle, which is itself pinned by
tests/test_oracle_pins.py.  The router weights are chosen so that the logits are exact in
the model dtype on any device, which makes the routing of a fixture unambiguous.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import moe_oracle as O  # noqa: E402

# name: dtype, T, H, E, K, I, normalize, loss_coeff
CASES = {
    "f32_t48_h64_e8_k2_i32": (torch.float32, 48, 64, 8, 2, 32, True, 0.01),
    "bf16_t64_h64_e8_k2_i64": (torch.bfloat16, 64, 64, 8, 2, 64, True, 0.001),
    "bf16_t40_h64_e16_k4_i32_nonorm": (torch.bfloat16, 40, 64, 16, 4, 32, False, 0.02),
}


def f32(t):
    return t.detach().to(torch.float32).numpy()


def build(name):
    dtype, T, H, E, K, I, norm, coeff = CASES[name]
    seed = 7
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=seed)
    # Router rows with a single power-of-two entry: logit[t, e] = +-2^s * x[t, c_e] is then
    # exact in the model dtype whatever the accumulation order, so every device computes
    # bit-identical logits and the routing of the fixture is unambiguous (ties included).
    g = torch.Generator().manual_seed(seed)
    cols = torch.randperm(H, generator=g)[:E]
    wr = torch.zeros(E, H)
    wr[torch.arange(E), cols] = torch.tensor([1.0, -1.0, 2.0, 0.5])[torch.arange(E) % 4]
    wr = wr.to(dtype)
    logits = O.router_linear(x.double(), wr.double())
    assert torch.equal(logits, logits.to(dtype).double()), "logits must be exact in the model dtype"
    v, _ = torch.sort(logits, dim=-1, descending=True)
    gap = float((v[:, :-1] - v[:, 1:])[:, :K].min())
    cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, normalize_topk_scores=norm,
                         loss_coeff=coeff)
    ref = O.forward_backward(x, wr, wgu, wd, dy, cfg, compute_dtype=torch.float64)
    out = dict(
        seed=np.int64(seed), gap=np.float64(gap), T=np.int64(T), H=np.int64(H), E=np.int64(E), K=np.int64(K),
        I=np.int64(I), normalize=np.int64(norm), loss_coeff=np.float64(coeff),
        is_bf16=np.int64(dtype == torch.bfloat16),
        x=x.float().numpy(), router_gate=wr.float().numpy(), expert_gate_up=wgu.float().numpy(),
        expert_down=wd.float().numpy(), dy=dy.float().numpy(),
        topk_idx=ref["topk_idx"].numpy().astype(np.int32), counts=ref["counts"].numpy().astype(np.int32),
        perm=ref["perm"].numpy().astype(np.int32), token_ids=ref["token_ids"].numpy().astype(np.int32),
        # float64 results stored as float32: 6e-8 relative, far inside the 1e-5 / 1e-2 bars
        scores_tk=f32(ref["scores_tk"]), y=f32(ref["y"]), dx=f32(ref["dx"]),
        d_router_gate=f32(ref["d_router_gate"]), d_expert_gate_up=f32(ref["d_expert_gate_up"]),
        d_expert_down=f32(ref["d_expert_down"]),
    )
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print(name, "seed", seed, "gap %.4f" % gap)


if __name__ == "__main__":
    for n in CASES:
        build(n)
