"""CPU restatement of the reference's expert-weight re-layout -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
module; the product path (arctictraining_amd.remap) runs HIP kernels and has no CPU fallback.

What it restates (numpy, byte moves only, so parity is bit-exact):
  pack_gate_up    arctic_training/model/moe/utils.py:232-251 -- per-expert nn.Linear weights
                  gate_proj / up_proj [I, H] are transposed, stacked over experts and
                  interleaved on the last dimension: out[e, h, 2i] = gate[e, i, h],
                  out[e, h, 2i+1] = up[e, i, h]
  pack_down       utils.py:253-254 (copy_weights with `.weight.T` per expert):
                  out[e, i, h] = down[e, h, i]
  unpack_gate_up  utils.py:366-379, unpack_down utils.py:381-395: the inverses

Pins (tests/test_remap.py): element-by-element index loops on small arrays (a dropped
transpose or a swapped gate/up parity fails them), the literal torch sequence of the reference
(`torch.stack((g, u), dim=-1).view(...)`) re-typed once as a cross-check of the numpy form,
round trips, and the forward of the installed transformers Qwen3MoeSparseMoeBlock against an
ArcticMoE oracle forward on the packed weights.
"""
import numpy as np


def pack_gate_up(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """gate, up [E, I, H] -> [E, H, 2I], gate in the even and up in the odd columns."""
    E, I, H = gate.shape
    return np.stack((gate.transpose(0, 2, 1), up.transpose(0, 2, 1)), axis=-1).reshape(E, H, 2 * I).copy()


def pack_down(down: np.ndarray) -> np.ndarray:
    """down [E, H, I] (nn.Linear [out=H, in=I]) -> expert_down [E, I, H]."""
    return down.transpose(0, 2, 1).copy()


def unpack_gate_up(gate_up: np.ndarray):
    """[E, H, 2I] -> (gate [E, I, H], up [E, I, H])."""
    E, H, I2 = gate_up.shape
    pair = gate_up.reshape(E, H, I2 // 2, 2)
    return pair[..., 0].transpose(0, 2, 1).copy(), pair[..., 1].transpose(0, 2, 1).copy()


def unpack_down(expert_down: np.ndarray) -> np.ndarray:
    """expert_down [E, I, H] -> down_proj weights [E, H, I]."""
    return expert_down.transpose(0, 2, 1).copy()
