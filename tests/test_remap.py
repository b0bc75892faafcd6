"""Expert-weight re-layout (checkpoint format <-> ArcticMoE parameters).

CPU part: the numpy oracle is pinned by element-by-element index loops, by the literal torch
sequence the reference runs (utils.py:232-251 / 366-379), by round trips, and through the
installed transformers Qwen3MoeSparseMoeBlock: its forward must equal the oracle's ArcticMoE
forward on the weights the remap oracle packed.
GPU part (marked gpu): the HIP kernels through the C ABI are bit-exact against the oracle,
including ragged tile edges, fused [E,2I,H] inputs, float32, and the headline shape by round
trip; the install / restore hooks reproduce the HF block's output and give its weights back
bit for bit.
"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import remap_oracle as RO


def _rand(shape, seed):
    return np.random.default_rng(seed).integers(0, 2**16, size=shape, dtype=np.uint16)


def test_oracle_pack_matches_index_definition():
    E, I, H = 2, 3, 5
    gate, up, down = _rand((E, I, H), 1), _rand((E, I, H), 2), _rand((E, H, I), 3)
    gu, dn = RO.pack_gate_up(gate, up), RO.pack_down(down)
    assert gu.shape == (E, H, 2 * I) and dn.shape == (E, I, H)
    for e in range(E):
        for i in range(I):
            for h in range(H):
                assert gu[e, h, 2 * i] == gate[e, i, h]
                assert gu[e, h, 2 * i + 1] == up[e, i, h]
                assert dn[e, i, h] == down[e, h, i]


def test_oracle_matches_reference_torch_sequence():
    E, I, H = 3, 4, 6
    g = torch.randn(E, I, H)
    u = torch.randn(E, I, H)
    # utils.py:232-247: per-expert `.weight.T` stacked, then stack(dim=-1).view
    gate_stacked = torch.stack([g[i].T for i in range(E)])
    up_stacked = torch.stack([u[i].T for i in range(E)])
    ref = torch.stack((gate_stacked, up_stacked), dim=-1).view(*up_stacked.shape[:-1], -1).contiguous()
    assert np.array_equal(RO.pack_gate_up(g.numpy(), u.numpy()), ref.numpy())
    # utils.py:366-374: unbind of the (-1, 2) view
    gate_un, up_un = torch.unbind(ref.view(-1, 2), dim=-1)
    gate_un = gate_un.view(*ref.shape[:-1], -1)
    g2, u2 = RO.unpack_gate_up(ref.numpy())
    assert np.array_equal(g2, torch.stack([x.T for x in gate_un.unbind()]).numpy())
    assert np.array_equal(g2, g.numpy()) and np.array_equal(u2, u.numpy())


def test_oracle_round_trip():
    E, I, H = 4, 24, 40
    gate, up, down = _rand((E, I, H), 4), _rand((E, I, H), 5), _rand((E, H, I), 6)
    g2, u2 = RO.unpack_gate_up(RO.pack_gate_up(gate, up))
    assert np.array_equal(g2, gate) and np.array_equal(u2, up)
    assert np.array_equal(RO.unpack_down(RO.pack_down(down)), down)


def _tiny_hf_block(dtype=torch.float64, E=8, K=2, H=32, I=16, seed=0):
    from transformers import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

    c = Qwen3MoeConfig(
        hidden_size=H, intermediate_size=4 * H, moe_intermediate_size=I, num_experts=E, num_experts_per_tok=K,
        norm_topk_prob=True, num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=2, vocab_size=64,
        hidden_act="silu", router_aux_loss_coef=0.0,
    )
    torch.manual_seed(seed)
    blk = Qwen3MoeSparseMoeBlock(c)
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn_like(p) * 0.2)
    return c, blk.to(dtype)


def test_packed_weights_reproduce_hf_block():
    c, blk = _tiny_hf_block()
    E, I, H = c.num_experts, c.moe_intermediate_size, c.hidden_size
    fused = blk.experts.gate_up_proj.detach().numpy()
    gu = torch.from_numpy(RO.pack_gate_up(fused[:, :I, :], fused[:, I:, :]))
    dn = torch.from_numpy(RO.pack_down(blk.experts.down_proj.detach().numpy()))
    x = torch.randn(2, 11, H, dtype=torch.float64)
    ocfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=c.num_experts_per_tok, loss_coeff=0.0)
    ref = O.forward(x.view(-1, H), blk.gate.weight.detach(), gu, dn, ocfg, compute_dtype=torch.float64)
    assert torch.allclose(ref["y"].view_as(x), blk(x), atol=5e-6)


# ------------------------------------------------------------------ GPU: the HIP kernels
@pytest.fixture(scope="module")
def ops(gpu_device):
    from arctictraining_amd import ops as _ops

    return _ops


def _as_np(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,E,I,H", [
    (torch.bfloat16, 3, 64, 128), (torch.bfloat16, 2, 72, 200), (torch.bfloat16, 1, 8, 8),
    (torch.bfloat16, 5, 192, 256), (torch.float32, 2, 36, 52), (torch.float32, 3, 128, 64),
])
def test_hip_remap_bit_exact(ops, gpu_device, dtype, E, I, H):
    print("remap", dtype, E, I, H, flush=True)
    g = torch.Generator().manual_seed(E * 1000 + I + H)
    gate, up = torch.randn(E, I, H, generator=g).to(dtype), torch.randn(E, I, H, generator=g).to(dtype)
    down = torch.randn(E, H, I, generator=g).to(dtype)
    gu = ops.remap_pack(gate.to(gpu_device), up.to(gpu_device))
    dn = ops.remap_pack(down.to(gpu_device))
    assert np.array_equal(_as_np(gu), RO.pack_gate_up(_as_np(gate), _as_np(up)))
    assert np.array_equal(_as_np(dn), RO.pack_down(_as_np(down)))
    # fused [E, 2I, H] input: two strided halves of one tensor
    fused = torch.cat((gate, up), dim=1).to(gpu_device)
    assert torch.equal(ops.remap_pack(fused[:, :I, :], fused[:, I:, :]), gu)
    # inverse
    g2, u2 = ops.remap_unpack(gu, two=True)
    assert torch.equal(g2.cpu(), gate) and torch.equal(u2.cpu(), up)
    assert torch.equal(ops.remap_unpack(dn, two=False).cpu(), down)
    out = torch.empty_like(fused)
    ops.remap_unpack(gu, two=True, out0=out[:, :I, :], out1=out[:, I:, :])
    assert torch.equal(out, fused)


@pytest.mark.gpu
def test_hip_remap_headline_shape_round_trip(ops, gpu_device):
    E, I, H = 128, 768, 2048
    g = torch.Generator(device=gpu_device).manual_seed(5)
    fused = torch.randn(E, 2 * I, H, device=gpu_device, generator=g).to(torch.bfloat16)
    gu = ops.remap_pack(fused[:, :I, :], fused[:, I:, :])
    # sampled elements against the definition, then the whole tensor by round trip
    rng = np.random.default_rng(3)
    for e, i, h in zip(rng.integers(0, E, 64), rng.integers(0, I, 64), rng.integers(0, H, 64)):
        assert gu[e, h, 2 * i] == fused[e, i, h] and gu[e, h, 2 * i + 1] == fused[e, I + i, h]
    back = torch.empty_like(fused)
    ops.remap_unpack(gu, two=True, out0=back[:, :I, :], out1=back[:, I:, :])
    assert torch.equal(back, fused)


@pytest.mark.gpu
@pytest.mark.parametrize("as_list", [False, True])
def test_install_and_restore_hooks(gpu_device, as_list):
    """A one-layer stand-in for a HF MoE model: install ArcticMoE from its block, compare the
    forward with the block's own, restore, and get the original weights back bit for bit."""
    from types import SimpleNamespace

    from arctictraining_amd import ArcticMoE
    from arctictraining_amd.remap import (
        detect_if_moe_model, remap_arctic_moe_to_orig_moe_mlp_params, remap_orig_moe_mlp_params_to_arctic_moe)

    c, blk = _tiny_hf_block(dtype=torch.float32, E=8, K=2, H=64, I=32, seed=3)
    c.architectures = ["Qwen3MoeForCausalLM"]
    blk = blk.to(gpu_device)
    E, I = c.num_experts, c.moe_intermediate_size
    if as_list:  # the per-expert nn.Linear form the reference reads
        fused, down = blk.experts.gate_up_proj.detach(), blk.experts.down_proj.detach()
        experts = torch.nn.ModuleList()
        for e in range(E):
            ex = torch.nn.Module()
            ex.gate_proj = torch.nn.Linear(c.hidden_size, I, bias=False, device=gpu_device)
            ex.up_proj = torch.nn.Linear(c.hidden_size, I, bias=False, device=gpu_device)
            ex.down_proj = torch.nn.Linear(I, c.hidden_size, bias=False, device=gpu_device)
            with torch.no_grad():
                ex.gate_proj.weight.copy_(fused[e, :I])
                ex.up_proj.weight.copy_(fused[e, I:])
                ex.down_proj.weight.copy_(down[e])
            experts.append(ex)
        mlp = torch.nn.Module()
        mlp.gate, mlp.experts = blk.gate, experts
    else:
        mlp = blk
    x = torch.randn(3, 17, c.hidden_size, device=gpu_device)
    with torch.no_grad():
        y_ref = blk(x)
    saved = {k: v.detach().clone() for k, v in mlp.state_dict().items()}

    layer = torch.nn.Module()
    layer.mlp = mlp
    dense_layer = torch.nn.Module()
    dense_layer.mlp = torch.nn.Linear(4, 4)  # a layer without experts is left alone
    model = torch.nn.Module()
    model.model = torch.nn.Module()
    model.model.layers = torch.nn.ModuleList([dense_layer, layer])
    model.config, model.dtype = c, torch.float32
    assert detect_if_moe_model(model)

    remap_orig_moe_mlp_params_to_arctic_moe(model, ep_size=1, is_resume=False, device=gpu_device)
    amoe = model.model.layers[1].mlp
    assert isinstance(amoe, ArcticMoE) and isinstance(model.model.layers[0].mlp, torch.nn.Linear)
    assert {n for n, _ in amoe.named_parameters()} == {"router_gate", "expert_gate_up", "expert_down"}
    assert all(p.device.type == "meta" for p in amoe._hide["orig_mlp"].parameters())
    with torch.no_grad():
        y = amoe(x)
    assert O.rel_l2(y.cpu(), y_ref.cpu()) <= 1e-5

    remap_arctic_moe_to_orig_moe_mlp_params(model)
    restored = model.model.layers[1].mlp
    assert not isinstance(restored, ArcticMoE)
    got = restored.state_dict()
    assert got.keys() == saved.keys()
    for k in saved:
        assert torch.equal(got[k], saved[k]), k


@pytest.mark.gpu
def test_install_and_restore_hooks_shared_expert(gpu_device):
    """The same round trip for a block with a shared expert and its sigmoid gate (the installed
    transformers Qwen2-MoE block; utils.py:268-289 and :400-418)."""
    from transformers import Qwen2MoeConfig
    from transformers.models.qwen2_moe.modeling_qwen2_moe import Qwen2MoeSparseMoeBlock

    from arctictraining_amd import ArcticMoE
    from arctictraining_amd.remap import remap_arctic_moe_to_orig_moe_mlp_params, remap_orig_moe_mlp_params_to_arctic_moe

    H, I, E, K = 64, 32, 8, 2
    c = Qwen2MoeConfig(
        hidden_size=H, moe_intermediate_size=I, shared_expert_intermediate_size=I, intermediate_size=I, num_experts=E,
        num_experts_per_tok=K, norm_topk_prob=True, hidden_act="silu", num_hidden_layers=1, num_attention_heads=1,
        num_key_value_heads=1, vocab_size=8,
    )
    c.architectures = ["Qwen2MoeForCausalLM"]
    blk = Qwen2MoeSparseMoeBlock(c).to(torch.float32)
    g = torch.Generator().manual_seed(5)
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.2)
    blk = blk.to(gpu_device)
    x = torch.randn(2, 19, H, generator=g).to(gpu_device)
    xr = x.clone().requires_grad_(True)
    y_ref = blk(xr)
    y_ref.sum().backward()
    saved = {k: v.detach().clone() for k, v in blk.state_dict().items()}
    # gradients of the block's own run, in the block's layout (the install empties the block)
    ref_grad = {k: p.grad.detach().cpu() for k, p in blk.named_parameters()}

    layer = torch.nn.Module()
    layer.mlp = blk
    model = torch.nn.Module()
    model.model = torch.nn.Module()
    model.model.layers = torch.nn.ModuleList([layer])
    model.config, model.dtype = c, torch.float32
    remap_orig_moe_mlp_params_to_arctic_moe(model, device=gpu_device)
    amoe = model.model.layers[0].mlp
    assert isinstance(amoe, ArcticMoE) and amoe._config.use_shared_expert
    amoe._config.loss_coeff = 0.0  # HF's block has no load-balance term in its gradient
    xa = x.clone().requires_grad_(True)
    y = amoe(xa)
    y.sum().backward()
    assert O.rel_l2(y.detach().cpu(), y_ref.detach().cpu()) <= 1e-5
    assert O.rel_l2(xa.grad.cpu(), xr.grad.cpu()) <= 1e-5
    assert O.rel_l2(amoe.shared_expert_gate_up.grad[:, 0::2].t().cpu(), ref_grad["shared_expert.gate_proj.weight"]) <= 1e-5
    assert O.rel_l2(amoe.shared_expert_gate_up.grad[:, 1::2].t().cpu(), ref_grad["shared_expert.up_proj.weight"]) <= 1e-5
    assert O.rel_l2(amoe.shared_expert_down.grad.t().cpu(), ref_grad["shared_expert.down_proj.weight"]) <= 1e-5
    assert O.rel_l2(amoe.shared_expert_output_gate.grad.t().cpu(), ref_grad["shared_expert_gate.weight"]) <= 1e-5
    assert O.rel_l2(amoe.router_gate.grad.cpu(), ref_grad["gate.weight"]) <= 1e-5

    remap_arctic_moe_to_orig_moe_mlp_params(model)
    got = model.model.layers[0].mlp.state_dict()
    assert got.keys() == saved.keys()
    for k in saved:
        assert torch.equal(got[k], saved[k]), k


@pytest.mark.gpu
@pytest.mark.parametrize("transposed", [True, False])
def test_install_and_restore_hooks_gpt_oss_layout(gpu_device, transposed):
    """The reference's non-list branch (utils.py:291-299): fused experts whose gate_up_proj
    INTERLEAVES gate and up, stored [E, 2I, H] (transposed on install) or already [E, H, 2I].
    The installed layer must hold exactly gate in the even and up in the odd columns."""
    from types import SimpleNamespace

    from arctictraining_amd import ArcticMoE
    from arctictraining_amd.remap import remap_arctic_moe_to_orig_moe_mlp_params, remap_orig_moe_mlp_params_to_arctic_moe

    E, K, H, I = 4, 2, 64, 48
    g = torch.Generator().manual_seed(8)
    gate_w, up_w = torch.randn(E, H, I, generator=g), torch.randn(E, H, I, generator=g)   # [in, out]
    interleaved = torch.stack((gate_w, up_w), dim=-1).reshape(E, H, 2 * I)                # ArcticMoE layout
    down_w = torch.randn(E, H, I, generator=g)                                            # nn.Linear layout [out, in]
    experts = torch.nn.Module()
    experts.gate_up_proj = torch.nn.Parameter((interleaved.transpose(1, 2) if transposed else interleaved).contiguous())
    experts.down_proj = torch.nn.Parameter(down_w.clone())
    mlp = torch.nn.Module()
    mlp.gate = torch.nn.Linear(H, E, bias=False)
    mlp.experts = experts
    mlp = mlp.to(gpu_device)
    saved = {k: v.detach().clone() for k, v in mlp.state_dict().items()}
    layer = torch.nn.Module()
    layer.mlp = mlp
    model = torch.nn.Module()
    model.model = torch.nn.Module()
    model.model.layers = torch.nn.ModuleList([layer])
    model.config = SimpleNamespace(hidden_size=H, num_experts_per_tok=K, router_aux_loss_coef=0.0, hidden_act="silu",
                                   intermediate_size=I, num_local_experts=E, architectures=["GptOssForCausalLM"])
    model.dtype = torch.float32
    remap_orig_moe_mlp_params_to_arctic_moe(model, device=gpu_device)
    amoe = model.model.layers[0].mlp
    assert isinstance(amoe, ArcticMoE) and amoe._config.return_router_scores
    assert torch.equal(amoe.expert_gate_up.detach().cpu(), interleaved)
    assert torch.equal(amoe.expert_down.detach().cpu(), down_w.transpose(1, 2))
    remap_arctic_moe_to_orig_moe_mlp_params(model)
    got = model.model.layers[0].mlp.state_dict()
    for k in saved:
        assert torch.equal(got[k], saved[k]), k


@pytest.mark.gpu
def test_fused_layout_mismatch_is_an_error(gpu_device):
    """A fused gate_up_proj that does not have the [E, 2I, H] shape of the architecture's format
    raises instead of being misread."""
    from types import SimpleNamespace

    from arctictraining_amd.remap import remap_orig_moe_mlp_params_to_arctic_moe

    E, K, H, I = 4, 2, 64, 48
    experts = torch.nn.Module()
    experts.gate_up_proj = torch.nn.Parameter(torch.zeros(E, H, 2 * I))   # gpt-oss layout under a Qwen architecture
    experts.down_proj = torch.nn.Parameter(torch.zeros(E, H, I))
    mlp = torch.nn.Module()
    mlp.gate = torch.nn.Linear(H, E, bias=False)
    mlp.experts = experts
    layer = torch.nn.Module()
    layer.mlp = mlp.to(gpu_device)
    model = torch.nn.Module()
    model.model = torch.nn.Module()
    model.model.layers = torch.nn.ModuleList([layer])
    model.config = SimpleNamespace(hidden_size=H, num_experts_per_tok=K, router_aux_loss_coef=0.0, hidden_act="silu",
                                   moe_intermediate_size=I, num_experts=E, architectures=["Qwen3MoeForCausalLM"])
    model.dtype = torch.float32
    with pytest.raises(ValueError, match="interleaves"):
        remap_orig_moe_mlp_params_to_arctic_moe(model, device=gpu_device)


def _gpt_oss_model(E, K, H, I, gate_up_param, down_w, flag=None):
    from types import SimpleNamespace

    experts = torch.nn.Module()
    experts.gate_up_proj = torch.nn.Parameter(gate_up_param)
    experts.down_proj = torch.nn.Parameter(down_w.clone())
    mlp = torch.nn.Module()
    mlp.gate = torch.nn.Linear(H, E, bias=False)
    mlp.experts = experts
    layer = torch.nn.Module()
    layer.mlp = mlp
    model = torch.nn.Module()
    model.model = torch.nn.Module()
    model.model.layers = torch.nn.ModuleList([layer])
    model.config = SimpleNamespace(hidden_size=H, num_experts_per_tok=K, router_aux_loss_coef=0.0, hidden_act="silu",
                                   intermediate_size=I, num_local_experts=E, architectures=["GptOssForCausalLM"])
    if flag is not None:
        model.config.fused_gate_up_transposed = flag
    model.dtype = torch.float32
    return model


def test_square_interleaved_gate_up_is_not_guessed():
    """hidden == 2 * intermediate: the shape of an interleaved gate_up_proj does not tell its orientation.
    Without the explicit flag the hook raises (no GPU needed: the error comes before any kernel)."""
    from arctictraining_amd.remap import remap_orig_moe_mlp_params_to_arctic_moe

    E, K, H, I = 2, 1, 64, 32
    g = torch.Generator().manual_seed(3)
    model = _gpt_oss_model(E, K, H, I, torch.randn(E, H, 2 * I, generator=g), torch.randn(E, H, I, generator=g))
    with pytest.raises(ValueError, match="square"):
        remap_orig_moe_mlp_params_to_arctic_moe(model, device="cpu")
    # a flag that contradicts an unambiguous shape is an error too
    model = _gpt_oss_model(E, K, H, 24, torch.randn(E, H, 48, generator=g), torch.randn(E, H, 24, generator=g), flag=True)
    with pytest.raises(ValueError, match="fused_gate_up_transposed"):
        remap_orig_moe_mlp_params_to_arctic_moe(model, device="cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("transposed", [True, False])
def test_square_interleaved_gate_up_follows_the_flag(gpu_device, transposed):
    """hidden == 2 * intermediate with fused_gate_up_transposed set: True transposes on install (what the
    reference always does, utils.py:296), False copies; both restore the original tensor."""
    from arctictraining_amd.remap import remap_arctic_moe_to_orig_moe_mlp_params, remap_orig_moe_mlp_params_to_arctic_moe

    E, K, H, I = 4, 2, 64, 32
    g = torch.Generator().manual_seed(9)
    gate_w, up_w = torch.randn(E, H, I, generator=g), torch.randn(E, H, I, generator=g)
    interleaved = torch.stack((gate_w, up_w), dim=-1).reshape(E, H, 2 * I)
    down_w = torch.randn(E, H, I, generator=g)
    stored = (interleaved.transpose(1, 2) if transposed else interleaved).contiguous()
    model = _gpt_oss_model(E, K, H, I, stored, down_w, flag=transposed).to(gpu_device)
    model.dtype = torch.float32
    saved = {k: v.detach().clone() for k, v in model.model.layers[0].mlp.state_dict().items()}
    remap_orig_moe_mlp_params_to_arctic_moe(model, device=gpu_device)
    amoe = model.model.layers[0].mlp
    assert torch.equal(amoe.expert_gate_up.detach().cpu(), interleaved)
    remap_arctic_moe_to_orig_moe_mlp_params(model)
    got = model.model.layers[0].mlp.state_dict()
    for k in saved:
        assert torch.equal(got[k], saved[k]), k
