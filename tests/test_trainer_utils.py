"""Host logic around the layer: expert-parameter tagging, optimizer group split, checkpoint
file name, timing report (arctic_training/model/moe/utils.py:61-68, 425-543; moe.py:465-509).
Runs on the CPU: the ArcticMoE module can be constructed (parameters only) without a GPU."""
import torch
import torch.nn.functional as F

from arctictraining_amd import ArcticMoE, MoEConfig
from arctictraining_amd import utils as U


def _model(n_moe=2):
    cfg = MoEConfig(act_fn=F.silu, input_dtype=torch.float32, intermediate_dim=8, model_dim=16, num_experts=4, top_k=2,
                    normalize_topk_scores=True)
    m = torch.nn.Module()
    m.embed = torch.nn.Embedding(10, 16)
    m.layers = torch.nn.ModuleList()
    for _ in range(n_moe):
        layer = torch.nn.Module()
        layer.attn = torch.nn.Linear(16, 16)
        layer.mlp = ArcticMoE(cfg)
        m.layers.append(layer)
    return m


def test_identify_expert_params_tags_only_expert_weights():
    m = _model()
    ptrs = U.identify_expert_params(m, ep_size=1)
    assert len(ptrs) == 4  # expert_gate_up + expert_down per layer
    for name, p in m.named_parameters():
        is_exp = name.endswith("expert_gate_up") or name.endswith("expert_down")
        assert U.is_expert_param(p, ptrs) == is_exp, name
        if is_exp:
            assert p.allreduce is False and p.group_name == "ep_size_1"
        else:
            assert not hasattr(p, "group_name")


def test_split_param_groups():
    m = _model()
    ptrs = U.identify_expert_params(m, ep_size=1)
    decay = [p for n, p in m.named_parameters() if p.dim() > 1]
    no_decay = [p for n, p in m.named_parameters() if p.dim() <= 1]
    groups = [
        {"name": "decay", "params": list(decay), "weight_decay": 0.1, "lr": 1e-3},
        {"name": "no_decay", "params": list(no_decay), "weight_decay": 0.0, "lr": 1e-3},
    ]
    out = U.split_params_into_different_moe_groups_for_optimizer(groups, ptrs)
    assert [g["name"] for g in out] == ["decay", "no_decay", "ep_size_1", "ep_size_1"]
    moe_decay, moe_no_decay = out[2], out[3]
    assert moe_decay["moe"] is True and moe_decay["weight_decay"] == 0.1 and len(moe_decay["params"]) == 4
    assert moe_no_decay["moe"] is True and moe_no_decay["weight_decay"] == 0.0 and moe_no_decay["params"] == []
    assert all(not U.is_expert_param(p, ptrs) for p in out[0]["params"])
    # every parameter is still in exactly one group
    ids = [id(p) for g in out for p in g["params"]]
    assert sorted(ids) == sorted(id(p) for p in m.parameters())
    # the result feeds a torch optimizer as is
    torch.optim.AdamW([g for g in out if g["params"]])
    # dict and tuple inputs are accepted, anything else is an error
    assert len(U.split_params_into_different_moe_groups_for_optimizer({"name": "g", "params": []}, ptrs)) == 1
    assert isinstance(U.split_params_into_different_moe_groups_for_optimizer(({"name": "g", "params": []},), ptrs), list)
    try:
        U.split_params_into_different_moe_groups_for_optimizer("nope", ptrs)
        raise AssertionError("expected ValueError")
    except ValueError:
        pass


def test_expert_ckpt_name():
    assert U.get_expert_ckpt_name("/ckpt", "step10", 3, 7) == "/ckpt/step10/ep_rank_3_moe_layer_7_model_states.pt"


def test_timers_install_and_forward_breakdown():
    m = _model()

    class Engine:
        def wall_clock_breakdown(self):
            return True

    U.amoe_install_deepspeed_timers(Engine(), m)
    layers = [x for x in m.modules() if isinstance(x, ArcticMoE)]
    assert all(x.wall_clock_breakdown and x.timers.wall_clock_breakdown for x in layers)
    for i, layer in enumerate(layers):
        layer.timers.times["moe-gate"] += 1.5 + i
        layer.timers.times["moe-expert-gemm"] += 4.0
        layer.timers.token_counts["tokens"] += 2000
    lines = []
    U.print_forward_breakdown(m, 0.0, printer=lines.append)
    text = "\n".join(lines)
    assert "layer=0 time  : moe-gate" in text and "layer=1 tokens: tokens:   2.00K" in text
    assert "all layers aggregate time (ms): moe-gate: 4.00 | moe-expert-gemm: 8.00" in text
    assert "all layers aggregate token counts (K): tokens: 4.00" in text
    # a model without ArcticMoE layers prints nothing
    lines.clear()
    U.print_forward_breakdown(torch.nn.Linear(2, 2), printer=lines.append)
    assert lines == []


class _FakeEngine:
    """The attributes of a DeepSpeed engine the checkpoint routines read."""

    def __init__(self, module, optimizer):
        self.module, self.optimizer, self.lr_scheduler = module, optimizer, None
        self.checkpoint_engine = U.TorchFileCheckpointEngine()
        self.skipped_steps, self.global_steps, self.global_samples = 1, 7, 56
        self.dp_world_size, self.mp_world_size, self.num_experts = 1, 1, [4]

    def _get_ckpt_name(self, save_dir, tag):
        return f"{save_dir}/{tag}/mp_rank_00_model_states.pt"

    def _get_optimizer_ckpt_name(self, save_dir, tag, ep_rank):
        return f"{save_dir}/{tag}/expp_rank_{ep_rank}_mp_rank_00_optim_states.pt"

    def zero_optimization(self):
        return False

    def module_state_dict(self, exclude_frozen_parameters=False):
        return self.module.state_dict()


def test_checkpoint_files_round_trip(tmp_path):
    torch.manual_seed(0)
    m = _model()
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn_like(p))
    opt = torch.optim.SGD(m.parameters(), lr=0.1, momentum=0.9)
    eng = _FakeEngine(m, opt)
    U.amoe_save_checkpoint(eng, str(tmp_path), "step7", client_state={"epoch": 3})
    tag_dir = tmp_path / "step7"
    assert sorted(p.name for p in tag_dir.iterdir()) == [
        "ep_rank_0_moe_layer_0_model_states.pt", "ep_rank_0_moe_layer_1_model_states.pt",
        "expp_rank_0_mp_rank_00_optim_states.pt", "mp_rank_00_model_states.pt",
    ]
    assert eng._curr_ckpt_path == str(tag_dir)
    main = torch.load(tag_dir / "mp_rank_00_model_states.pt", weights_only=True)
    assert main["global_steps"] == 7 and main["epoch"] == 3 and main["num_experts"] == [4]
    # the main file holds the dense parameters only; each layer file holds that layer's ArcticMoE
    assert set(main["module"]) == {"embed.weight", "layers.0.attn.weight", "layers.0.attn.bias",
                                   "layers.1.attn.weight", "layers.1.attn.bias"}
    layer1 = torch.load(tag_dir / "ep_rank_0_moe_layer_1_model_states.pt", weights_only=True)
    assert set(layer1) == {"layers.1.mlp.router_gate", "layers.1.mlp.expert_gate_up", "layers.1.mlp.expert_down"}
    # a file holds its own tensors only, not the storage they were views of
    assert all(t.untyped_storage().nbytes() == t.numel() * t.element_size() for t in layer1.values())

    fresh = _model()
    state = dict(main["module"])
    U.amoe_load_state_dict(str(tmp_path), "step7", state, old_moe_load=False, model=fresh, device="cpu")
    assert set(state) == set(m.state_dict())
    fresh.load_state_dict(state)
    for (n, a), (_, b) in zip(m.named_parameters(), fresh.named_parameters()):
        assert torch.equal(a, b), n


def test_monkey_patch_needs_deepspeed():
    import importlib.util

    import pytest

    if importlib.util.find_spec("deepspeed") is None:
        with pytest.raises(ImportError, match="DeepSpeed"):
            U.monkey_patch_ds_moe()
    else:
        U.monkey_patch_ds_moe()
        from deepspeed.runtime.engine import DeepSpeedEngine

        assert DeepSpeedEngine._save_moe_checkpoint is U.amoe_save_checkpoint


def test_layer_with_no_tokens_returns_empty_and_zero_gradients():
    """An empty batch launches nothing (so it runs without a GPU): empty output of the input's
    shape, zero gradients for every parameter (what moe.py:219-323 yields for zero tokens)."""
    m = _model(1).layers[0].mlp
    with torch.no_grad():
        for p in m.parameters():
            p.fill_(0.5)
    x = torch.zeros(2, 0, 16, requires_grad=True)
    y = m(x)
    assert y.shape == (2, 0, 16) and y.dtype == x.dtype
    y.sum().backward()
    for n, p in m.named_parameters():
        assert p.grad is not None and not p.grad.any(), n


def test_layer_needs_the_hip_library_for_real_work():
    """There is no CPU fallback: tokens on a CPU tensor are refused, loudly."""
    import pytest

    m = _model(1).layers[0].mlp
    with pytest.raises(RuntimeError):
        m(torch.zeros(4, 16))
