"""Host-side logic of the layer module that needs no GPU."""
import torch

from arctictraining_amd import moe


def test_index_cache_is_bounded():
    """Token counts change from step to step; the cache of split offsets must not grow with
    the number of distinct sizes."""
    cache = moe._INDEX_CACHE
    for T in range(512, 1512):
        offs = moe._token_offsets(T, 16, "cpu")
        assert offs.dtype == torch.int32 and offs[0] == 0 and offs[-1] == T and offs.numel() == 17
        assert bool((offs[1:] >= offs[:-1]).all())
        ids = moe._token_ids(T, "cpu")
        assert ids.numel() == T
    assert len(cache) <= cache.max_entries
    # a hit returns the cached tensor itself
    a = moe._token_offsets(1511, 16, "cpu")
    assert moe._token_offsets(1511, 16, "cpu") is a


def test_activation_classification():
    import torch.nn.functional as F

    from arctictraining_amd import ops

    assert moe.classify_activation(F.silu) == ops.ACT_SILU
    assert moe.classify_activation(F.gelu) == ops.ACT_GELU
    assert moe.classify_activation(F.relu) == ops.ACT_RELU
    assert moe.classify_activation(lambda x: x * torch.sigmoid(1.702 * x)) == ops.ACT_GPT_OSS


def test_layer_without_gate_parameter_shapes():
    """is_gated=False: one plain [E,H,I] projection instead of the interleaved [E,H,2I] pair
    (moe.py:101-106), the shared expert likewise (:118-124)."""
    import torch.nn.functional as F

    from arctictraining_amd import ArcticMoE, MoEConfig

    cfg = MoEConfig(act_fn=F.silu, input_dtype=torch.float32, intermediate_dim=6, model_dim=8, normalize_topk_scores=True,
                    num_experts=4, top_k=2, is_gated=False, use_shared_expert=True)
    m = ArcticMoE(cfg)
    assert tuple(m.expert_gate_up.shape) == (4, 8, 6) and tuple(m.expert_down.shape) == (4, 6, 8)
    assert tuple(m.shared_expert_gate_up.shape) == (8, 6)
    gated = ArcticMoE(MoEConfig(act_fn=F.silu, input_dtype=torch.float32, intermediate_dim=6, model_dim=8,
                                normalize_topk_scores=True, num_experts=4, top_k=2))
    assert tuple(gated.expert_gate_up.shape) == (4, 8, 12)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus above 1 exits with a message and without touching a device."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "ONE GPU" in r.stdout


def test_bench_configurations_are_the_baseline_ones():
    import importlib.util
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert set(bench.CONFIGS) == {"c1", "c2", "c3", "c4", "c5"}
    # (dtype, T, H, E, K, I, extra): the headline configuration of the metric
    assert bench.CONFIGS["c3"][:6] == ("bfloat16", 16384, 2048, 128, 8, 768)
    assert bench.CONFIGS["c1"][:6] == ("float32", 2048, 512, 8, 2, 1024)
