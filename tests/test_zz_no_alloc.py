"""The entry point that allocates nothing (amoe_permute_plan_static) against amoe_permute_plan,
through the C ABI: bit-exact on every output, on two calls in a row, the second with a smaller
input (the library's scratch array keeps the first call's contents)."""
import pytest
import torch

from arctictraining_amd import _lib

pytestmark = pytest.mark.gpu


def _plan(lib, static, assign, scores, E):
    T, K = assign.shape
    R, dev = T * K, assign.device
    i32 = dict(dtype=torch.int32, device=dev)
    # outputs pre-filled so that an entry the kernels skip shows up
    outs = [torch.full((E,), -7, **i32), torch.full((E + 1,), -7, **i32), torch.full((R,), -7, **i32),
            torch.full((R,), -7, **i32), torch.full((T, K), -7, **i32), torch.full((R,), -7.0, device=dev)]
    stream = torch.cuda.current_stream().cuda_stream
    args = [assign.data_ptr(), scores.data_ptr(), T, K, E] + [o.data_ptr() for o in outs]
    if static:
        rc = lib.amoe_permute_plan_static(*args, stream)
    else:
        ws = torch.empty(max(lib.amoe_permute_workspace_bytes(R, E), 16), dtype=torch.uint8, device=dev)
        rc = lib.amoe_permute_plan(*args, ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc, "permute_plan")
    torch.cuda.synchronize()
    return outs


def test_permute_plan_static_matches_workspace_variant(gpu_device):
    lib = _lib.load()
    g = torch.Generator().manual_seed(77)
    # the second call is smaller in every dimension: stale counters of the first must not leak
    for T, K, E in ((16384, 8, 128), (1000, 3, 60)):
        print("permute_plan_static", T, K, E, flush=True)
        assign = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
        assign[assign == 5] = 6  # an empty expert
        scores = torch.rand(T, K, generator=g)
        a, s = assign.to(gpu_device), scores.to(gpu_device)
        ref = _plan(lib, False, a, s, E)
        got = _plan(lib, True, a, s, E)
        for name, r, o in zip(("counts", "offsets", "token_of", "slot_of", "row_of", "scores_perm"), ref, got):
            assert torch.equal(r, o), name
        assert int(ref[0].sum()) == T * K and int(ref[0][5]) == 0


def test_permute_plan_static_allocates_nothing_and_runs_under_capture(gpu_device):
    """What the entry point is for: a call leaves the device's free memory unchanged, and a call recorded
    into a HIP graph (after one eager warm-up call) replays to the same plan as the workspace variant."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    T, K, E = 4096, 4, 32
    assign = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32).to(gpu_device)
    scores = torch.rand(T, K, generator=g).to(gpu_device)
    R = T * K
    i32 = dict(dtype=torch.int32, device=gpu_device)
    outs = [torch.full((E,), -7, **i32), torch.full((E + 1,), -7, **i32), torch.full((R,), -7, **i32),
            torch.full((R,), -7, **i32), torch.full((T, K), -7, **i32), torch.full((R,), -7.0, device=gpu_device)]
    args = [assign.data_ptr(), scores.data_ptr(), T, K, E] + [o.data_ptr() for o in outs]

    def call(stream):
        _lib.check(lib.amoe_permute_plan_static(*args, stream), "permute_plan_static")

    call(torch.cuda.current_stream().cuda_stream)   # warm-up: the scratch address is looked up on the first call
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "the call changed the device's free memory"
    ref = _plan(lib, False, assign, scores, E)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        for o in outs:
            o.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        for name, r, o in zip(("counts", "offsets", "token_of", "slot_of", "row_of", "scores_perm"), ref, outs):
            assert torch.equal(r, o), f"{name}, replay {rep}"


def test_permute_plan_static_rejects_oversize(gpu_device):
    lib = _lib.load()
    p = torch.empty(16, dtype=torch.int32, device=gpu_device).data_ptr()
    assert lib.amoe_permute_plan_static(p, None, 1 << 20, 2, 512, p, p, p, p, p, None, None) == -2
    assert b"scratch" in lib.amoe_last_error()
