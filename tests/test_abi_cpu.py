"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the
header declares, the ctypes table mirrors the header, and argument errors are rejected
before any HIP call (so they are testable without a GPU)."""
import ctypes
import os
import re

import pytest

from arctictraining_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "arctic_moe_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(amoe_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from arctictraining_amd.build import build

        build()
    return _lib.load()


def test_header_symbols_exported(lib):
    names = _declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"


def test_ctypes_table_matches_header():
    assert sorted(_lib.SIGNATURES) == _declared_symbols()


def test_version_and_error_string(lib):
    assert lib.amoe_version() >= 100
    assert isinstance(lib.amoe_last_error(), bytes)


def test_workspace_queries(lib):
    assert lib.amoe_permute_workspace_bytes(131072, 128) >= (131072 // 512) * 128 * 4
    assert lib.amoe_grouped_gemm_workspace_bytes(131072, 128) >= 16 * (131072 // 256 + 128)
    assert lib.amoe_permute_workspace_bytes(0, 8) == 0


P = 0x1000  # a non-null fake pointer: validation must fail before it is ever dereferenced


def test_router_argument_errors(lib):
    assert lib.amoe_router_topk_fwd(None, 1, 4, 8, 2, 1, P, P, P, None) == -1
    assert b"null" in lib.amoe_last_error()
    assert lib.amoe_router_topk_fwd(P, 7, 4, 8, 2, 1, P, P, P, None) == -1  # bad dtype
    assert lib.amoe_router_topk_fwd(P, 1, 0, 8, 2, 1, P, P, P, None) == -1  # T = 0
    assert lib.amoe_router_topk_fwd(P, 1, 4, 1024, 2, 1, P, P, P, None) == -2  # E too large
    assert b"exceeds" in lib.amoe_last_error()
    assert lib.amoe_router_topk_fwd(P, 1, 4, 8, 9, 1, P, P, P, None) == -2  # K > E
    assert lib.amoe_router_topk_fwd(P, 1, 4, 64, 32, 1, P, P, P, None) == -2  # K > 16
    assert lib.amoe_router_bwd(P, P, P, None, 1, 4, 8, 2, 1, 0.0, P, None) == -1


def test_permute_argument_errors(lib):
    assert lib.amoe_permute_plan(P, None, 4, 2, 8, P, P, P, P, P, None, None, 0, None) == -1
    assert lib.amoe_permute_plan(P, None, 4, 2, 8, P, P, P, P, P, P, P, 0, None) == -1  # scores_perm without scores
    assert lib.amoe_permute_plan(P, None, 4, 2, 8, P, P, P, P, P, None, P, 0, None) == -3  # workspace too small
    assert b"workspace" in lib.amoe_last_error()
    assert lib.amoe_permute_plan(P, None, 1 << 20, 4096, 8, P, P, P, P, P, None, P, 1 << 30, None) == -2  # R >= 2^31
    assert lib.amoe_permute_plan(P, None, 4, 2, 600, P, P, P, P, P, None, P, 1 << 20, None) == -2


def test_permute_tiled_argument_errors(lib):
    f = lib.amoe_permute_plan_tiled
    big = 1 << 20
    assert f(P, None, 4, 2, 8, P, P, P, P, P, None, P, big, None, big, 1, 0, None) == -1   # no GEMM workspace
    assert f(P, None, 4, 2, 8, P, P, P, P, P, None, P, big, P, 8, 1, 0, None) == -3        # GEMM workspace too small
    assert f(P, None, 4, 2, 8, P, P, P, P, P, None, P, big, P, big, 5, 0, None) == -1      # dtype
    assert f(P, None, 4, 2, 8, P, P, P, P, P, None, P, big, P, big, 1, 4, None) == -1      # tile_cfg
    assert f(P, None, 4, 2, 8, P, P, P, P, P, None, P, 0, P, big, 1, 0, None) == -3        # plan workspace too small


def test_permute_static_argument_errors(lib):
    assert lib.amoe_permute_plan_static(None, None, 4, 2, 8, P, P, P, P, P, None, None) == -1
    assert lib.amoe_permute_plan_static(P, None, 4, 2, 8, P, P, P, P, P, P, None) == -1  # scores_perm without scores
    assert lib.amoe_permute_plan_static(P, None, 4, 2, 600, P, P, P, P, P, None, None) == -2  # E too large
    # ceil(T*K/512) * E beyond the built-in scratch of 2^20 counters: rejected before any HIP call
    assert lib.amoe_permute_plan_static(P, None, 1 << 20, 2, 512, P, P, P, P, P, None, None) == -2
    assert b"scratch" in lib.amoe_last_error()


def test_row_kernel_argument_errors(lib):
    assert lib.amoe_gather_rows_fwd(P, P, P, 1, 8, 12, None) == -2  # bf16 row not a multiple of 8
    assert lib.amoe_gather_rows_fwd(P, P, P, 0, 8, 6, None) == -2  # f32 row not a multiple of 4
    assert lib.amoe_gather_rows_fwd(P, None, P, 1, 8, 16, None) == -1
    assert lib.amoe_combine_fwd(P, P, P, P, 1, 4, 17, 64, None) == -2  # K > 16
    assert lib.amoe_combine_bwd(P, P, P, P, None, None, 1, 4, 2, 64, None) == -1  # d_scores is required
    assert lib.amoe_gather_rows_bwd(P, P, None, P, 1, 0, 2, 64, None) == -1
    assert lib.amoe_gated_act_bwd(P, P, None, None, P, None, 1, 4, 64, 0, 0, 9, None) == -1  # bad activation
    assert lib.amoe_gated_act_bwd(P, P, P, None, P, P, 1, 4, 64, 2, 2, 0, None) == -1  # d_row_scale needs slot_of
    assert lib.amoe_gated_act_bwd(P, P, P, P, P, P, 1, 4, 64, 3, 2, 0, None) == -1  # T*K != R


def test_gemm_argument_errors(lib):
    big = 1 << 20
    # bf16 reduction length must be a multiple of 32
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 48, 64, P, big, 0, None) == -2
    assert b"multiple of 32" in lib.amoe_last_error()
    assert lib.amoe_grouped_gemm_nt(P, None, P, P, P, 1, 128, 4, 64, 48, P, big, 0, None) == -2
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 64, 64, P, 8, 0, None) == -3  # workspace
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 64, 64, P, big, 9, None) == -1  # tile_cfg
    assert lib.amoe_grouped_gemm_nn(P, None, None, P, P, 1, 128, 4, 64, 64, P, big, 0, None) == -1
    assert lib.amoe_grouped_gemm_wgrad(P, None, P, None, P, P, 1, 128, 4, 60, 64, 0, None) == -2
    assert lib.amoe_grouped_gemm_wgrad(P, None, P, None, P, P, 0, 128, 1000, 64, 64, 0, None) == -2  # E too large
    assert lib.amoe_grouped_gemm_wgrad(P, P, P, P, P, P, 1, 128, 4, 64, 64, 0, None) == -2  # both operands gathered
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 64, 64, P, big, 4, None) == -1  # retired tile_cfg
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 64, 64, P, big, 0x100 | 4, None) == -1  # flag on a bad shape
    assert lib.amoe_grouped_gemm_nn(P, None, P, P, P, 1, 128, 4, 64, 64, P, big, 0x200, None) == -1  # unknown flag
    assert lib.amoe_grouped_gemm_gateup_act_fwd(P, None, P, P, None, P, P, 1, 128, 4, 64, 64, 7, P, big, 0, None) == -1
    assert lib.amoe_grouped_gemm_gateup_act_fwd(P, None, P, P, None, None, P, 0, 128, 4, 64, 64, 0, P, big, 0, None) == -2


def test_gated_bwd_gemm_argument_errors(lib):
    big = 1 << 20
    f = lib.amoe_grouped_gemm_nt_gated_bwd
    assert f(P, None, P, P, None, None, P, None, 1, 128, 4, 64, 64, 0, P, big, 0, None) == -1  # gate_up is required
    assert f(P, None, P, P, P, None, P, None, 0, 128, 4, 64, 64, 0, P, big, 0, None) == -2  # float32
    assert b"bf16 and float16 only" in lib.amoe_last_error()
    assert f(P, None, P, P, P, None, P, None, 2, 128, 4, 64, 48, 0, P, big, 0, None) == -2  # float16 is accepted up to the shape checks
    assert b"multiple of 32" in lib.amoe_last_error()
    assert f(P, None, P, P, P, None, P, None, 1, 128, 4, 64, 48, 0, P, big, 0, None) == -2  # H not a multiple of 32
    assert f(P, None, P, P, P, None, P, None, 1, 128, 4, 64, 64, 9, P, big, 0, None) == -1  # activation
    assert f(P, None, P, P, P, None, P, None, 1, 128, 4, 64, 64, 0, P, 8, 0, None) == -3  # workspace
    assert lib.amoe_gated_bwd_score_parts(768, 0) == 3 and lib.amoe_gated_bwd_score_parts(768, 1) == 6
    assert lib.amoe_gated_bwd_score_parts(0, 0) == 0
    assert lib.amoe_score_grad_gather(None, 3, P, P, 4, 2, None) == -1
    assert lib.amoe_score_grad_gather(P, 0, P, P, 4, 2, None) == -1


def test_remap_argument_errors(lib):
    assert lib.amoe_remap_pack(None, P, P, 1, 2, 64, 64, 64 * 64, None) == -1
    assert lib.amoe_remap_pack(P, P, P, 5, 2, 64, 64, 64 * 64, None) == -1  # dtype
    assert lib.amoe_remap_pack(P, P, P, 1, 2, 60, 64, 60 * 64, None) == -2  # bf16 extents are multiples of 8
    assert lib.amoe_remap_pack(P, P, P, 0, 2, 62, 64, 62 * 64, None) == -2  # float32: multiples of 4
    assert lib.amoe_remap_pack(P, P, P, 1, 2, 64, 64, 100, None) == -1  # expert stride below I*H
    assert lib.amoe_remap_unpack(P, None, P, 1, 2, 64, 64, 64 * 64, None) == -1
    assert lib.amoe_remap_unpack(P, P, None, 1, 0, 64, 64, 64 * 64, None) == -1  # E


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libarctic_moe_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_cpu_tensor_is_rejected():
    import torch

    from arctictraining_amd import ops

    with pytest.raises(RuntimeError, match="GPU"):
        ops.router_topk_fwd(torch.zeros(4, 8), 2, True)
