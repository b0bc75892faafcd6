"""The static check of the compiled bf16 grouped-GEMM kernels (arctictraining_amd/asm_check.py,
also run by every build): its data-flow pass flags a premature use, and the source in the tree
passes it (no GPU needed)."""
import os
import shutil

import pytest

from arctictraining_amd import asm_check
from arctictraining_amd.asm_check import check_kernel
from arctictraining_amd.build import HIPCC_FLAGS, SRC_DIR


def test_checker_flags_a_premature_use():
    bad = ["ds_read_b64_tr_b16 v[4:5], v9 offset:0", "v_mov_b32_e32 v7, v4", "s_waitcnt lgkmcnt(0)", "s_endpgm"]
    good = ["ds_read_b64_tr_b16 v[4:5], v9 offset:0", "s_waitcnt vmcnt(3) lgkmcnt(0)", "v_mov_b32_e32 v7, v4", "s_endpgm"]
    loop = [".LBB0_1:", "s_waitcnt lgkmcnt(0)", "v_mov_b32_e32 v7, v4", "ds_read_b64_tr_b16 v[4:5], v9 offset:0",
            "s_cbranch_scc1 .LBB0_1", "v_mov_b32_e32 v8, v5", "s_endpgm"]
    assert check_kernel(bad)[0]
    assert not check_kernel(good)[0]
    v, n = check_kernel(loop)
    assert n == 1 and len(v) == 1 and "v8, v5" in v[0]   # the use after the loop exit lacks a wait


@pytest.mark.timeout(600)
def test_transposing_reads_are_awaited_before_use(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    # one of the four groups the build compiles (the plain row-grouped products: persistent kernel,
    # K-strided B operand read with the transposing read); the build itself checks all four
    flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-fvisibility=hidden")] + ["-DAMOE_GEMM_PART=1"]
    asm = asm_check.compile_to_assembly(os.path.join(SRC_DIR, "gemm_bf16.hip"), str(tmp_path / "gemm_bf16.s"), flags)
    n_kernels, n_tr = asm_check.check_assembly(asm, min_kernels=10)
    assert n_kernels >= 10 and n_tr > 0
