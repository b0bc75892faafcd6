"""Static check of the compiled bf16 grouped-GEMM kernels (no GPU needed).

The transposing LDS reads of gemm_bf16.hip are issued as inline assembly, so the compiler does
not know that their destination registers are filled asynchronously; the kernel waits for them
itself (`s_waitcnt lgkmcnt(0)`) before the first MFMA that consumes them.  A compiler-inserted
register copy, or a reuse of such a register, between the read and the wait would silently
read stale data.  This test compiles the source to gfx950 assembly and proves, by a forward
data-flow pass over every kernel's control-flow graph, that no instruction touches a register
with such a read still outstanding.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "arctictraining_amd", "csrc", "gemm_bf16.hip")

_REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_KERNEL = re.compile(r"^(_Z\w*grouped_gemm_bf16_kernel\w*):")
_BRANCH = re.compile(r"^\s*(s_cbranch_\w+|s_branch)\s+(\.LBB\d+_\d+)")


def _regs(text):
    out = set()
    for m in _REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def _kernels(asm_lines):
    """name -> list of instruction lines (labels kept) for every GEMM kernel in the file."""
    kernels, cur = {}, None
    for line in asm_lines:
        m = _KERNEL.match(line)
        if m:
            cur = kernels.setdefault(m.group(1), [])
            continue
        if cur is None:
            continue
        s = line.strip()
        if s.startswith(".Lfunc_end"):
            cur = None
            continue
        if not s or s.startswith(";") or (s.startswith(".") and not _LABEL.match(s)):
            continue
        cur.append(s.split(";")[0].strip())
    return kernels


def _blocks(lines):
    """Split into basic blocks: (label or None, instructions, successors)."""
    blocks, cur_label, cur = [], "entry", []
    for s in lines:
        m = _LABEL.match(s)
        if m:
            blocks.append([cur_label, cur, None])
            cur_label, cur = m.group(1), []
            continue
        cur.append(s)
        if _BRANCH.match(s) or s.startswith("s_endpgm"):
            blocks.append([cur_label, cur, None])
            cur_label, cur = None, []
    blocks.append([cur_label, cur, None])
    index = {b[0]: i for i, b in enumerate(blocks) if b[0]}
    for i, b in enumerate(blocks):
        succ = []
        last = b[1][-1] if b[1] else ""
        m = _BRANCH.match(last)
        if m:
            succ.append(index[m.group(2)])
        if not last.startswith("s_branch") and not last.startswith("s_endpgm") and i + 1 < len(blocks):
            succ.append(i + 1)
        b[2] = succ
    return blocks


def _transfer(instrs, pending, violations=None, where=""):
    pending = set(pending)
    for s in instrs:
        op = s.split()[0]
        if op == "s_waitcnt" and "lgkmcnt(0)" in s:
            pending.clear()
            continue
        if op == "s_waitcnt":
            continue
        touched = _regs(s)
        if op == "ds_read_b64_tr_b16":
            dst, _, rest = s[len(op):].partition(",")
            if violations is not None and (_regs(rest) | _regs(dst)) & pending:
                violations.append(f"{where}: {s}")
            pending |= _regs(dst)
            continue
        if violations is not None and touched & pending:
            violations.append(f"{where}: {s}  (outstanding: {sorted(touched & pending)})")
    return pending


def check_kernel(lines):
    blocks = _blocks(lines)
    pend_in = [set() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        i = work.pop()
        out = _transfer(blocks[i][1], pend_in[i])
        for j in blocks[i][2]:
            if not out <= pend_in[j]:
                pend_in[j] |= out
                work.append(j)
    violations = []
    for i, b in enumerate(blocks):
        _transfer(b[1], pend_in[i], violations, b[0] or f"block {i}")
    n_tr = sum(1 for b in blocks for s in b[1] if s.startswith("ds_read_b64_tr_b16"))
    return violations, n_tr


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
    out = tmp_path / "gemm_bf16.s"
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "--cuda-device-only", "-S", SRC, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=580)
    kernels = _kernels(out.read_text().splitlines())
    assert len(kernels) >= 20, f"expected every tile/layout instance, found {len(kernels)}"
    total_tr = 0
    for name, lines in kernels.items():
        violations, n_tr = check_kernel(lines)
        total_tr += n_tr
        assert not violations, f"{name}: {violations[:5]}"
        # No kernel may touch scratch (private) memory: neither spilled registers nor an index
        # array the compiler could not keep in registers (a select between freshly loaded row
        # indices once became a lookup in a scratch array and cost 5 % of the weight gradients).
        private = [l.strip() for l in lines if re.match(r"\s*scratch_(load|store)", l)]
        assert not private, f"{name} uses scratch memory: {private[:3]}"
    assert total_tr > 0, "no transposing reads found: the check is looking at the wrong instruction"
