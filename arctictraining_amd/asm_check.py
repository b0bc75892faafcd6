"""Static check of compiled gfx950 assembly: LDS reads issued as inline assembly must be
awaited before anything touches their destination registers.

The transposing LDS reads of csrc/gemm_bf16.hip are inline assembly (through the compiler builtin
they force a full drain of the direct-to-LDS loads in flight), so the compiler does not know that
their destination registers are filled asynchronously; the kernel waits for them itself
(`s_waitcnt lgkmcnt(0)`) before the first MFMA that consumes them.  A compiler-inserted register
copy, or a reuse of such a register, between the read and the wait would silently read stale data.
`check_source` compiles a source file to assembly and proves, by a forward data-flow pass over
every kernel's control-flow graph, that no instruction touches a register with such a read still
outstanding, and that no kernel uses scratch memory.  The build runs it on every build; a
violation fails the build.
"""
import os
import re
import shutil
import subprocess

_REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_KERNEL = re.compile(r"^(_Z\w*grouped_gemm_(?:rows|wgrad)_(?:bf16|f16)_kernel\w*):")
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




def check_m0(lines):
    """Every instruction that writes M0 must be followed at once (wait states aside) by the
    direct-to-LDS load that reads it, and every such load preceded by a write: a load scheduled
    between another load's write of M0 and that load would land in the wrong place."""
    bad = []
    instrs = [s for s in lines if not _LABEL.match(s)]
    for i, s in enumerate(instrs):
        op = s.split()[0]
        writes_m0 = op.startswith("s_") and re.match(r"\S+\s+m0\b", s) is not None
        if writes_m0:
            j = i + 1
            while j < len(instrs) and instrs[j].startswith("s_nop"):
                j += 1
            # (one independent vector instruction may serve as the wait state)
            if j < len(instrs) and not instrs[j].startswith("global_load_lds") and j + 1 < len(instrs) and instrs[j][0] == "v":
                j += 1
            if j >= len(instrs) or not instrs[j].startswith("global_load_lds"):
                bad.append(f"write of m0 not followed by its load: {s}")
        if op.startswith("global_load_lds"):
            k = i - 1
            while k >= 0 and (instrs[k].startswith("s_nop") or instrs[k][0] == "v") and i - k <= 2:
                k -= 1
            if k < 0 or re.match(r"s_\S+\s+m0\b", instrs[k]) is None:
                bad.append(f"direct-to-LDS load without a write of m0 right before it: {s}")
    return bad


def check_assembly(asm_text: str, min_kernels: int = 1, require_tr: bool = True):
    """Returns (number of kernels, number of transposing reads); raises RuntimeError on a violation
    (and, unless require_tr is False, when the text holds no transposing read at all)."""
    kernels = _kernels(asm_text.splitlines())
    if len(kernels) < min_kernels:
        raise RuntimeError(f"expected at least {min_kernels} GEMM kernels in the assembly, found {len(kernels)}")
    total_tr = 0
    for name, lines in kernels.items():
        violations, n_tr = check_kernel(lines)
        total_tr += n_tr
        if violations:
            raise RuntimeError(f"{name}: register touched while a transposing LDS read is outstanding: {violations[:5]}")
        # No kernel may touch scratch (private) memory: neither spilled registers nor an index
        # array the compiler could not keep in registers (a select between freshly loaded row
        # indices once became a lookup in a scratch array and cost 5 % of the weight gradients).
        # (only the kernels that write M0 in inline assembly: the compiler tracks its own uses)
        m0 = check_m0(lines) if "grouped_gemm_rows_" in name else []
        if m0:
            raise RuntimeError(f"{name}: {m0[:3]}")
        private = [l.strip() for l in lines if re.match(r"\s*scratch_(load|store)", l)]
        if private:
            raise RuntimeError(f"{name} uses scratch memory: {private[:3]}")
    if total_tr == 0 and require_tr:
        raise RuntimeError("no transposing reads found: the check is looking at the wrong instruction")
    return len(kernels), total_tr


def compile_to_assembly(src: str, out: str, flags) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", src, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc -S failed on {src}:\n{r.stderr}")
    with open(out) as fh:
        return fh.read()
