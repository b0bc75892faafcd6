"""Build libarctic_moe_hip.so (gfx950) in-tree with hipcc.

    python -m arctictraining_amd.build [--force]

Replaces the reference's JIT op builder (arctic_training/op_builder/builder.py:351-434,
op_builder/moe_ops.py:75-103): the sources are compiled ahead of time into one C-ABI
shared library that sits next to the package and is loaded with ctypes.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(SRC_DIR, "build")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libarctic_moe_hip.so")

# (source, object name, extra flags); the 16-bit grouped GEMM is compiled as four groups of entry points in parallel
GEMM_PARTS = 4
SOURCES = [(f, os.path.splitext(f)[0], []) for f in ("api.hip", "router.hip", "permute.hip", "rows.hip", "gemm_f32.hip", "remap.hip")]
SOURCES = [("gemm_bf16.hip", f"gemm_bf16_p{i}", [f"-DAMOE_GEMM_PART={i}"]) for i in range(GEMM_PARTS)] + SOURCES

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the expert-layer kernels cannot be built")


def _compile(item) -> str:
    src, name, extra = item
    obj = os.path.join(OBJ_DIR, name + ".o")
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra, "-c", os.path.join(SRC_DIR, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _check_gemm_assembly(part: int):
    """Compile one group of gemm_bf16.hip to assembly and run the static check of its inline-assembly
    LDS reads (asm_check.py); raises, and so fails the build, on a violation.  Returns the numbers of
    kernels and of transposing reads checked."""
    from . import asm_check

    flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-fvisibility=hidden")] + [f"-DAMOE_GEMM_PART={part}"]
    asm = asm_check.compile_to_assembly(os.path.join(SRC_DIR, "gemm_bf16.hip"), os.path.join(OBJ_DIR, f"gemm_bf16_p{part}.s"), flags)
    return asm_check.check_assembly(asm, min_kernels=1, require_tr=False)


STAMP_PATH = os.path.join(LIB_DIR, "build_commit.txt")


def _stamp_commit() -> None:
    """Record which commit the library was built from next to it (the stamp travels with the built
    library to machines that have no git history; measurements quote it).  Two lines: the commit of
    the tree, and the last commit that changed a file under csrc/ (the kernels themselves: a profile
    taken at that commit stays the profile of the library through commits that touch no kernel)."""
    try:
        root = os.path.dirname(PKG_DIR)

        def git(*args):
            r = subprocess.run(["git", "-C", root, *args], capture_output=True, text=True, timeout=10)
            return r.stdout.strip() if r.returncode == 0 else ""

        head = git("rev-parse", "--short=12", "HEAD")
        if not head:
            return
        dirty = git("status", "--porcelain", "--untracked-files=no")
        kernels = git("log", "-1", "--format=%h", "--abbrev=12", "--", "arctictraining_amd/csrc")
        kdirty = git("status", "--porcelain", "--untracked-files=no", "--", "arctictraining_amd/csrc")
        with open(STAMP_PATH, "w") as fh:
            fh.write(head + ("+uncommitted" if dirty else "") + "\n")
            fh.write("kernels " + (kernels or head) + ("+uncommitted" if kdirty else "") + "\n")
    except Exception:
        pass  # no git here: leave whatever stamp came with the tree


def build(force: bool = True, jobs: int = 8) -> str:
    """Compile every HIP source, check the GEMM assembly, and link the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    if not force and os.path.exists(LIB_PATH):
        newest = max(
            os.path.getmtime(os.path.join(root, f))
            for root in (SRC_DIR, os.path.join(PKG_DIR, "..", "include"))
            for f in os.listdir(root)
            if f.endswith((".hip", ".h"))
        )
        if os.path.getmtime(LIB_PATH) >= newest:
            return LIB_PATH
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs_f = [ex.submit(_compile, item) for item in SOURCES]
        checks = [ex.submit(_check_gemm_assembly, i) for i in range(GEMM_PARTS)]
        objs = [f.result() for f in objs_f]
        # a violation raises here: no library is linked from a source that fails the check
        counts = [c.result() for c in checks]
        n_kernels, n_tr = sum(c[0] for c in counts), sum(c[1] for c in counts)
        if n_kernels < 40 or n_tr == 0:
            raise RuntimeError(f"expected at least 40 GEMM kernels with transposing reads in the assembly, found {n_kernels} / {n_tr}")
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    _stamp_commit()
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
