"""ctypes binding of libarctic_moe_hip.so (the C ABI declared in include/arctic_moe_hip.h).

The library is the product path: there is no fallback.  If it has not been built, or an
entry point reports an error, a RuntimeError is raised.
"""
import ctypes
import os
import threading

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "lib", "libarctic_moe_hip.so")

_c_int = ctypes.c_int
_c_void_p = ctypes.c_void_p
_c_size_t = ctypes.c_size_t
_c_float = ctypes.c_float

# name -> (restype, argtypes); mirrors include/arctic_moe_hip.h one to one
SIGNATURES = {
    "amoe_version": (_c_int, []),
    "amoe_last_error": (ctypes.c_char_p, []),
    "amoe_router_topk_fwd": (_c_int, [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "amoe_router_bwd": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_void_p, _c_void_p],
    ),
    "amoe_permute_workspace_bytes": (_c_size_t, [_c_int, _c_int]),
    "amoe_permute_plan": (
        _c_int,
        [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
         _c_void_p, _c_size_t, _c_void_p],
    ),
    "amoe_permute_plan_tiled": (
        _c_int,
        [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
         _c_void_p, _c_size_t, _c_void_p, _c_size_t, _c_int, _c_int, _c_void_p],
    ),
    "amoe_permute_plan_static": (
        _c_int,
        [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
         _c_void_p],
    ),
    "amoe_gather_rows_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p]),
    "amoe_gather_rows_bwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p]),
    "amoe_combine_fwd": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p]),
    "amoe_combine_bwd": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    ),
    "amoe_grouped_gemm_workspace_bytes": (_c_size_t, [_c_int, _c_int]),
    "amoe_grouped_gemm_gateup_act_fwd": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_void_p, _c_size_t, _c_int, _c_void_p],
    ),
    "amoe_grouped_gemm_nn": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_size_t,
         _c_int, _c_void_p],
    ),
    "amoe_grouped_gemm_nt": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_size_t,
         _c_int, _c_void_p],
    ),
    "amoe_grouped_gemm_wgrad": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_void_p],
    ),
    "amoe_gated_bwd_score_parts": (_c_int, [_c_int, _c_int]),
    "amoe_grouped_gemm_nt_gated_bwd": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_void_p, _c_size_t, _c_int, _c_void_p],
    ),
    "amoe_score_grad_gather": (_c_int, [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p]),
    "amoe_remap_pack": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, ctypes.c_longlong, _c_void_p],
    ),
    "amoe_remap_unpack": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, ctypes.c_longlong, _c_void_p],
    ),
    "amoe_gated_act_bwd": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_void_p],
    ),
}

_lib = None
_lock = threading.Lock()


def load():
    """Load the shared library once and attach the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m arctictraining_amd.build` "
                "(the expert layer has no fallback implementation)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a negative return code into a RuntimeError carrying the library's message
    (the reference surfaces TORCH_CHECK failures the same way, top_k_gating.cpp:40-62)."""
    if rc != 0:
        msg = load().amoe_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")
