"""ctypes binding of libflashpop_hip.so (declarations: include/flashpop_hip.h)."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_longlong, c_size_t, c_void_p, POINTER, c_double

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libflashpop_hip.so"
LIB_PATH = os.path.join(_HERE, LIB_NAME)

_P, _I, _Z = c_void_p, c_int, c_size_t
_D = POINTER(c_double)
_L, _F = c_longlong, c_double

# name -> argument types, in the order of include/flashpop_hip.h
SIGNATURES = {
    "fp_retention_fwd": [_P, _P, _P, _P, _D, _P, _P, _I, _I, _I, _I, _I, _P],
    "fp_retention_bwd": [_P, _P, _P, _P, _D, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    "fp_retention_checkpoint_bytes": [_I, _I, _I, _I, _I, POINTER(c_int)],
    "fp_retention_fwd_ckpt": [_P, _P, _P, _P, _D, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "fp_retention_bwd_ckpt": [_P, _P, _P, _P, _D, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    "fp_retention_workspace_bytes": [_I, _I, _I, _I, _I],
    "fp_retention_fwd_split": [_P, _P, _P, _P, _D, _P, _P, _I, _I, _I, _I, _I, _P, _Z, _P],
    "fp_retention_fwd_split_static": [_P, _P, _P, _P, _D, _P, _P, _I, _I, _I, _I, _I, _P],
    "fp_retention_bwd_split": [_P, _P, _P, _P, _D, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _Z, _I, _P],
    "fp_pop_retention_fwd": [_P, _P, _P, _P, _D, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "fp_pop_retention_bwd": [_P, _P, _P, _P, _D, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "fp_pop_fused_fwd": [_P] * 7 + [_D] + [_P] * 3 + [_I] * 7 + [_P],
    "fp_pop_fused_bwd": [_P] * 7 + [_D] + [_P] * 10 + [_I] * 7 + [_P],
    "fp_retention_decode_step": [_P, _P, _P, _P, _D, _P, _P, _I, _I, _I, _I, _P],
    "fp_rotary_qk": [_P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P],
    "fp_gated_group_norm_fwd": [_P, _P, _P, _L, _I, _I, _F, _P],
    "fp_gated_group_norm_bwd": [_P, _P, _P, _P, _P, _L, _I, _I, _F, _P],
    "fp_set_backward_choice": [_I, _I],
    "fp_last_error": [],
    "fp_version": [],
}

_lib = None


def bind(path: str) -> ctypes.CDLL:
    """Open a library exporting the flashpop C ABI and declare its prototypes."""
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.argtypes = argtypes
        fn.restype = {"fp_last_error": c_char_p, "fp_retention_workspace_bytes": c_size_t,
                      "fp_retention_checkpoint_bytes": c_size_t}.get(name, c_int)
    return lib


def load() -> ctypes.CDLL:
    """The HIP library built in-tree.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it first (python flash-pop_amd/build.py, or "
                "__graft_entry__.build()). flash_pop_amd has no non-HIP execution path.")
        _lib = bind(LIB_PATH)
    return _lib


def decays_array(head_decays) -> ctypes.Array:
    vals = [float(g) for g in head_decays]
    return (c_double * len(vals))(*vals)


def check(lib: ctypes.CDLL, rc: int) -> None:
    if rc != 0:
        raise RuntimeError(f"flashpop_hip error {rc}: {lib.fp_last_error().decode()}")
