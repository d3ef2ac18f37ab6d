"""Loader of libalignedkv_hip.so.  There is no fallback: without the built library every op raises."""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_float, c_int, c_size_t, c_void_p

_PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_PKG, "csrc")
LIB_PATH = os.environ.get("ALIGNEDKV_LIB", os.path.join(_PKG, "libalignedkv_hip.so"))
HEADER = os.path.join(os.path.dirname(_PKG), "include", "alignedkv.h")

_lib = None

_P = c_void_p
_I = c_int
# name -> (restype, argtypes); mirrors include/alignedkv.h
SIGNATURES = {
    "akv_version": (c_int, []),
    "akv_last_error": (ctypes.c_char_p, []),
    "akv_k_cache_save": (c_int, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "akv_k_cache_compute": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, c_float, _I, _P]),
    "akv_v_cache_save": (c_int, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "akv_v_cache_test_compute": (c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "akv_v_cache_compute_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "akv_v_cache_compute": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, _I, _I, _I, _I, _I, _I, _I, _P]),
    "akv_decode_step_gqa": (c_int, [_P] * 14 + [_I] + [_P] * 3 + [_I, _P, c_size_t] + [_P] * 3 + [_I] * 10 + [_P] + [_I] * 2 + [_P]),
    "akv_dense_decode_step_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "akv_dense_decode_step": (c_int, [_P] * 8 + [_I, _P, c_size_t] + [_I] * 5 + [_P]),
    "akv_reload_tuning": (c_int, []),
    "akv_profile_enable": (c_int, [_I]),
    "akv_copy_probe": (c_int, [_P, _P, c_size_t, _P]),
    "akv_profile_read": (c_int, [_P]),
    "akv_profile_read_empty": (c_int, [_P]),
    "akv_decode_step_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "akv_decode_step": (c_int, [_P] * 14 + [_I] + [_P] * 3 + [_I, _P, c_size_t] + [_P] * 3 + [_I] * 12 + [_P]),
    "akv_decode_step_desc": (c_int, [_P] * 5 + [_I] + [_P] * 4 + [_I, _P, _I, _I, _P]),
    "akv_decode_step_static": (c_int, [_P] * 14 + [_I] + [_P] * 3 + [_I] + [_P] * 3 + [_I] * 12 + [_P]),
}


class StepDesc(ctypes.Structure):
    """akv_step_desc of include/alignedkv.h."""
    _fields_ = ([(n, _P) for n in ("k_first_8", "k_mid_4", "k_last_4", "v_first_8", "v_mid_4", "v_last_4", "k_exp_column_max",
                                   "v_exp_column_max", "restk", "restv", "scores", "probs", "workspace")]
                + [("workspace_bytes", c_size_t)]
                + [(n, _I) for n in ("row_stride", "bsz", "n_q_heads", "n_kv_heads", "n_max_blocks", "max_seq_len", "head_dim",
                                     "d_block", "k_block", "top_max_k")])


def build(verbose: bool = False) -> str:
    """Compile every HIP source of the library for gfx950 (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-B", "-j8", "-C", CSRC]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libalignedkv_hip.so failed (see output above)")
    global _lib
    _lib = None
    return LIB_PATH


def load_library() -> ctypes.CDLL:
    """dlopen the in-tree library and attach the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP library has not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'` in the repository root). "
            "alignedkv_amd has no CPU or PyTorch fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)     # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, lib=None) -> None:
    if rc != 0:
        lib = lib or load_library()
        raise RuntimeError(lib.akv_last_error().decode("utf-8", "replace"))
