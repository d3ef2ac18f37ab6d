"""ctypes front end of oracle/akv_oracle.c (test infrastructure, see that file's header)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libakv_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "akv_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libakv_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.akvo_init()
        _lib.akvo_float_to_half.restype = ctypes.c_uint16
        _lib.akvo_float_to_half.argtypes = [ctypes.c_float]
        _lib.akvo_half_to_float.restype = ctypes.c_float
        _lib.akvo_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.akvo_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a)
    assert a.dtype == dt, (a.dtype, dt)
    return a


def k_cache_save(first_8, mid_4, last_4, k_new_bits, n_blocks, d_block, start_pos, seqlen):
    B, H, NBmax, D, _ = first_8.shape
    kn = _c(k_new_bits, np.uint16)
    for a in (first_8, mid_4, last_4):
        assert a.flags.c_contiguous
    lib().akvo_k_cache_save(_p(first_8), _p(mid_4), _p(last_4), _p(kn), B, H, n_blocks, NBmax, D, d_block,
                            start_pos, seqlen)


def k_cache_compute(first_8, mid_4, last_4, sum_u8, max_u8, q_bits, n_blocks, d_block, sqrt_dim,
                    reference=False):
    B, H, NBmax, D, _ = first_8.shape
    s = np.zeros((B, H, 1, (n_blocks + 1) * d_block), np.uint16)
    lv = np.zeros((B, H, D), np.uint8)
    lib().akvo_k_cache_compute(_p(first_8), _p(mid_4), _p(last_4), _p(_c(sum_u8, np.uint8)),
                               _p(_c(max_u8, np.uint8)), _p(_c(q_bits, np.uint16)), _p(s), _p(lv),
                               B, H, n_blocks, NBmax, D, d_block, ctypes.c_float(sqrt_dim), int(reference))
    return s.view(np.float16), lv


def v_cache_save(first_8, mid_4, last_4, v_new_bits, start_pos, seq_len):
    B, H, Lmax, D = first_8.shape
    vn = _c(v_new_bits, np.uint16)
    lib().akvo_v_cache_save(_p(first_8), _p(mid_4), _p(last_4), _p(vn), B, H, Lmax, D, start_pos, seq_len,
                            vn.shape[1])


def v_cache_test_compute(first_8, test_s_value_bits, test_s_index, top_max_k):
    B, H, Lmax, D = first_8.shape
    o = np.zeros((B, H, 1, D), np.uint16)
    lib().akvo_v_cache_test_compute(_p(first_8), _p(_c(test_s_value_bits, np.uint16)),
                                    _p(_c(test_s_index, np.int32)), _p(o), B, H, Lmax, D, top_max_k)
    return o.view(np.float16)


def v_cache_compute(first_8, mid_4, last_4, s_bits, amin_u8, n_tokens, reference=False):
    B, H, Lmax, D = first_8.shape
    sb = _c(s_bits, np.uint16)
    o = np.zeros((B, H, 1, D), np.uint16)
    lv = np.zeros((B, H, max(n_tokens, 1)), np.uint8)
    lib().akvo_v_cache_compute(_p(first_8), _p(mid_4), _p(last_4), _p(sb), _p(_c(amin_u8, np.uint8)), _p(o),
                               _p(lv), B, H, Lmax, D, sb.shape[-1], n_tokens, int(reference))
    return o.view(np.float16), lv[:, :, :n_tokens]


def dense_attention(q_bits, k_bits, v_bits):
    q = _c(q_bits, np.uint16)
    k = _c(k_bits, np.uint16)
    v = _c(v_bits, np.uint16)
    B, L, H, D = k.shape
    out = np.zeros((B, 1, H, D), np.uint16)
    scratch = np.zeros((B, H, L), np.float32)
    lib().akvo_dense_attention(_p(q), _p(k), _p(v), _p(out), _p(scratch), B, H, L, D)
    return out.view(np.float16)


def num_threads() -> int:
    return int(lib().akvo_num_threads())
