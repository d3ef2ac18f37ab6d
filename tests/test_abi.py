"""CPU-only checks of the C ABI: the in-tree library loads, exports every symbol that
include/alignedkv.h declares, and rejects bad arguments before touching the GPU."""
import ctypes
import os
import re

import pytest

import alignedkv_amd
from alignedkv_amd import _lib


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        alignedkv_amd.build()
    return alignedkv_amd.load_library()


def declared_symbols():
    text = open(_lib.HEADER).read()
    return sorted(set(re.findall(r"AKV_API\s+[\w\s\*]+?\b(akv_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(lib):
    names = declared_symbols()
    assert len(names) >= 14 and "akv_k_cache_compute" in names and "akv_decode_step" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes prototype"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.akv_version() >= 100


def test_null_and_shape_errors_are_reported_without_a_launch(lib):
    z = ctypes.c_void_p(0)
    assert lib.akv_k_cache_save(z, z, z, z, 1, 1, 1, 1, 128, 64, 0, 64, z) == 1
    assert b"null pointer" in lib.akv_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.akv_k_cache_save(p, p, p, p, 1, 1, 1, 1, 128, 60, 0, 64, z) == 1
    assert b"d_block" in lib.akv_last_error()
    assert lib.akv_v_cache_save(p, p, p, p, 1, 1, 16, 128, 8, 16, 16, z) == 1
    assert b"outside the plane" in lib.akv_last_error()
    assert lib.akv_v_cache_compute(p, p, p, p, p, p, z, z, 0, 1, 1, 16, 128, 16, 16, 0, z) == 1
    assert b"workspace" in lib.akv_last_error()
    assert lib.akv_decode_step(*([p] * 14), 0, p, p, p, 64, p, 1 << 30, z, z, z, 1, 1, 1, 64, 96, 64, 32, 0, 0, 0, 0, 0, z) == 1
    assert b"head_dim 96" in lib.akv_last_error()
    assert lib.akv_v_cache_compute_workspace_bytes(8, 32, 128, 4096) >= 8 * 32 * 128 * 4
    assert lib.akv_v_cache_compute_workspace_bytes(0, 32, 128, 4096) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load_library()


def test_reference_import_paths_resolve_to_this_library():
    """The import lines of the reference's callers (extension/k_cache_file.py:3, extension/v_cache_file.py:5,
    model/KVCache_AlignedKV.py:10-11, model/Llama_AlignedKV.py:14, example.py:4) work unchanged and give the same objects."""
    from extension.KV_cache_cpp_extention import cuda_module
    from extension.k_cache_file import K_Cache_Class
    from extension.v_cache_file import V_Cache_Class
    from model.KVCache_AlignedKV import QuantizedCache_AlignedKV
    import alignedkv_amd.extension.KV_cache_cpp_extention as impl
    import alignedkv_amd.extension.k_cache_file as kimpl
    import alignedkv_amd.extension.v_cache_file as vimpl
    import alignedkv_amd.model.KVCache_AlignedKV as cimpl
    assert cuda_module is impl.cuda_module
    assert K_Cache_Class is kimpl.K_Cache_Class and V_Cache_Class is vimpl.V_Cache_Class
    assert QuantizedCache_AlignedKV is cimpl.QuantizedCache_AlignedKV
    # the five ops of the reference's binding (extension/csrc/KV_cache_ops.cpp:69-75)
    for op in ("k_cache_save", "k_cache_compute", "v_cache_save", "v_cache_test_compute", "v_cache_compute"):
        assert callable(getattr(cuda_module, op))
    import extension.k_cache_file as kf
    assert kf.column_block == 64 and kf.cdiv(65, 64) == 2
