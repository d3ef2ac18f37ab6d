"""`from extension.KV_cache_cpp_extention import cuda_module` (reference: extension/k_cache_file.py:3,
extension/v_cache_file.py:5): the same object as alignedkv_amd.extension.KV_cache_cpp_extention.cuda_module."""
from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module  # noqa: F401

__all__ = ["cuda_module"]
