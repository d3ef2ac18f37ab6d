"""`from extension.k_cache_file import K_Cache_Class` (reference: model/KVCache_AlignedKV.py:12)."""
from alignedkv_amd.extension.k_cache_file import K_Cache_Class, cdiv, column_block  # noqa: F401

__all__ = ["K_Cache_Class", "cdiv", "column_block"]
