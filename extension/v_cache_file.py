"""`from extension.v_cache_file import V_Cache_Class` (reference: model/KVCache_AlignedKV.py:13)."""
from alignedkv_amd.extension.v_cache_file import V_Cache_Class, cdiv, column_block  # noqa: F401

__all__ = ["V_Cache_Class", "cdiv", "column_block"]
