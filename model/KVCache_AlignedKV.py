"""`from model.KVCache_AlignedKV import QuantizedCache_AlignedKV` (reference: model/Llama_AlignedKV.py:14)."""
from alignedkv_amd.model.KVCache_AlignedKV import QuantizedCache_AlignedKV  # noqa: F401

__all__ = ["QuantizedCache_AlignedKV"]
