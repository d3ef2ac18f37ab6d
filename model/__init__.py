"""Import-path alias: `from model.KVCache_AlignedKV import QuantizedCache_AlignedKV` (reference:
model/Llama_AlignedKV.py:14, example.py:3) resolves to alignedkv_amd.model.KVCache_AlignedKV."""
