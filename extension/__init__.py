"""Import-path alias: the reference's callers import `extension.KV_cache_cpp_extention`, `extension.k_cache_file` and
`extension.v_cache_file` (reference: extension/k_cache_file.py:3, extension/v_cache_file.py:5,
model/KVCache_AlignedKV.py:12-13).  The modules of the same names here re-export the objects of
`alignedkv_amd.extension`, so those import lines work unchanged with this repository's root on sys.path."""
