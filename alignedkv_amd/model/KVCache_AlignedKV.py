"""Counterpart of the reference's model/KVCache_AlignedKV.py: one cache object for all layers that
computes attention itself (auto_compute), prefill dense and decode through the split-plane ops."""
from __future__ import annotations

import math
from typing import List, Optional

import torch
import torch.nn.functional as F

from ..extension.k_cache_file import K_Cache_Class
from ..extension.v_cache_file import V_Cache_Class

def _cache_base():
    """transformers' Cache when it is the plain base class the reference was written against (4.44);
    newer releases turn max_batch_size / max_cache_len into read-only properties of Cache and want layer
    descriptions in its constructor, none of which this cache uses, so it then stands on its own."""
    try:
        from transformers.cache_utils import Cache
    except Exception:
        return object
    for name in ("max_batch_size", "max_cache_len"):
        if isinstance(getattr(Cache, name, None), property):
            return object
    return Cache


_HFCache = _cache_base()


def _compiling() -> bool:
    try:
        from transformers.utils import is_torchdynamo_compiling
        return bool(is_torchdynamo_compiling())
    except Exception:
        return False


class QuantizedCache_AlignedKV(_HFCache):
    """reference: model/KVCache_AlignedKV.py:18-135.  `config` needs num_hidden_layers,
    num_attention_heads, num_key_value_heads, hidden_size (or head_dim), max_position_embeddings."""

    def __init__(self, config, max_batch_size: int, max_cache_len: Optional[int], device, dtype=None,
                 literal_colmax: bool = True, literal_broadcast: bool = False) -> None:
        try:
            super().__init__()
        except Exception:
            pass   # newer transformers want layer descriptions in Cache.__init__; none of that state is used here
        self.max_batch_size = max_batch_size
        self.max_cache_len = config.max_position_embeddings if max_cache_len is None else max_cache_len
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.dtype = dtype if dtype is not None else torch.float32
        kv = getattr(config, "num_key_value_heads", None)
        self.num_key_value_heads = config.num_attention_heads if kv is None else kv
        assert config.num_attention_heads == self.num_key_value_heads, "We don't support GQA yet."
        register = _compiling()
        self.key_cache: List[K_Cache_Class] = []
        self.value_cache: List[V_Cache_Class] = []
        for idx in range(config.num_hidden_layers):
            self.key_cache.append(K_Cache_Class(max_batch_size, self.max_cache_len, self.num_key_value_heads,
                                                self.head_dim, idx, device, register, literal_colmax))
            self.value_cache.append(V_Cache_Class(max_batch_size, self.max_cache_len, self.num_key_value_heads,
                                                  self.head_dim, idx, device, register, 32, literal_colmax,
                                                  literal_broadcast))
        self.reference = False   # True: every plane is read (dense-in-planes baseline), model/KVCache_AlignedKV.py:46

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        raise Exception("This function is not used in AlignedKV")

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.key_cache[layer_idx].current_cache_len

    def get_max_length(self) -> Optional[int]:
        return self.max_cache_len

    def reset(self):
        for k, v in zip(self.key_cache, self.value_cache):
            k.zerolize()
            v.zerolize()

    # ---- prefill: dense attention on the incoming fp16 tensors, planes written on the side --------------
    def prefill_k(self, q, k, seqlen: int, layer_id: int):
        self.key_cache[layer_id].save(k, 0, seqlen)
        return torch.matmul(q.transpose(1, 2), k.permute(0, 2, 3, 1)) / math.sqrt(self.head_dim)

    def prefill_v(self, scores, v, seqlen: int, layer_id: int):
        self.value_cache[layer_id].save(v, 0, seqlen)
        return torch.matmul(scores, v.transpose(1, 2)).transpose(1, 2).contiguous()

    def prefill(self, q, k, v, seqlen: int, mask, layer_id: int):
        scores = self.prefill_k(q, k, seqlen, layer_id)
        if mask is not None:
            scores = scores + mask
        scores = F.softmax(scores.float(), dim=-1).type_as(q)
        return self.prefill_v(scores, v, seqlen, layer_id)

    # ---- decode: K op -> mask -> fp32 softmax -> V op (model/KVCache_AlignedKV.py:101-124) --------------
    def decoding_k(self, q, k, start_pos: int, seqlen: int, layer_id: int):
        self.key_cache[layer_id].save(k, start_pos, seqlen)
        return self.key_cache[layer_id].decoding_compute(q, start_pos, seqlen, self.reference)

    def decoding_v(self, scores, v, start_pos: int, seqlen: int, layer_id: int):
        self.value_cache[layer_id].save(v, start_pos, seqlen)
        return self.value_cache[layer_id].decoding_compute(scores, start_pos, seqlen, self.reference)

    def decoding(self, q, k, v, start_pos: int, seqlen: int, mask, layer_id: int):
        scores = self.decoding_k(q, k, start_pos, seqlen, layer_id)
        if mask is not None:
            scores[:, :, :, :start_pos + seqlen] += mask
        scores = F.softmax(scores.float(), dim=-1).type_as(q)
        output = self.decoding_v(scores, v, start_pos, seqlen, layer_id)
        return output.view(q.shape[0], q.shape[1], q.shape[2], q.shape[3])

    def auto_compute(self, q, k, v, layer_id: int, mask=None):
        seqlen = q.shape[1]
        start_pos = self.get_seq_length(layer_id)
        if mask is not None:
            mask = mask[:, :, :, :start_pos + seqlen]
        if start_pos == 0:
            return self.prefill(q, k, v, seqlen, mask, layer_id)
        return self.decoding(q, k, v, start_pos, seqlen, mask, layer_id)
