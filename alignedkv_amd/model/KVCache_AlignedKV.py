"""Counterpart of the reference's model/KVCache_AlignedKV.py: one cache object for all layers that
computes attention itself (auto_compute), prefill dense and decode through the split-plane ops."""
from __future__ import annotations

import math
from typing import List, Optional

import torch
import torch.nn.functional as F

from ..extension._plane_cache import column_block
from ..extension.k_cache_file import K_Cache_Class
from ..extension.KV_cache_cpp_extention import _stream_ptr, cuda_module
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
                 literal_colmax: bool = True, literal_broadcast: bool = False, k_block: int = 64) -> None:
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
                                                self.head_dim, idx, device, register, literal_colmax, k_block))
            self.value_cache.append(V_Cache_Class(max_batch_size, self.max_cache_len, self.num_key_value_heads,
                                                  self.head_dim, idx, device, register, 32, literal_colmax,
                                                  literal_broadcast))
        self.reference = False   # True: every plane is read (dense-in-planes baseline), model/KVCache_AlignedKV.py:46
        # True: a decode step is one call of the fused HIP step (4 launches); False: the reference's sequence
        # of ops and framework kernels (K op -> mask -> softmax -> probe op -> V op), kept for A/B checks.
        self.fused = self.head_dim in (64, 128, 256)
        self.literal_broadcast = literal_broadcast
        # False: the fused step may leave the probabilities' record in memory (`_probs`) unwritten where it keeps them on
        # chip (AKV_STEP_NO_PROBS_RECORD); nothing of the reference's API reads them
        self.record_probabilities = True
        self._device = device
        # fp16 scratch rows of the fused step, one pair per stream: steps issued on different streams may overlap
        # (all layers of one stream share a pair, their steps are ordered)
        self._score_buffers = {}
        self._prepared = {}

    def _buffers(self, device=None):
        device = self._device if device is None else device
        return self._score_buffers.get(_stream_ptr(device), (None, None))

    @property
    def _scores(self):
        """fp16 scores [B, H, width] the fused step last wrote on the current stream (debug output)."""
        return self._buffers()[0]

    @property
    def _probs(self):
        """fp16 probabilities [B, H, width] the fused step last wrote on the current stream (debug output; with
        record_probabilities = False a step that keeps them on chip leaves this unwritten)."""
        return self._buffers()[1]

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

    def _fused_mask(self, mask, width: int):
        """[B|1, 1, 1, width] additive mask -> 2-d uint8 view, or False if the fused step cannot take it."""
        if mask is None:
            return None
        if mask.dim() != 4 or mask.shape[1] != 1 or mask.shape[2] != 1 or mask.shape[-1] < width:
            return False
        if mask.dtype != torch.half or mask.shape[0] not in (1, self.max_batch_size):
            return False
        return mask.reshape(mask.shape[0], mask.shape[-1]).contiguous().view(torch.uint8)

    def _prepared_step(self, layer_id: int, device):
        """The fused step of a layer with its per-layer arguments checked once (PreparedDecodeStep); prepared again
        when a rest buffer or a column-maximum tensor was replaced (the unfused path and a prefill do that) or the
        current stream changed."""
        kc, vc = self.key_cache[layer_id], self.value_cache[layer_id]
        key = (kc._rest.data_ptr(), vc._rest.data_ptr(), kc._colmax.data_ptr(), vc._colmax.data_ptr(), _stream_ptr(device))
        st = self._prepared.get(layer_id)
        if st is None or st.key != key:
            B, H = self.max_batch_size, self.num_key_value_heads
            scores, probs = self._buffers(device)
            if scores is None:
                width = (kc.n_max_blocks + 1) * column_block
                scores = torch.empty((B, H, width), dtype=torch.half, device=device)
                probs = torch.empty((B, H, width), dtype=torch.half, device=device)
                self._score_buffers[_stream_ptr(device)] = (scores, probs)
            st = cuda_module.prepare_decode_step(
                (kc.k_cache_first_8, kc.k_cache_mid_4, kc.k_cache_last_4),
                (vc.v_cache_first_8, vc.v_cache_mid_4, vc.v_cache_last_4),
                kc._colmax, vc._colmax, kc._rest.view(torch.uint8), vc._rest.view(torch.uint8),
                scores.view(torch.uint8), probs.view(torch.uint8), B, H, kc.k_n_max_blocks,
                self.max_cache_len, self.head_dim, column_block, kc.k_block, vc.top_max_k, key=key)
            self._prepared[layer_id] = st
        return st

    def decoding_fused(self, q, k, v, start_pos: int, mask2d, layer_id: int):
        """One decode step through akv_decode_step_gqa; same state transitions as decoding_k + decoding_v."""
        kc, vc = self.key_cache[layer_id], self.value_cache[layer_id]
        kc._check_save(k, start_pos, 1, "new_k")
        vc._check_save(v, start_pos, 1, "new_v")
        assert tuple(q.shape) == tuple(k.shape), f"q.shape: {tuple(q.shape)} != {tuple(k.shape)}"
        assert kc.reststartpos + kc._restlen == start_pos
        step = self._prepared_step(layer_id, q.device)
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        out = torch.empty_like(q)
        klv = vlv = amin = None
        if kc.record_levels or vc.record_levels:
            B, H, D = self.max_batch_size, self.num_key_value_heads, self.head_dim
            flushed = kc.reststartpos + (column_block if kc._restlen + 1 == column_block else 0)
            klv = torch.empty((B, H, D), dtype=torch.uint8, device=q.device)
            vlv = torch.empty((B, H, flushed), dtype=torch.uint8, device=q.device) if flushed else None
            amin = torch.empty((B, H), dtype=torch.uint8, device=q.device)
        mask_stride = 0
        if mask2d is not None:
            if mask2d.shape[1] < 2 * (start_pos + 1):
                raise RuntimeError(f"mask: shape {tuple(mask2d.shape)} does not cover {start_pos + 1} halves")
            mask_stride = 0 if mask2d.shape[0] == 1 else mask2d.stride(0) // 2
        # (the step takes the fp16 tensors as they are: it reads their bytes)
        if q.device.index != torch.cuda.current_device():
            with torch.cuda.device(q.device):
                step(q, k, v, out, mask2d, mask_stride, start_pos, self.reference, self.literal_broadcast, klv, vlv, amin,
                     self.record_probabilities)
        else:
            step(q, k, v, out, mask2d, mask_stride, start_pos, self.reference, self.literal_broadcast, klv, vlv, amin,
                 self.record_probabilities)
        kc._advance_after_fused_step()
        vc._advance_after_fused_step()
        if klv is not None:
            kc.last_levels, vc.last_levels, vc.last_alignment_min = klv, vlv, amin
        return out

    def decoding(self, q, k, v, start_pos: int, seqlen: int, mask, layer_id: int):
        if self.fused and seqlen == 1:
            mask2d = self._fused_mask(mask, start_pos + seqlen)
            if mask2d is not False:
                return self.decoding_fused(q, k, v, start_pos, mask2d, layer_id)
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
