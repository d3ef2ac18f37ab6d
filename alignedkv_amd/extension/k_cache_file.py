"""K half of the host hot path: counterpart of the reference's extension/k_cache_file.py
(K_Cache_Class: planes :45-55, save :69-118, decoding_compute :132-159) on top of the HIP ops."""
from __future__ import annotations

import math

import torch

from ._plane_cache import PlaneCacheBase, cdiv, column_block, exponent_bits
from .KV_cache_cpp_extention import cuda_module


class K_Cache_Class(PlaneCacheBase):
    def __init__(self, bsz: int, max_seq_len: int, n_local_kv_heads: int, head_dim: int, layer_idx: int,
                 device="cuda:0", register_buffer: bool = False, literal_colmax: bool = True, k_block: int = column_block):
        super().__init__(bsz, max_seq_len, n_local_kv_heads, head_dim, device, literal_colmax)
        # k_block: tokens per block of the planes (the ops' d_block).  The reference uses column_block = 64 for the
        # planes and for the flush unit alike; with 256 a channel's nibble row of a block is a whole 128-byte line
        # (a skipped row then saves exactly its bytes of HBM traffic) while tokens still arrive 64 at a time.
        assert k_block % column_block == 0, f"k_block {k_block} must be a multiple of {column_block}"
        self.k_block = k_block
        nb = self.k_n_max_blocks = cdiv(max_seq_len, k_block)
        # [bsz, heads, blocks, head_dim, slot]: the sequence is innermost within a block
        self.k_cache_first_8 = self._alloc(f"k_cache_first_8_layer_{layer_idx}",
                                           (bsz, n_local_kv_heads, nb, head_dim, k_block), register_buffer)
        self.k_cache_mid_4 = self._alloc(f"k_cache_mid_4_layer_{layer_idx}",
                                         (bsz, n_local_kv_heads, nb, head_dim, k_block // 2), register_buffer)
        self.k_cache_last_4 = self._alloc(f"k_cache_last_4_layer_{layer_idx}",
                                          (bsz, n_local_kv_heads, nb, head_dim, k_block // 2), register_buffer)
        self._colmax = torch.zeros((bsz, 1, n_local_kv_heads, head_dim), dtype=torch.uint8, device=device)
        self.last_levels = None     # uint8 [bsz, heads, head_dim] of the last decoding_compute when record_levels
        self.last_scores = None     # fp16 copy of the scores it returned (debug record, with record_levels)
        self.record_levels = False

    # names the reference exposes
    @property
    def k_cache_exp_column_max(self):
        return self._colmax

    @k_cache_exp_column_max.setter
    def k_cache_exp_column_max(self, t):
        self._colmax = t

    @property
    def restk(self):
        return self._rest

    @property
    def restklen(self):
        return self._restlen

    def zerolize(self):
        self.k_cache_first_8.zero_()
        self.k_cache_mid_4.zero_()
        self.k_cache_last_4.zero_()
        self._colmax = torch.zeros_like(self._colmax)
        self._zero_state()

    def _store_planes(self, tokens: torch.Tensor, start_pos: int, n_tokens: int):
        if self.k_block == column_block:
            seqlen = tokens.shape[1]
            cuda_module.k_cache_save(self.k_cache_first_8, self.k_cache_mid_4, self.k_cache_last_4,
                                     tokens.view(torch.uint8), self.bsz, self.n_local_kv_heads, n_tokens // column_block,
                                     self.n_max_blocks, self.head_dim, column_block, start_pos, seqlen)
        elif n_tokens:
            # whole 64-token tiles, possibly ending inside a block: exactly the tokens that leave the rest buffer
            tokens = tokens[:, :n_tokens].contiguous()
            cuda_module.k_cache_save(self.k_cache_first_8, self.k_cache_mid_4, self.k_cache_last_4,
                                     tokens.view(torch.uint8), self.bsz, self.n_local_kv_heads, cdiv(n_tokens, self.k_block),
                                     self.k_n_max_blocks, self.head_dim, self.k_block, start_pos, n_tokens)

    def save(self, new_k: torch.Tensor, start_pos: int, seqlen: int):
        self._save(new_k, start_pos, seqlen, "new_k")

    def decoding_compute(self, q: torch.Tensor, start_pos: int, seqlen: int, reference: bool = False):
        """Scaled scores of one decode token against the whole cache: planes through the HIP op,
        the unflushed tail by an fp16 matmul, -inf beyond the valid length.  Returns fp16
        [bsz, heads, 1, (flushed_blocks + 1) * 64]."""
        assert q.shape[2] == self.n_local_kv_heads, "we currently only support MHA, don't support GQA"
        want = (self.bsz, seqlen, self.n_local_kv_heads, self.head_dim)
        assert tuple(q.shape) == want, f"q.shape: {tuple(q.shape)} != {want}"
        assert self._restlen + self.reststartpos == start_pos + seqlen
        q = q.contiguous()
        exp_sum = exponent_bits(q) + self._colmax                       # <= 62, fits uint8
        exp_sum_max = torch.max(exp_sum, dim=3, keepdim=True).values
        levels = None
        if self.record_levels:
            levels = torch.empty((self.bsz, self.n_local_kv_heads, self.head_dim), dtype=torch.uint8, device=q.device)
        s = cuda_module.k_cache_compute(self.k_cache_first_8, self.k_cache_mid_4, self.k_cache_last_4,
                                        exp_sum.contiguous(), exp_sum_max.contiguous(), q.view(torch.uint8),
                                        self.bsz, self.n_local_kv_heads, cdiv(self.reststartpos, self.k_block),
                                        self.k_n_max_blocks, self.head_dim, self.k_block, self.reststartpos,
                                        1.0 / math.sqrt(self.head_dim), reference, levels_out=levels)
        self.last_levels = levels
        s = s.view(torch.half)
        rest = self._rest[:, :self._restlen].permute(0, 2, 3, 1)        # [bsz, heads, head_dim, restlen]
        s[:, :, :, self.reststartpos:self.reststartpos + self._restlen] = \
            torch.matmul(q.transpose(1, 2), rest) / math.sqrt(self.head_dim)
        s[:, :, :, start_pos + seqlen:] = float("-inf")
        if self.record_levels:
            self.last_scores = s.clone()     # the caller adds its mask in place
        return s
