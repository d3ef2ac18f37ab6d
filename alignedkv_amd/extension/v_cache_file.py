"""V half of the host hot path: counterpart of the reference's extension/v_cache_file.py
(V_Cache_Class: planes :46-57, save :72-116, test_compute :119-143, decoding_compute :145-190)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ._plane_cache import PlaneCacheBase, cdiv, column_block, exponent_bits
from .KV_cache_cpp_extention import cuda_module

FP16_EXP_BIAS = 2 ** 4 - 1


class V_Cache_Class(PlaneCacheBase):
    def __init__(self, bsz: int, max_seq_len: int, n_local_kv_heads: int, head_dim: int, layer_id: int,
                 device="cuda:0", register_buffer: bool = False, top_max_k: int = 32,
                 literal_colmax: bool = True, literal_broadcast: bool = False):
        super().__init__(bsz, max_seq_len, n_local_kv_heads, head_dim, device, literal_colmax)
        self.v_cache_first_8 = self._alloc(f"v_cache_first_8_layer_{layer_id}",
                                           (bsz, n_local_kv_heads, max_seq_len, head_dim), register_buffer)
        self.v_cache_mid_4 = self._alloc(f"v_cache_mid_4_layer_{layer_id}",
                                         (bsz, n_local_kv_heads, max_seq_len, head_dim // 2), register_buffer)
        self.v_cache_last_4 = self._alloc(f"v_cache_last_4_layer_{layer_id}",
                                          (bsz, n_local_kv_heads, max_seq_len, head_dim // 2), register_buffer)
        self._colmax = torch.zeros((bsz, 1, n_local_kv_heads, head_dim), dtype=torch.uint8, device=device)
        self.top_max_k = top_max_k
        # False: the alignment threshold of (b, h) pairs the probe and the column maxima of the same
        # (b, h).  True: the reference expression as written, whose [B,H,1,D] - [B,1,H,D] broadcast makes
        # entry b*H+h pair the probe of (b // H, b % H) with the maxima of (b // H, h)
        # (extension/v_cache_file.py:156-160, extension/csrc/V_cache.cu:195,337).
        self.literal_broadcast = literal_broadcast
        self.last_levels = None
        self.last_probs = None
        self.last_alignment_min = None
        self.record_levels = False

    @property
    def v_cache_exp_column_max(self):
        return self._colmax

    @v_cache_exp_column_max.setter
    def v_cache_exp_column_max(self, t):
        self._colmax = t

    @property
    def restv(self):
        return self._rest

    @property
    def restvlen(self):
        return self._restlen

    def zerolize(self):
        self.v_cache_first_8.zero_()
        self.v_cache_mid_4.zero_()
        self.v_cache_last_4.zero_()
        self._colmax = torch.zeros_like(self._colmax)
        self._zero_state()

    def _store_planes(self, tokens: torch.Tensor, start_pos: int, n_tokens: int):
        cuda_module.v_cache_save(self.v_cache_first_8, self.v_cache_mid_4, self.v_cache_last_4,
                                 tokens.view(torch.uint8), self.bsz, self.n_local_kv_heads, self.max_seq_len,
                                 self.head_dim, start_pos, n_tokens)

    def save(self, new_v: torch.Tensor, start_pos: int, seqlen: int):
        self._save(new_v, start_pos, seqlen, "new_v")

    def test_compute(self, s: torch.Tensor, start_pos: int, seqlen: int, top_max_k: int):
        """Exponent (LSB cleared) of a cheap estimate of |o|: the largest probability of every residue
        class mod top_max_k times the magnitude of that token's high-byte-only V row."""
        width = s.shape[-1]
        if start_pos + seqlen == width:
            groups = cdiv(width, top_max_k)
            s = F.pad(s, (0, groups * top_max_k - width), "constant", 0)
        else:
            groups = width // top_max_k
            s = s[..., :groups * top_max_k]
        value, index = torch.max(s.reshape(self.bsz, self.n_local_kv_heads, groups, top_max_k), dim=2, keepdim=True)
        test_o = cuda_module.v_cache_test_compute(self.v_cache_first_8, self.v_cache_mid_4, self.v_cache_last_4,
                                                  value.contiguous().view(torch.uint8),
                                                  index.to(torch.int32).contiguous().view(torch.uint8), self.bsz,
                                                  self.n_local_kv_heads, self.max_seq_len, self.head_dim, top_max_k)
        # the reference writes `& 0x1F - 1`, which Python parses as `& 0x1E` (extension/v_cache_file.py:142)
        return exponent_bits(test_o.view(torch.half)) & (0x1F - 1)

    def alignment_min(self, test_o_exp: torch.Tensor) -> torch.Tensor:
        """uint8 threshold per (b, h): min over channels of test_o_exp + 15 - column max, wrapping uint8."""
        if self.literal_broadcast:
            full = test_o_exp + FP16_EXP_BIAS - self._colmax                      # [B,H,H,D]
            return torch.min(full, dim=-1, keepdim=True).values.contiguous()      # first B*H bytes are read
        al = test_o_exp.view(self.bsz, self.n_local_kv_heads, self.head_dim) + FP16_EXP_BIAS \
            - self._colmax.view(self.bsz, self.n_local_kv_heads, self.head_dim)
        return torch.min(al, dim=-1).values.contiguous()

    def decoding_compute(self, s: torch.Tensor, start_pos: int, seqlen: int, reference: bool = False):
        """softmax(scores) @ V for one decode token: flushed tokens through the HIP op (fetch level per
        token from the alignment threshold), the unflushed tail by an fp16 matmul.
        s: fp16 probabilities [bsz, heads, 1, width]; returns fp16 [bsz, heads, 1, head_dim]."""
        assert s.shape[1] == self.n_local_kv_heads, "we currently only support MHA, don't support GQA"
        assert tuple(s.shape) == (self.bsz, self.n_local_kv_heads, 1, s.shape[-1]), f"s.shape: {tuple(s.shape)}"
        assert start_pos + seqlen <= self.max_seq_len, f"start_pos + seqlen: {start_pos + seqlen} > {self.max_seq_len}"
        assert start_pos == 0 or seqlen == 1, f"start_pos: {start_pos}, seqlen: {seqlen}"
        assert self.reststartpos + self._restlen == start_pos + seqlen
        flushed = self.reststartpos
        s_cut = s[:, :, :, :flushed]
        probe_exp = self.test_compute(s_cut if flushed else s, start_pos, seqlen, self.top_max_k)
        amin = self.alignment_min(probe_exp)
        levels = None
        if self.record_levels and flushed:
            levels = torch.empty((self.bsz, self.n_local_kv_heads, flushed), dtype=torch.uint8, device=s.device)
        o = cuda_module.v_cache_compute(self.v_cache_first_8, self.v_cache_mid_4, self.v_cache_last_4,
                                        s_cut.view(torch.uint8), amin, self.bsz, self.n_local_kv_heads,
                                        self.max_seq_len, self.head_dim, s_cut.stride()[-2], flushed, reference,
                                        levels_out=levels)
        self.last_levels, self.last_alignment_min = levels, amin
        if self.record_levels:
            self.last_probs = s      # the probabilities the levels above were derived from (debug record)
        o = o.view(torch.half)
        o += torch.matmul(s[:, :, :, flushed:start_pos + seqlen], self._rest.transpose(1, 2)[:, :, :self._restlen, :])
        return o
