"""State shared by the K and V cache classes: geometry, column-max exponents, the fp16 rest buffer
and the argument checks of save().  The reference keeps two copies of this logic
(extension/k_cache_file.py:14-118, extension/v_cache_file.py:15-116)."""
from __future__ import annotations

import torch

bits_in_a_channel = 256
column_block = bits_in_a_channel // 4   # 64 tokens per flushed block (extension/k_cache_file.py:5-6)


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def exponent_bits(x: torch.Tensor) -> torch.Tensor:
    """Exponent field of every fp16 element as uint8 (extension/k_cache_file.py:77-78,98-99,136)."""
    return (x.view(torch.int16) >> 10).to(torch.uint8) & 0x1F


class PlaneCacheBase(torch.nn.Module):
    """Bookkeeping of one layer's K or V cache.  Subclasses own the planes and call `_store_planes`."""

    def __init__(self, bsz: int, max_seq_len: int, n_local_kv_heads: int, head_dim: int, device, literal_colmax: bool):
        super().__init__()
        self.bsz = bsz
        self.max_seq_len = max_seq_len
        self.n_local_kv_heads = n_local_kv_heads
        self.head_dim = head_dim
        self.n_max_blocks = cdiv(max_seq_len, column_block)
        self.device = device
        # True: exponent of the signed maximum at prefill, as the reference computes it
        # (extension/k_cache_file.py:77-78); False: exponent of the largest magnitude.
        self.literal_colmax = literal_colmax
        self.reststartpos = 0
        self.current_cache_len = 0
        self._rest = None
        self._restlen = 0
        self._colmax = None

    def _alloc(self, name: str, shape, register_buffer: bool) -> torch.Tensor:
        t = torch.zeros(shape, dtype=torch.uint8, device=self.device)
        if register_buffer:
            self.register_buffer(name, t)
            t = getattr(self, name)
            torch._dynamo.mark_static_address(t)
        return t

    def _new_rest(self) -> torch.Tensor:
        return torch.zeros((self.bsz, column_block, self.n_local_kv_heads, self.head_dim), dtype=torch.half,
                           device=self.device)

    def _check_save(self, new: torch.Tensor, start_pos: int, seqlen: int, what: str):
        want = (self.bsz, seqlen, self.n_local_kv_heads, self.head_dim)
        assert tuple(new.shape) == want, f"{what}.shape: {tuple(new.shape)} != {want}"
        assert start_pos + seqlen <= self.max_seq_len, f"start_pos + seqlen: {start_pos + seqlen} > {self.max_seq_len}"
        assert start_pos == 0 or seqlen == 1, f"start_pos: {start_pos}, seqlen: {seqlen}"
        assert start_pos == self.current_cache_len, "start pos != current KV-Cache len"
        assert new.dtype == torch.half, f"{what} must be fp16, got {new.dtype}"

    def _save(self, new: torch.Tensor, start_pos: int, seqlen: int, what: str):
        """Exponent tracking + rest buffer + flush policy (extension/k_cache_file.py:75-118)."""
        self._check_save(new, start_pos, seqlen, what)
        new = new.contiguous()
        self.current_cache_len += seqlen
        if start_pos == 0:
            if self.literal_colmax:
                self._colmax = exponent_bits(torch.max(new, dim=1, keepdim=True).values)
            else:
                self._colmax = exponent_bits(new).max(dim=1, keepdim=True).values
            tail = seqlen % column_block
            self._store_planes(new, 0, seqlen - tail)
            self._rest = self._new_rest()
            self._rest[:, :tail] = new[:, seqlen - tail:]
            self._restlen = tail
            self.reststartpos = seqlen - tail
        else:
            self._colmax = torch.maximum(self._colmax, exponent_bits(new))
            self._rest[:, self._restlen:self._restlen + seqlen] = new
            self._restlen += seqlen
            if self._restlen == column_block:
                self._store_planes(self._rest, self.reststartpos, column_block)
                self._restlen = 0
                self.reststartpos += column_block
                self._rest = self._new_rest()

    def _store_planes(self, tokens: torch.Tensor, start_pos: int, n_tokens: int):
        raise NotImplementedError

    def _advance_after_fused_step(self):
        """Host counters after the fused step appended one token (and flushed a full rest buffer)."""
        d = self.__dict__     # plain integers: no need for torch.nn.Module.__setattr__ on every step
        d["current_cache_len"] += 1
        d["_restlen"] += 1
        if d["_restlen"] == column_block:
            d["_restlen"] = 0
            d["reststartpos"] += column_block

    def _zero_state(self):
        # the reference leaves the rest buffer untouched here (extension/k_cache_file.py:62-67); a prefill
        # always follows a reset and re-creates it, clearing it as well is harmless
        self.current_cache_len = 0
        self.reststartpos = 0
        self._restlen = 0
        self._rest = None
