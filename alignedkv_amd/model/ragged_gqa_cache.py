"""Split-precision KV cache for grouped-query attention with a length per sequence.

Beyond the reference (which asserts multi-head attention and keeps one scalar length per layer,
model/KVCache_AlignedKV.py:32, extension/k_cache_file.py:74): per query head the algorithm is unchanged
-- the reference's fetch levels, substitution constants, 64-token rest buffer -- applied to the planes of
the query head's KV head, i.e. AlignedKV on `repeat_kv`-ed keys and values without materialising them.
Lengths live in an int32 device tensor that the fused step advances itself, so a decode step needs no
host-side knowledge of which sequences flush their rest buffer.
"""
from __future__ import annotations

import torch

from ..extension._plane_cache import cdiv, column_block, exponent_bits
from ..extension.KV_cache_cpp_extention import cuda_module


class RaggedGQACache:
    def __init__(self, n_layers: int, bsz: int, max_seq_len: int, n_q_heads: int, n_kv_heads: int, head_dim: int,
                 device="cuda", literal_colmax: bool = True, k_block: int = column_block):
        """k_block: tokens per block of the K planes (64, or 256 for head_dim 64 / 128 and 2 to 16 query heads per KV
        head: a nibble row of a channel is then a whole 128-byte line)."""
        assert n_q_heads % n_kv_heads == 0 and k_block in (column_block, 4 * column_block)
        self.n_layers, self.bsz, self.max_seq_len = n_layers, bsz, max_seq_len
        self.n_q_heads, self.n_kv_heads, self.head_dim = n_q_heads, n_kv_heads, head_dim
        self.k_block = k_block
        self.n_max_blocks = cdiv(max_seq_len, k_block)     # K plane blocks
        self.literal_colmax = literal_colmax
        self.reference = False
        self.record_levels = False
        z = lambda *shape: torch.zeros(shape, dtype=torch.uint8, device=device)
        B, H, D, cb, NB = bsz, n_kv_heads, head_dim, column_block, self.n_max_blocks
        self.k_planes = [(z(B, H, NB, D, k_block), z(B, H, NB, D, k_block // 2), z(B, H, NB, D, k_block // 2))
                         for _ in range(n_layers)]
        self.v_planes = [(z(B, H, max_seq_len, D), z(B, H, max_seq_len, D // 2), z(B, H, max_seq_len, D // 2))
                         for _ in range(n_layers)]
        self.k_colmax = [z(B, 1, H, D) for _ in range(n_layers)]
        self.v_colmax = [z(B, 1, H, D) for _ in range(n_layers)]
        self.restk = [torch.zeros((B, cb, H, D), dtype=torch.half, device=device) for _ in range(n_layers)]
        self.restv = [torch.zeros((B, cb, H, D), dtype=torch.half, device=device) for _ in range(n_layers)]
        self.seq_lens = [torch.zeros(B, dtype=torch.int32, device=device) for _ in range(n_layers)]
        self.len_bound = [0] * n_layers          # host-side upper bound of seq_lens (sizes the launches)
        width = (cdiv(max_seq_len, cb) + 1) * cb
        self.scores = torch.empty((B, n_q_heads, width), dtype=torch.half, device=device)
        self.probs = torch.empty((B, n_q_heads, width), dtype=torch.half, device=device)
        self.last_k_levels = self.last_v_levels = self.last_alignment_min = None

    def _colmax(self, x: torch.Tensor) -> torch.Tensor:
        if self.literal_colmax:   # exponent of the signed maximum, as the reference's prefill computes it
            return exponent_bits(torch.max(x, dim=1, keepdim=True).values)
        return exponent_bits(x).max(dim=1, keepdim=True).values

    def prefill(self, layer: int, b: int, k: torch.Tensor, v: torch.Tensor):
        """Stores the prompt of sequence b: k, v fp16 [1, S, n_kv_heads, head_dim].  Whole 64-token blocks go
        into the planes, the remainder into the rest buffer (extension/k_cache_file.py:76-96)."""
        S = k.shape[1]
        assert tuple(k.shape) == (1, S, self.n_kv_heads, self.head_dim) and k.shape == v.shape and S <= self.max_seq_len
        k, v = k.contiguous(), v.contiguous()
        H, D, cb = self.n_kv_heads, self.head_dim, column_block
        tail = S % cb
        kp = [p[b:b + 1] for p in self.k_planes[layer]]
        vp = [p[b:b + 1] for p in self.v_planes[layer]]
        if S - tail:
            # whole 64-token tiles; with 256-token blocks the last block may be partly filled
            cuda_module.k_cache_save(*kp, k[:, :S - tail].contiguous().view(torch.uint8), 1, H, cdiv(S - tail, self.k_block),
                                     self.n_max_blocks, D, self.k_block, 0, S - tail)
        cuda_module.v_cache_save(*vp, v.view(torch.uint8), 1, H, self.max_seq_len, D, 0, S - tail)
        self.k_colmax[layer][b:b + 1] = self._colmax(k)
        self.v_colmax[layer][b:b + 1] = self._colmax(v)
        self.restk[layer][b, :tail] = k[0, S - tail:]
        self.restv[layer][b, :tail] = v[0, S - tail:]
        self.seq_lens[layer][b] = S
        self.len_bound[layer] = max(self.len_bound[layer], S)

    def decode(self, layer: int, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask2d=None, bound=None) -> torch.Tensor:
        """One decode step for every sequence: q fp16 [bsz,1,n_q_heads,head_dim], k/v [bsz,1,n_kv_heads,head_dim].
        Returns fp16 [bsz,1,n_q_heads,head_dim] and advances the lengths.  bound: upper bound of the lengths that
        sizes the launches (default: the largest length this object has seen)."""
        B, Hq, Hkv, D = self.bsz, self.n_q_heads, self.n_kv_heads, self.head_dim
        assert tuple(q.shape) == (B, 1, Hq, D) and tuple(k.shape) == (B, 1, Hkv, D) and k.shape == v.shape
        fixed_bound = bound is not None
        bound = self.len_bound[layer] if bound is None else bound
        assert bound + 1 <= self.max_seq_len, "cache full"
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        out = torch.empty_like(q)
        klv = vlv = amin = None
        flushed = (bound + 1) // column_block * column_block
        if self.record_levels:
            klv = torch.empty((B, Hq, D), dtype=torch.uint8, device=q.device)
            vlv = torch.full((B, Hq, max(flushed, 1)), 255, dtype=torch.uint8, device=q.device)
            amin = torch.zeros((B, Hq), dtype=torch.uint8, device=q.device)
        cuda_module.decode_step_gqa(self.k_planes[layer], self.v_planes[layer], self.k_colmax[layer], self.v_colmax[layer],
                                    self.restk[layer].view(torch.uint8), self.restv[layer].view(torch.uint8),
                                    q.view(torch.uint8), k.view(torch.uint8), v.view(torch.uint8), mask2d,
                                    out.view(torch.uint8), self.scores.view(torch.uint8), self.probs.view(torch.uint8),
                                    B, Hq, Hkv, self.n_max_blocks, self.max_seq_len, D, column_block, 32, bound,
                                    self.seq_lens[layer], self.reference, klv, vlv if flushed else None, amin,
                                    k_block=self.k_block)
        if not fixed_bound:
            self.len_bound[layer] = bound + 1
        self.last_k_levels, self.last_v_levels, self.last_alignment_min = klv, vlv, amin
        return out

    def capture_decode(self, layer: int):
        """One decode step of `layer` as a HIP graph.  With the capacity as the length bound every argument of
        akv_decode_step_gqa is constant from step to step (the lengths live on the device and the step advances
        them itself), so the five launches of a step are captured once and replayed: the host then pays one graph
        launch per step instead of five kernel launches, which is what bounds small batches.
        Returns (graph, q, k, v, out): write the step's inputs into q, k, v, call graph.replay(), read out.
        The caller keeps the lengths below the capacity (the step does not check them on the device)."""
        assert not self.record_levels, "level recording sizes its buffers per step"
        dev = self.seq_lens[layer].device
        q = torch.zeros((self.bsz, 1, self.n_q_heads, self.head_dim), dtype=torch.half, device=dev)
        k = torch.zeros((self.bsz, 1, self.n_kv_heads, self.head_dim), dtype=torch.half, device=dev)
        v = torch.zeros_like(k)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = self.decode(layer, q, k, v, bound=self.max_seq_len - 1)
        return graph, q, k, v, out
