"""Dense fp16 decode attention on the HIP library (akv_dense_decode_step): the baseline the
split-precision path is compared with.  Not part of the reference's interface."""
from __future__ import annotations

import time

import torch

from ._lib import check, load_library


class DenseKVCache:
    """Head-major fp16 K and V caches [bsz, heads, max_seq_len, head_dim] for one layer."""

    def __init__(self, bsz: int, max_seq_len: int, n_heads: int, head_dim: int, device="cuda"):
        self.lib = load_library()
        self.bsz, self.max_seq_len, self.n_heads, self.head_dim = bsz, max_seq_len, n_heads, head_dim
        self.k = torch.zeros((bsz, n_heads, max_seq_len, head_dim), dtype=torch.half, device=device)
        self.v = torch.zeros_like(self.k)
        self.cur_len = 0
        self.row_stride = (max_seq_len + 7) // 8 * 8
        self.scores = torch.empty((bsz, n_heads, self.row_stride), dtype=torch.half, device=device)
        self.probs = torch.empty_like(self.scores)
        need = self.lib.akv_dense_decode_step_workspace_bytes(bsz, n_heads, head_dim, max_seq_len)
        self.ws = torch.empty(need, dtype=torch.uint8, device=device)

    def prefill(self, k: torch.Tensor, v: torch.Tensor):
        """k, v: fp16 [bsz, seqlen, heads, head_dim]."""
        n = k.shape[1]
        self.k[:, :, :n] = k.transpose(1, 2)
        self.v[:, :, :n] = v.transpose(1, 2)
        self.cur_len = n

    def step_args(self, q, k_new, v_new, out):
        return [self.k.data_ptr(), self.v.data_ptr(), q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), out.data_ptr(),
                self.scores.data_ptr(), self.probs.data_ptr(), self.row_stride, self.ws.data_ptr(), self.ws.numel(),
                self.bsz, self.n_heads, self.max_seq_len, self.head_dim, self.cur_len,
                torch.cuda.current_stream().cuda_stream]

    def decode(self, q, k_new, v_new):
        """One decode step; q, k_new, v_new fp16 [bsz,1,heads,head_dim] contiguous.  Returns fp16 [bsz,1,heads,head_dim]."""
        out = torch.empty_like(q)
        check(self.lib.akv_dense_decode_step(*self.step_args(q.contiguous(), k_new.contiguous(), v_new.contiguous(), out)),
              self.lib)
        self.cur_len += 1
        return out


def bench(torch_mod, lib, B, H, D, L_total, n_layers, steps, aligned_sec):
    """Times the dense step at the same shape (cache of L_total - 1 tokens + 1 appended), rotating over
    n_layers caches like the AlignedKV leg.  Returns extra fields for the benchmark's JSON line."""
    if D != 128:
        return {}
    g = torch.Generator(device="cuda").manual_seed(4242)
    caches = []
    for _ in range(n_layers):
        c = DenseKVCache(B, L_total + 7, H, D)
        c.k.normal_(generator=g)
        c.v.normal_(generator=g)
        c.cur_len = L_total - 1
        caches.append(c)
    q = torch.randn((B, 1, H, D), device="cuda", generator=g).half()
    kn = torch.randn((B, 1, H, D), device="cuda", generator=g).half()
    vn = torch.randn((B, 1, H, D), device="cuda", generator=g).half()
    out = torch.empty_like(q)
    args = [c.step_args(q, kn, vn, out) for c in caches]
    for i in range(10):
        lib.akv_dense_decode_step(*args[i % n_layers])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        rc = lib.akv_dense_decode_step(*args[i % n_layers])
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    if rc != 0:
        raise RuntimeError(lib.akv_last_error().decode())
    dense_bytes = 2 * B * H * L_total * D * 2
    return {"dense_fp16_hip_us": round(sec * 1e6, 2), "dense_fp16_hip_gbps": round(dense_bytes / sec / 1e9, 1),
            "speedup_vs_dense_fp16_hip": round(sec / aligned_sec, 3)}
