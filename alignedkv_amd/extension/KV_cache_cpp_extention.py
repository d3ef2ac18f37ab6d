"""Drop-in for the reference's extension/KV_cache_cpp_extention.py: exposes `cuda_module` with the
five ops k_cache_save, k_cache_compute, v_cache_save, v_cache_test_compute, v_cache_compute
(reference binding: extension/csrc/KV_cache_ops.cpp:69-75), same positional signatures and the
same "every tensor crosses as torch.uint8" convention.

Here the ops are thin marshalling over the C ABI of libalignedkv_hip.so (include/alignedkv.h):
torch supplies device memory and the current stream, the arithmetic is in the HIP library.
Nothing is compiled at import time and there is no fallback implementation.
"""
from __future__ import annotations

import torch

from .._lib import check, load_library


def _stream_ptr(device) -> int:
    """Raw handle of the current stream of `device` (the fast path of torch.cuda.current_stream(device).cuda_stream)."""
    try:
        index = device.index if isinstance(device, torch.device) else torch.device(device).index
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index)
    except (AttributeError, TypeError):
        return torch.cuda.current_stream(device).cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _require(name: str, t: torch.Tensor, min_bytes: int, device=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch.Tensor, got {type(t).__name__}")
    if t.dtype != torch.uint8:
        raise RuntimeError(f"{name}: expected dtype torch.uint8 (pass .view(torch.uint8)), got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name}: expected a tensor on the GPU, got device {t.device}")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name}: on {t.device}, other arguments on {device}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name}: must be contiguous")
    if t.numel() < min_bytes:
        raise RuntimeError(f"{name}: holds {t.numel()} bytes, the scalar arguments imply {min_bytes}")


class _AlignedKVModule:
    """The object bound to the name `cuda_module`."""

    def __init__(self):
        self._workspaces = {}

    def _workspace(self, device, nbytes: int) -> torch.Tensor:
        # one scratch buffer per (device, stream): calls on one stream are ordered, so they can share it
        key = (device, torch.cuda.current_stream(device).cuda_stream)
        ws = self._workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
            self._workspaces[key] = ws
        return ws

    # ---- K ---------------------------------------------------------------------------------
    def k_cache_save(self, k_cache_first_8, k_cache_mid_4, k_cache_last_4, k_new, bsz, n_kv_heads, n_blocks,
                     n_max_blocks, d_head, d_block, start_pos, seqlen):
        lib = load_library()
        dev = k_new.device if isinstance(k_new, torch.Tensor) else None
        plane = bsz * n_kv_heads * n_max_blocks * d_head * d_block
        _require("k_cache_first_8", k_cache_first_8, plane, dev)
        _require("k_cache_mid_4", k_cache_mid_4, plane // 2, dev)
        _require("k_cache_last_4", k_cache_last_4, plane // 2, dev)
        _require("k_new", k_new, bsz * seqlen * n_kv_heads * d_head * 2, dev)
        with torch.cuda.device(dev):
            check(lib.akv_k_cache_save(_ptr(k_cache_first_8), _ptr(k_cache_mid_4), _ptr(k_cache_last_4), _ptr(k_new),
                                       bsz, n_kv_heads, n_blocks, n_max_blocks, d_head, d_block, start_pos, seqlen,
                                       _stream_ptr(dev)), lib)

    def k_cache_compute(self, k_cache_first_8, k_cache_mid_4, k_cache_last_4, k_column_max_multiply_q,
                        k_column_max_multiply_q_max, q, bsz, n_kv_heads, n_blocks, n_max_blocks, d_head, d_block,
                        seqlen, sqrt_dim, reference, levels_out=None):
        lib = load_library()
        dev = q.device if isinstance(q, torch.Tensor) else None
        plane = bsz * n_kv_heads * n_max_blocks * d_head * d_block
        _require("k_cache_first_8", k_cache_first_8, plane, dev)
        _require("k_cache_mid_4", k_cache_mid_4, plane // 2, dev)
        _require("k_cache_last_4", k_cache_last_4, plane // 2, dev)
        _require("k_column_max_multiply_q", k_column_max_multiply_q, bsz * n_kv_heads * d_head, dev)
        _require("k_column_max_multiply_q_max", k_column_max_multiply_q_max, bsz * n_kv_heads, dev)
        _require("q", q, bsz * n_kv_heads * d_head * 2, dev)
        if levels_out is not None:
            _require("levels_out", levels_out, bsz * n_kv_heads * d_head, dev)
        s = torch.empty((bsz, n_kv_heads, 1, (n_blocks + 1) * d_block * 2), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            check(lib.akv_k_cache_compute(_ptr(k_cache_first_8), _ptr(k_cache_mid_4), _ptr(k_cache_last_4),
                                          _ptr(k_column_max_multiply_q), _ptr(k_column_max_multiply_q_max), _ptr(q),
                                          _ptr(s), _ptr(levels_out), bsz, n_kv_heads, n_blocks, n_max_blocks, d_head,
                                          d_block, seqlen, float(sqrt_dim), int(bool(reference)), _stream_ptr(dev)),
                  lib)
        return s

    # ---- V ---------------------------------------------------------------------------------
    def v_cache_save(self, v_cache_first_8, v_cache_mid_4, v_cache_last_4, v_new, bsz, n_local_kv_heads, max_seq_len,
                     head_dim, start_pos, seq_len):
        lib = load_library()
        if not isinstance(v_new, torch.Tensor) or v_new.dim() != 4:
            raise RuntimeError("v_new: expected a 4-d uint8 view [bsz, seqlen, heads, head_dim*2]")
        dev = v_new.device
        plane = bsz * n_local_kv_heads * max_seq_len * head_dim
        v_new_seq = v_new.size(1)
        _require("v_cache_first_8", v_cache_first_8, plane, dev)
        _require("v_cache_mid_4", v_cache_mid_4, plane // 2, dev)
        _require("v_cache_last_4", v_cache_last_4, plane // 2, dev)
        _require("v_new", v_new, bsz * v_new_seq * n_local_kv_heads * head_dim * 2, dev)
        with torch.cuda.device(dev):
            check(lib.akv_v_cache_save(_ptr(v_cache_first_8), _ptr(v_cache_mid_4), _ptr(v_cache_last_4), _ptr(v_new),
                                       bsz, n_local_kv_heads, max_seq_len, head_dim, start_pos, seq_len, v_new_seq,
                                       _stream_ptr(dev)), lib)

    def v_cache_test_compute(self, v_cache_first_8, v_cache_mid_4, v_cache_last_4, test_s_value, test_s_index, bsz,
                             n_local_kv_heads, max_seq_len, head_dim, top_max_k):
        lib = load_library()
        dev = test_s_value.device if isinstance(test_s_value, torch.Tensor) else None
        plane = bsz * n_local_kv_heads * max_seq_len * head_dim
        _require("v_cache_first_8", v_cache_first_8, plane, dev)
        _require("test_s_value", test_s_value, bsz * n_local_kv_heads * top_max_k * 2, dev)
        _require("test_s_index", test_s_index, bsz * n_local_kv_heads * top_max_k * 4, dev)
        test_o = torch.empty((bsz, n_local_kv_heads, 1, head_dim * 2), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            check(lib.akv_v_cache_test_compute(_ptr(v_cache_first_8), _ptr(v_cache_mid_4), _ptr(v_cache_last_4),
                                               _ptr(test_s_value), _ptr(test_s_index), _ptr(test_o), bsz,
                                               n_local_kv_heads, max_seq_len, head_dim, top_max_k, _stream_ptr(dev)),
                  lib)
        return test_o

    def v_cache_compute(self, v_cache_first_8, v_cache_mid_4, v_cache_last_4, s, s_exp_expect_alignment_min, bsz,
                        n_local_kv_heads, max_seq_len, head_dim, s_last_dim, start_pos_add_seqlen, reference,
                        levels_out=None):
        lib = load_library()
        dev = v_cache_first_8.device if isinstance(v_cache_first_8, torch.Tensor) else None
        plane = bsz * n_local_kv_heads * max_seq_len * head_dim
        n_tok = start_pos_add_seqlen
        _require("v_cache_first_8", v_cache_first_8, plane, dev)
        _require("v_cache_mid_4", v_cache_mid_4, plane // 2, dev)
        _require("v_cache_last_4", v_cache_last_4, plane // 2, dev)
        # `s` may be a sliced view (row stride s_last_dim, reference: extension/v_cache_file.py:150,184):
        # only its base pointer and the stride argument are used, like in the reference op
        if not isinstance(s, torch.Tensor) or s.dtype != torch.uint8 or not s.is_cuda:
            raise RuntimeError("s: expected a uint8 view of the fp16 probabilities on the GPU")
        if n_tok > 0:
            if s.stride(-1) != 1:
                raise RuntimeError("s: innermost dimension must be dense")
            span = ((bsz * n_local_kv_heads - 1) * s_last_dim + n_tok) * 2
            avail = s.untyped_storage().nbytes() - s.storage_offset()
            if span > avail:
                raise RuntimeError(f"s: rows of stride {s_last_dim} halves need {span} bytes, storage has {avail}")
        _require("s_exp_expect_alignment_min", s_exp_expect_alignment_min, bsz * n_local_kv_heads, dev)
        if levels_out is not None:
            _require("levels_out", levels_out, bsz * n_local_kv_heads * n_tok, dev)
        o = torch.empty((bsz, n_local_kv_heads, 1, head_dim * 2), dtype=torch.uint8, device=dev)
        need = lib.akv_v_cache_compute_workspace_bytes(bsz, n_local_kv_heads, head_dim, n_tok)
        ws = self._workspace(dev, need)
        with torch.cuda.device(dev):
            check(lib.akv_v_cache_compute(_ptr(v_cache_first_8), _ptr(v_cache_mid_4), _ptr(v_cache_last_4), _ptr(s),
                                          _ptr(s_exp_expect_alignment_min), _ptr(o), _ptr(levels_out), _ptr(ws),
                                          ws.numel(), bsz, n_local_kv_heads, max_seq_len, head_dim, s_last_dim,
                                          n_tok, int(bool(reference)), _stream_ptr(dev)), lib)
        return o

    # ---- fused decode step (no counterpart among the reference's five ops: it replaces the Python glue
    #      of model/KVCache_AlignedKV.py:116-124 around them) -----------------------------------------------
    def decode_step(self, k_planes, v_planes, k_exp_column_max, v_exp_column_max, restk, restv, q, k_new, v_new,
                    mask, out, scores, probs, bsz, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block,
                    top_max_k, cur_len, rest_start, rest_len, reference, literal_broadcast,
                    k_levels_out=None, v_levels_out=None, amin_out=None, record_probs=True):
        """All tensors as torch.uint8 views on one device; see akv_decode_step in include/alignedkv.h.
        record_probs=False: AKV_STEP_NO_PROBS_RECORD (probs may be left unwritten where the step does not need it)."""
        lib = load_library()
        dev = q.device
        kplane = bsz * n_kv_heads * n_max_blocks * head_dim * d_block
        vplane = bsz * n_kv_heads * max_seq_len * head_dim
        tok = bsz * n_kv_heads * head_dim * 2
        for name, t, n in (("k_first_8", k_planes[0], kplane), ("k_mid_4", k_planes[1], kplane // 2),
                           ("k_last_4", k_planes[2], kplane // 2), ("v_first_8", v_planes[0], vplane),
                           ("v_mid_4", v_planes[1], vplane // 2), ("v_last_4", v_planes[2], vplane // 2),
                           ("k_exp_column_max", k_exp_column_max, tok // 2), ("v_exp_column_max", v_exp_column_max, tok // 2),
                           ("restk", restk, tok * d_block), ("restv", restv, tok * d_block), ("q", q, tok),
                           ("k_new", k_new, tok), ("v_new", v_new, tok), ("out", out, tok)):
            _require(name, t, n, dev)
        row_stride = scores.shape[-1] // 2
        _require("scores", scores, bsz * n_kv_heads * row_stride * 2, dev)
        _require("probs", probs, bsz * n_kv_heads * row_stride * 2, dev)
        mask_stride = 0
        if mask is not None:
            if mask.dtype != torch.uint8 or mask.dim() != 2 or mask.stride(-1) != 1 or not mask.is_cuda:
                raise RuntimeError("mask: expected a 2-d uint8 view [rows, 2*len] of an fp16 mask on the GPU")
            if mask.shape[0] not in (1, bsz) or mask.shape[1] < 2 * (cur_len + 1):
                raise RuntimeError(f"mask: shape {tuple(mask.shape)} does not cover {bsz} x {cur_len + 1} halves")
            mask_stride = 0 if mask.shape[0] == 1 else mask.stride(0) // 2
        flushed = rest_start + (d_block if rest_len + 1 == d_block else 0)
        if k_levels_out is not None:
            _require("k_levels_out", k_levels_out, bsz * n_kv_heads * head_dim, dev)
        if v_levels_out is not None:
            _require("v_levels_out", v_levels_out, bsz * n_kv_heads * flushed, dev)
        if amin_out is not None:
            _require("amin_out", amin_out, bsz * n_kv_heads, dev)
        need = lib.akv_decode_step_workspace_bytes(bsz, n_kv_heads, head_dim, max_seq_len)
        ws = self._workspace(dev, need)
        with torch.cuda.device(dev):
            check(lib.akv_decode_step(_ptr(k_planes[0]), _ptr(k_planes[1]), _ptr(k_planes[2]), _ptr(v_planes[0]),
                                      _ptr(v_planes[1]), _ptr(v_planes[2]), _ptr(k_exp_column_max),
                                      _ptr(v_exp_column_max), _ptr(restk), _ptr(restv), _ptr(q), _ptr(k_new),
                                      _ptr(v_new), _ptr(mask), mask_stride, _ptr(out), _ptr(scores), _ptr(probs),
                                      row_stride, _ptr(ws), ws.numel(), _ptr(k_levels_out), _ptr(v_levels_out),
                                      _ptr(amin_out), bsz, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block,
                                      top_max_k, cur_len, rest_start, rest_len, int(bool(reference)),
                                      _step_flags(literal_broadcast, record_probs), _stream_ptr(dev)), lib)

    def decode_step_gqa(self, k_planes, v_planes, k_exp_column_max, v_exp_column_max, restk, restv, q, k_new, v_new,
                        mask, out, scores, probs, bsz, n_q_heads, n_kv_heads, n_max_blocks, max_seq_len, head_dim,
                        d_block, top_max_k, cur_len, seq_lens, reference, k_levels_out=None, v_levels_out=None,
                        amin_out=None, k_block=None, literal_broadcast=False, record_probs=True):
        """Fused step with grouped-query heads and optional per-sequence lengths (seq_lens: int32 device tensor
        [bsz], incremented by the step; cur_len then bounds them).  See akv_decode_step_gqa in include/alignedkv.h."""
        lib = load_library()
        dev = q.device
        k_block = d_block if k_block is None else k_block     # tokens per K plane block (n_max_blocks counts these)
        kplane = bsz * n_kv_heads * n_max_blocks * head_dim * k_block
        vplane = bsz * n_kv_heads * max_seq_len * head_dim
        tok_q, tok_kv = bsz * n_q_heads * head_dim * 2, bsz * n_kv_heads * head_dim * 2
        for name, t, n in (("k_first_8", k_planes[0], kplane), ("k_mid_4", k_planes[1], kplane // 2),
                           ("k_last_4", k_planes[2], kplane // 2), ("v_first_8", v_planes[0], vplane),
                           ("v_mid_4", v_planes[1], vplane // 2), ("v_last_4", v_planes[2], vplane // 2),
                           ("k_exp_column_max", k_exp_column_max, tok_kv // 2),
                           ("v_exp_column_max", v_exp_column_max, tok_kv // 2), ("restk", restk, tok_kv * d_block),
                           ("restv", restv, tok_kv * d_block), ("q", q, tok_q), ("k_new", k_new, tok_kv),
                           ("v_new", v_new, tok_kv), ("out", out, tok_q)):
            _require(name, t, n, dev)
        row_stride = scores.shape[-1] // 2
        _require("scores", scores, bsz * n_q_heads * row_stride * 2, dev)
        _require("probs", probs, bsz * n_q_heads * row_stride * 2, dev)
        if seq_lens is not None:
            if seq_lens.dtype != torch.int32 or not seq_lens.is_cuda or seq_lens.numel() != bsz or not seq_lens.is_contiguous():
                raise RuntimeError("seq_lens: expected a contiguous int32 tensor [bsz] on the GPU")
        mask_stride = 0
        if mask is not None:
            if mask.dtype != torch.uint8 or mask.dim() != 2 or mask.stride(-1) != 1 or not mask.is_cuda:
                raise RuntimeError("mask: expected a 2-d uint8 view [rows, 2*len] of an fp16 mask on the GPU")
            if mask.shape[0] not in (1, bsz) or mask.shape[1] < 2 * (cur_len + 1):
                raise RuntimeError(f"mask: shape {tuple(mask.shape)} does not cover {bsz} x {cur_len + 1} halves")
            mask_stride = 0 if mask.shape[0] == 1 else mask.stride(0) // 2
        flushed = (cur_len + 1) // d_block * d_block
        if k_levels_out is not None:
            _require("k_levels_out", k_levels_out, bsz * n_q_heads * head_dim, dev)
        if v_levels_out is not None:
            _require("v_levels_out", v_levels_out, bsz * n_q_heads * flushed, dev)
        if amin_out is not None:
            _require("amin_out", amin_out, bsz * n_q_heads, dev)
        need = lib.akv_decode_step_workspace_bytes(bsz, n_q_heads, head_dim, max_seq_len)
        ws = self._workspace(dev, need)
        with torch.cuda.device(dev):
            check(lib.akv_decode_step_gqa(_ptr(k_planes[0]), _ptr(k_planes[1]), _ptr(k_planes[2]), _ptr(v_planes[0]),
                                          _ptr(v_planes[1]), _ptr(v_planes[2]), _ptr(k_exp_column_max),
                                          _ptr(v_exp_column_max), _ptr(restk), _ptr(restv), _ptr(q), _ptr(k_new),
                                          _ptr(v_new), _ptr(mask), mask_stride, _ptr(out), _ptr(scores), _ptr(probs),
                                          row_stride, _ptr(ws), ws.numel(), _ptr(k_levels_out), _ptr(v_levels_out),
                                          _ptr(amin_out), bsz, n_q_heads, n_kv_heads, n_max_blocks, max_seq_len,
                                          head_dim, d_block, k_block, top_max_k, cur_len, _ptr(seq_lens),
                                          int(bool(reference)), _step_flags(literal_broadcast, record_probs), _stream_ptr(dev)), lib)


def _step_flags(literal_broadcast, record_probs) -> int:
    """flags of the fused step: AKV_STEP_LITERAL_BROADCAST = 1, AKV_STEP_NO_PROBS_RECORD = 2 (include/alignedkv.h)"""
    return (1 if literal_broadcast else 0) | (0 if record_probs else 2)


class PreparedDecodeStep:
    """The fused step for one layer of a multi-head cache with everything that does not change between its steps
    checked and converted once into an akv_step_desc: plane, column-maximum, rest-buffer, score and workspace pointers
    and the geometry.  A call checks only the three token tensors and the output (fp16 or uint8 views, contiguous) and
    passes 15 arguments.  Made by `cuda_module.prepare_decode_step`; `key` lets the owner notice that one of the
    captured tensors was replaced (then it prepares again)."""

    def __init__(self, lib, desc, tok_bytes, device, stream, key, keep):
        import ctypes
        self._fn = lib.akv_decode_step_desc
        self._lib = lib
        self._desc = desc
        self._desc_ref = ctypes.byref(desc)
        self._tok = tok_bytes
        self.device = device
        self.stream = stream
        self.key = key
        self._keep = keep               # the tensors behind the pointers

    def __call__(self, q, k_new, v_new, out, mask, mask_stride, cur_len, reference, literal_broadcast,
                 k_levels_out=None, v_levels_out=None, amin_out=None, record_probs=True):
        tok = self._tok
        for t in (q, k_new, v_new, out):
            if t.numel() * t.element_size() != tok or not t.is_contiguous() or t.device != self.device:
                raise RuntimeError("decode step: q, k_new, v_new and out must be contiguous fp16 tensors (or uint8 views) of "
                                   f"{tok} bytes on {self.device}")
        rc = self._fn(self._desc_ref, q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), _ptr(mask), mask_stride,
                      out.data_ptr(), _ptr(k_levels_out), _ptr(v_levels_out), _ptr(amin_out), cur_len, None,
                      1 if reference else 0, (1 if literal_broadcast else 0) | (0 if record_probs else 2), self.stream)
        if rc != 0:
            check(rc, self._lib)


def _prepare_decode_step(self, k_planes, v_planes, k_exp_column_max, v_exp_column_max, restk, restv, scores, probs,
                         bsz, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block, k_block, top_max_k, key=None):
    """The checks of `decode_step_gqa` on the per-layer tensors of a multi-head cache, once; returns a
    PreparedDecodeStep bound to the current stream of their device (a call on another stream needs another one).
    n_max_blocks counts K plane blocks of k_block tokens."""
    lib = load_library()
    dev = k_planes[0].device
    kplane = bsz * n_kv_heads * n_max_blocks * head_dim * k_block
    vplane = bsz * n_kv_heads * max_seq_len * head_dim
    tok = bsz * n_kv_heads * head_dim * 2
    for name, t, n in (("k_first_8", k_planes[0], kplane), ("k_mid_4", k_planes[1], kplane // 2),
                       ("k_last_4", k_planes[2], kplane // 2), ("v_first_8", v_planes[0], vplane),
                       ("v_mid_4", v_planes[1], vplane // 2), ("v_last_4", v_planes[2], vplane // 2),
                       ("k_exp_column_max", k_exp_column_max, tok // 2), ("v_exp_column_max", v_exp_column_max, tok // 2),
                       ("restk", restk, tok * d_block), ("restv", restv, tok * d_block)):
        _require(name, t, n, dev)
    row_stride = scores.shape[-1] // 2
    _require("scores", scores, bsz * n_kv_heads * row_stride * 2, dev)
    _require("probs", probs, bsz * n_kv_heads * row_stride * 2, dev)
    need = lib.akv_decode_step_workspace_bytes(bsz, n_kv_heads, head_dim, max_seq_len)
    ws = self._workspace(dev, need)
    from .._lib import StepDesc
    desc = StepDesc(*(_ptr(t) for t in (*k_planes, *v_planes, k_exp_column_max, v_exp_column_max, restk, restv, scores, probs, ws)),
                    ws.numel(), row_stride, bsz, n_kv_heads, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block, k_block,
                    top_max_k)
    keep = (k_planes, v_planes, k_exp_column_max, v_exp_column_max, restk, restv, scores, probs, ws)
    return PreparedDecodeStep(lib, desc, tok, dev, _stream_ptr(dev), key, keep)


_AlignedKVModule.prepare_decode_step = _prepare_decode_step

cuda_module = _AlignedKVModule()
