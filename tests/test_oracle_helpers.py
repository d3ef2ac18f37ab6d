"""Pins the three oracle helpers that sit on the "truth" side of nearly every comparison and have no pin of their
own elsewhere: k_sum_and_max, softmax_fp32_to_half and dense_attention.  Each is held against something that does
not share its formula: nested Python loops over scalars, torch's own softmax / matmul, float64 closed forms and
known answers."""
import math

import numpy as np
import pytest
import torch

from oracle import akv_oracle as O
from tests.common import make_qkv, ulp_diff_fp16


# ---- k_sum_and_max (extension/k_cache_file.py:136-138) ---------------------------------------------------
def _exp_scalar(h):
    """exponent field of one fp16 value from its bits, sign stripped"""
    bits = int(np.array(h, np.float16).view(np.uint16))
    return (bits >> 10) & 0x1F


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_k_sum_and_max_brute_force(seed):
    rng = np.random.default_rng(seed)
    B, H, D = 2, 4, 8
    # values over the whole exponent range, both signs, zeros and subnormals included
    q = (rng.standard_normal((B, 1, H, D)) * np.exp(rng.uniform(-12, 8, (B, 1, H, D)))).astype(np.float16)
    q[0, 0, 0, 0] = 0.0
    q[1, 0, 2, 3] = np.float16(3e-7)
    colmax = rng.integers(0, 32, (B, 1, H, D)).astype(np.uint8)
    s, mx = O.k_sum_and_max(q, colmax)
    assert s.dtype == np.uint8 and mx.dtype == np.uint8
    assert s.shape == (B, 1, H, D) and mx.shape == (B, 1, H, 1)
    for b in range(B):
        for h in range(H):
            best = 0
            for d in range(D):
                want = (_exp_scalar(q[b, 0, h, d]) + int(colmax[b, 0, h, d])) & 0xFF
                assert int(s[b, 0, h, d]) == want, (b, h, d)
                best = max(best, want)
            assert int(mx[b, 0, h, 0]) == best, (b, h)


def test_k_sum_and_max_known_answers():
    # 1.0 has exponent field 15, 2.0 -> 16, 0.5 -> 14, -4.0 -> 17 (the sign is not part of the field), 0 -> 0
    q = np.array([1.0, 2.0, 0.5, -4.0, 0.0, 65504.0, 6e-8, -1.0], np.float16).reshape(1, 1, 1, 8)
    cm = np.array([0, 1, 2, 3, 31, 0, 5, 15], np.uint8).reshape(1, 1, 1, 8)
    s, mx = O.k_sum_and_max(q, cm)
    assert s.reshape(-1).tolist() == [15, 17, 16, 20, 31, 30, 5, 30]
    assert int(mx.reshape(-1)[0]) == 31


# ---- softmax_fp32_to_half (model/KVCache_AlignedKV.py:121) ------------------------------------------------
def _score_rows(seed, rows, width):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, width)) * rng.uniform(0.2, 6.0, (rows, 1))).astype(np.float16)
    # -inf tails of different lengths (the positions past the valid length, extension/k_cache_file.py:158)
    for r in range(rows):
        cut = int(rng.integers(1, width + 1))
        x[r, cut:] = -np.inf
    return x


def test_softmax_against_torch():
    x = _score_rows(7, 3000, 257)
    got = O.softmax_fp32_to_half(x)
    want = torch.softmax(torch.from_numpy(x).float(), dim=-1).half().numpy()
    assert got.dtype == np.float16
    # torch and NumPy differ in how they order the fp32 sum and evaluate exp: at most the last fp16 bit, rarely
    d = ulp_diff_fp16(got, want)
    assert d.max() <= 1
    assert (d == 0).mean() >= 0.999
    assert np.all(got[np.isneginf(x.astype(np.float32))] == 0)


def test_softmax_against_float64_closed_form():
    x = _score_rows(11, 500, 96)
    got = O.softmax_fp32_to_half(x).astype(np.float64)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=-1, keepdims=True))
    want = e / e.sum(axis=-1, keepdims=True)
    # one fp16 rounding of a value that fp32 arithmetic got right to ~1e-6 relative
    spacing = np.abs(np.spacing(want.astype(np.float16))).astype(np.float64)
    assert np.all(np.abs(got - want) <= 0.5 * spacing + 4e-6 * want + 1e-12)
    # probabilities: non-negative, order-preserving inside a row, rows sum to one up to the fp16 roundings
    assert np.all(got >= 0)
    assert np.all(np.abs(got.sum(axis=-1) - 1.0) <= 96 * 2.0 ** -12)
    order = np.argsort(x64, axis=-1)
    assert np.all(np.diff(np.take_along_axis(got, order, axis=-1), axis=-1) >= 0)


def test_softmax_known_answers():
    ninf = -np.inf
    x = np.array([[0.0, 0.0, 0.0, 0.0], [5.0, ninf, ninf, ninf], [1.0, 1.0, ninf, ninf], [0.0, math.log(3.0), ninf, ninf]],
                 np.float16)
    p = O.softmax_fp32_to_half(x)
    assert p[0].tolist() == [0.25, 0.25, 0.25, 0.25]
    assert p[1].tolist() == [1.0, 0.0, 0.0, 0.0]
    assert p[2].tolist() == [0.5, 0.5, 0.0, 0.0]
    # fp16(log 3) = 1.0986328125; softmax = 1 / (1 + e^x), e^x / (1 + e^x), rounded to fp16
    t = math.exp(float(np.float16(math.log(3.0))))
    assert p[3, 0] == np.float16(1 / (1 + t)) and p[3, 1] == np.float16(t / (1 + t))
    # shifting a row by a constant changes nothing (as long as the fp16 scores stay exact)
    a = np.array([[0.5, -1.25, 3.0, ninf]], np.float16)
    assert np.array_equal(O.softmax_fp32_to_half(a), O.softmax_fp32_to_half((a + np.float16(8.0)).astype(np.float16)))


# ---- dense_attention (model/Llama_AlignedKV.py:130-139) ----------------------------------------------------
def _torch_dense_branch(q, k, v, mask):
    """The dense branch as the reference writes it, on head-major tensors, with torch's own fp16 matmul and softmax."""
    qt = torch.from_numpy(q).transpose(1, 2)             # [B,H,1,D]
    kt = torch.from_numpy(k).transpose(1, 2)             # [B,H,L,D]
    vt = torch.from_numpy(v).transpose(1, 2)
    w = torch.matmul(qt, kt.transpose(2, 3)) / math.sqrt(q.shape[-1])
    if mask is not None:
        w = w + torch.from_numpy(mask)[:, :, :, :kt.shape[-2]]
    w = torch.nn.functional.softmax(w, dim=-1, dtype=torch.float32).to(qt.dtype)
    o = torch.matmul(w, vt)
    return o.transpose(1, 2).contiguous().numpy()        # [B,1,H,D]


@pytest.mark.parametrize("with_mask", [False, True])
def test_dense_attention_against_torch(with_mask):
    B, H, D, L = 2, 4, 64, 150
    q, k, v = make_qkv(B, L, H, D, seed=5)
    mask = None
    if with_mask:
        mask = np.zeros((B, 1, 1, L), np.float16)
        mask[0, ..., 100:] = -np.inf                     # a shorter sequence in the batch
        mask[1, ..., 7] = np.float16(-3.5)
    got = O.dense_attention(q, k, v, mask)
    want = _torch_dense_branch(q, k, v, mask)
    assert got.shape == (B, 1, H, D) and got.dtype == np.float16
    # two fp16 matmuls and an fp16 probability vector: the routines may round a score to the neighbouring fp16
    # value, which moves the output by well under 1e-3 at these magnitudes
    err = np.max(np.abs(got.astype(np.float32) - want.astype(np.float32)))
    assert err <= 1e-3, err


def test_dense_attention_against_float64():
    B, H, D, L = 1, 3, 32, 40
    q, k, v = make_qkv(B, L, H, D, seed=9, k_kind="plain")
    got = O.dense_attention(q, k, v).astype(np.float64)
    q64, k64, v64 = (a.astype(np.float64) for a in (q, k, v))
    w = np.einsum("bhd,blhd->bhl", q64[:, 0], k64) / math.sqrt(D)
    e = np.exp(w - w.max(axis=-1, keepdims=True))
    p = e / e.sum(axis=-1, keepdims=True)
    want = np.einsum("bhl,blhd->bhd", p, v64)[:, None]
    # fp16 scores (relative 2^-11 of |w| <= ~3) perturb the probabilities by a few 1e-3 relative
    assert np.max(np.abs(got - want)) <= 4e-3
    # a transposed operand, a missing 1/sqrt(D) or a softmax over the wrong axis is far outside that
    wrong = np.einsum("bhl,blhd->bhd", np.exp(w * math.sqrt(D) - (w * math.sqrt(D)).max(-1, keepdims=True)) /
                      np.exp(w * math.sqrt(D) - (w * math.sqrt(D)).max(-1, keepdims=True)).sum(-1, keepdims=True), v64)[:, None]
    assert np.max(np.abs(wrong - want)) > 5e-2


def test_dense_attention_one_hot():
    # q picks channel 2; the key of token 5 is large there: the output is (almost exactly) the value row of token 5
    B, H, D, L = 1, 2, 16, 12
    q = np.zeros((B, 1, H, D), np.float16)
    q[..., 2] = 8
    k = np.zeros((B, L, H, D), np.float16)
    k[:, 5, :, 2] = 16
    v = np.arange(B * L * H * D, dtype=np.float32).reshape(B, L, H, D).astype(np.float16) / 64
    o = O.dense_attention(q, k, v)
    assert np.array_equal(o[:, 0], v[:, 5])
