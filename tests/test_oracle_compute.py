"""Pins the floating-point half of the oracle against textbook routines: a float64 matmul on the
original values (level 0 / reference=True) or on values truncated by closed form (levels 1, 2),
brute-force loops on tiny inputs, and the independent C restatement."""
import math

import numpy as np
import pytest

from oracle import akv_oracle as O
from tests.common import make_qkv, ulp_diff_fp16


def _trunc(bits, level):
    b = bits.astype(np.uint32)
    return np.where(level == 0, b, np.where(level == 1, (b & 0xFFF0) | 0x8, (b & 0xFF00) | 0x80)).astype(np.uint16)


def _setup_k(B, H, D, L, seed, cb=64, k_kind="outlier"):
    q, k, _ = make_qkv(B, L, H, D, seed, k_kind)
    planes = O.k_planes_alloc(B, H, L + cb, D, cb)
    O.k_cache_save(*planes, O.as_bits(k), L // cb, cb, 0, L)
    colmax = O.colmax_prefill(k)
    ksum, kmax = O.k_sum_and_max(q, colmax)
    return q, k, planes, ksum, kmax


@pytest.mark.parametrize("reference", [True, False])
def test_k_compute_vs_float64_matmul(oracle_c, reference):
    B, H, D, L, cb = 2, 4, 128, 256, 64
    q, k, planes, ksum, kmax = _setup_k(B, H, D, L, 1)
    s, lv = O.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), L // cb, cb, 1 / math.sqrt(D), reference, True)
    if reference:
        assert not lv.any()
    else:
        assert set(np.unique(lv)) == {0, 1, 2}
    kt = _trunc(O.as_bits(k), lv.transpose(0, 1, 2)[:, None, :, :])       # [B,L,H,D]
    want = np.einsum("blhd,bhd->bhl", O.as_half(kt).astype(np.float64), q[:, 0].astype(np.float64))
    want = want * float(np.float16(1 / math.sqrt(D)))
    got = s[:, :, 0, :L].astype(np.float64)
    assert np.all(np.isnan(s[:, :, 0, L:].astype(np.float32)))
    # fp32 accumulation + one fp16 rounding
    assert np.max(np.abs(got - want)) <= np.max(np.abs(want)) * 2.0 ** -10
    assert ulp_diff_fp16(s[:, :, 0, :L], want.astype(np.float16)).max() <= 1
    sc, lvc = oracle_c.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), L // cb, cb, 1 / math.sqrt(D), reference)
    assert np.array_equal(lvc, lv)
    assert ulp_diff_fp16(sc[:, :, 0, :L], s[:, :, 0, :L]).max() <= 1


def test_k_compute_scale_is_rounded_to_half(oracle_c):
    # with q = one-hot and K = 1.0 the score is exactly half(1/sqrt(D)) as the kernel multiplies
    # by __float2half2_rn(sqrt_dim)
    B, H, D, cb = 1, 4, 128, 64
    k = np.ones((B, cb, H, D), np.float16)
    q = np.zeros((B, 1, H, D), np.float16)
    q[..., 3] = 1
    planes = O.k_planes_alloc(B, H, 2 * cb, D, cb)
    O.k_cache_save(*planes, O.as_bits(k), 1, cb, 0, cb)
    ksum, kmax = O.k_sum_and_max(q, O.colmax_prefill(k))
    for fn in (lambda: O.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), 1, cb, 1 / math.sqrt(D), True),
               lambda: oracle_c.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), 1, cb, 1 / math.sqrt(D), True)[0]):
        s = fn()
        assert np.all(s[:, :, 0, :cb] == np.float16(1 / math.sqrt(D)))
        assert float(s[0, 0, 0, 0]) == 0.08837890625


@pytest.mark.parametrize("reference", [True, False])
def test_v_compute_vs_float64_matmul(oracle_c, reference):
    B, H, D, L = 2, 3, 128, 200
    rng = np.random.default_rng(3)
    _, _, v = make_qkv(B, L, H, D, 2)
    planes = O.v_planes_alloc(B, H, L + 8, D)
    O.v_cache_save(*planes, O.as_bits(v), 0, L)
    p = O.softmax_fp32_to_half((rng.standard_normal((B, H, 1, L + 8)) * 3).astype(np.float16))
    amin = rng.integers(0, 16, (B, H)).astype(np.uint8)
    o, lv = O.v_cache_compute(*planes, O.as_bits(p), amin, L, reference, True)
    if not reference:
        assert len(np.unique(lv)) == 3
    vt = _trunc(O.as_bits(v), lv.transpose(0, 2, 1)[..., None])          # [B,L,H,1]
    want = np.einsum("blhd,bhl->bhd", O.as_half(vt).astype(np.float64), p[:, :, 0, :L].astype(np.float64))
    assert ulp_diff_fp16(o[:, :, 0], want.astype(np.float16)).max() <= 1
    oc, lvc = oracle_c.v_cache_compute(*planes, O.as_bits(p), amin, L, reference)
    assert np.array_equal(lvc, lv)
    assert ulp_diff_fp16(oc, o).max() <= 1


def test_v_test_compute_bruteforce(oracle_c):
    B, H, D, L, K = 2, 3, 8, 96, 32
    rng = np.random.default_rng(4)
    _, _, v = make_qkv(B, L, H, D, 5)
    planes = O.v_planes_alloc(B, H, L, D)
    O.v_cache_save(*planes, O.as_bits(v), 0, L)
    p = O.softmax_fp32_to_half(rng.standard_normal((B, H, 1, L)).astype(np.float16))
    tv, ti = O.bucket_max(p, L, K)
    to = O.v_cache_test_compute(planes[0], O.as_bits(tv), ti, K)
    want = np.zeros((B, H, D))
    for b in range(B):
        for h in range(H):
            for i in range(K):
                col = p[b, h, 0, i::K]
                g = int(np.argmax(col))
                assert ti[b, h, 0, i] == g and tv[b, h, 0, i] == col[g]
                tok = g * K + i
                row = (O.as_bits(v[b, tok, h]).astype(np.uint32) & 0x7F00) | 0x80
                want[b, h] += O.as_half(row.astype(np.uint16)).astype(np.float64) * float(col[g])
    assert ulp_diff_fp16(to[:, :, 0], want.astype(np.float16)).max() <= 1
    toc = oracle_c.v_cache_test_compute(planes[0], O.as_bits(tv), ti, K)
    assert ulp_diff_fp16(toc, to).max() <= 1
    # |v| with the low byte replaced by 0x80 bounds the true |v| from above within 2^-3 relative
    assert np.all(want >= 0)


def test_bucket_max_views_and_ties():
    K = 4
    p = np.array([0.1, 0.5, 0.2, 0.0, 0.1, 0.5, 0.9, 0.0, 0.3, 0.1, 0.9, 0.0], np.float16).reshape(1, 1, 1, 12)
    tv, ti = O.bucket_max(p, 12, K)
    assert tv.reshape(-1).tolist() == [np.float16(0.3), np.float16(0.5), np.float16(0.9), 0.0]
    assert ti.reshape(-1).tolist() == [2, 0, 1, 0]          # first maximal index wins
    # width != valid length: only whole groups of the given view are scanned
    tv, ti = O.bucket_max(p[..., :10], 11, K)
    assert ti.reshape(-1).tolist() == [0, 0, 1, 0] and tv.reshape(-1)[0] == np.float16(0.1)
    # width == valid length, not a multiple: zero padded
    tv, ti = O.bucket_max(p[..., :10], 10, K)
    assert ti.reshape(-1).tolist() == [2, 0, 1, 0] and tv.reshape(-1)[2] == np.float16(0.9)


def test_alignment_min_literal_index_mapping():
    rng = np.random.default_rng(7)
    for B, H, D in ((1, 4, 8), (3, 4, 8), (9, 2, 4)):
        to = (rng.integers(0, 16, (B, H, 1, D)) * 2).astype(np.uint8)
        cm = rng.integers(0, 31, (B, 1, H, D)).astype(np.uint8)
        lit = O.alignment_min(to, cm, True)
        ok = O.alignment_min(to, cm, False)
        for b in range(B):
            for h in range(H):
                f = b * H + h
                b2, h2, h3 = f // (H * H), (f // H) % H, f % H
                assert (b2, h2, h3) == (b // H, b % H, h)
                want = min((int(to[b2, h2, 0, d]) + 15 - int(cm[b2, 0, h3, d])) & 0xFF for d in range(D))
                assert lit[b, h] == want
                assert ok[b, h] == min((int(to[b, h, 0, d]) + 15 - int(cm[b, 0, h, d])) & 0xFF for d in range(D))


def test_test_o_exponent_clears_lsb():
    x = np.array([1.0, 2.0, 0.5, 3.0, 1e-3], np.float16)
    e = O.exponent_bits(x)
    assert np.array_equal(O.test_o_exponent(x), e & 0x1E)
    assert O.test_o_exponent(np.array([1.0], np.float16))[0] == 14     # 15 & 0x1E


def test_colmax_literal_vs_abs():
    x = np.array([[-8.0, 1.0], [0.5, -0.25]], np.float16).T.reshape(1, 2, 1, 2)   # [B,S,H,D]
    lit = O.colmax_prefill(x, True).reshape(-1)
    ab = O.colmax_prefill(x, False).reshape(-1)
    assert lit.tolist() == [15, 14] and ab.tolist() == [18, 14]
    upd = O.colmax_update(O.colmax_prefill(x, True), np.array([-16.0, 0.1], np.float16).reshape(1, 1, 1, 2))
    assert upd.reshape(-1).tolist() == [19, 14]


@pytest.mark.parametrize("prefill,steps,k_block", [(1, 70, 64), (63, 3, 64), (64, 2, 64), (130, 66, 64), (200, 1, 64),
                                                   (1, 70, 256), (200, 130, 256), (320, 2, 256)])
def test_cache_state_machine_and_reference_mode_matches_dense(prefill, steps, k_block):
    B, H, D = 2, 4, 32
    L = prefill + steps
    q, k, v = make_qkv(B, L, H, D, prefill, n_outliers=0)
    rng = np.random.default_rng(9)
    c = O.OracleCache(B, L + 3, H, D, reference=True, k_block=k_block)
    c.save(k[:, :prefill], v[:, :prefill], 0, prefill)
    for t in range(prefill, L):
        qt = rng.standard_normal((B, 1, H, D)).astype(np.float16)
        o = c.decode(qt, k[:, t:t + 1], v[:, t:t + 1])
        assert c.rest_start + c.rest_len == c.cur_len == t + 1 and c.rest_start % 64 == 0
        want = O.dense_attention(qt, k[:, :t + 1], v[:, :t + 1]).astype(np.float32)
        assert np.max(np.abs(o.astype(np.float32) - want)) <= 5e-3   # half-rounded scale + fp16 scores
    # planes hold exactly the first rest_start tokens, whatever mix of prefill and flushes wrote them
    R = c.rest_start
    one = O.OracleCache(B, L + 3, H, D, k_block=k_block)
    if R:
        O.k_cache_save(*one.k_planes, O.as_bits(k[:, :R]), O.cdiv(R, k_block), k_block, 0, R)
        O.v_cache_save(*one.v_planes, O.as_bits(v[:, :R]), 0, R)
    for a, b in zip(c.k_planes + c.v_planes, one.k_planes + one.v_planes):
        assert np.array_equal(a, b)
    assert np.array_equal(c.restk[:, :c.rest_len], k[:, R:L]) and np.array_equal(c.restv[:, :c.rest_len], v[:, R:L])
    assert np.array_equal(c.k_colmax, np.maximum(O.colmax_prefill(k[:, :prefill]),
                                                 O.exponent_bits(k[:, prefill:L]).max(axis=1, keepdims=True)))


def test_aligned_mode_close_to_dense_and_saves_bytes():
    B, H, D, L = 1, 8, 128, 1024
    q, k, v = make_qkv(B, L + 1, H, D, 11)
    c = O.OracleCache(B, L + 64, H, D)
    c.save(k[:, :L], v[:, :L], 0, L)
    o = c.decode(q, k[:, L:], v[:, L:])
    want = O.dense_attention(q, k, v)
    assert np.max(np.abs(o.astype(np.float32) - want.astype(np.float32))) < 2e-2
    by = O.algorithmic_bytes(c.last["k_levels"], c.last["v_levels"], B, H, D, c.last["R"], c.last["L"])
    assert by["total"] < 0.8 * by["dense"]
