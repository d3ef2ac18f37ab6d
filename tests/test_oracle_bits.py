"""Pins the integer / byte half of the oracle: plane split, packing layouts, fetch levels.

Every check is against something the oracle does not itself compute the same way: exhaustive
closed forms, flat-index loops written from the reference kernels' index expressions
(extension/csrc/K_cache.cu:45-56, extension/csrc/V_cache.cu:30-39) and the independent C restatement.
"""
import numpy as np
import pytest

from oracle import akv_oracle as O

ALL = np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_split_and_reconstruct_exhaustive():
    hi, mid, last = O.split_fp16(ALL)
    assert hi.max() == 255 and mid.max() == 15 and last.max() == 15
    a = ALL.astype(np.uint32)
    assert np.array_equal(O.reconstruct(hi, mid, last, 0), ALL)
    assert np.array_equal(O.reconstruct(hi, mid, last, 1), ((a & 0xFFF0) | 0x8).astype(np.uint16))
    assert np.array_equal(O.reconstruct(hi, mid, last, 2), ((a & 0xFF00) | 0x80).astype(np.uint16))


def test_substitution_is_interval_midpoint():
    # For finite values the substituted constant sits in the middle of the dropped-bit interval:
    # the truncation error is at most half the interval (8 ulp at level 1, 128 ulp at level 2).
    hi, mid, last = O.split_fp16(ALL)
    finite = ((ALL >> 10) & 0x1F) != 31
    v = O.as_half(ALL).astype(np.float64)
    for level, n in ((1, 16), (2, 256)):
        r = O.as_half(O.reconstruct(hi, mid, last, level)).astype(np.float64)
        lo = O.as_half((ALL.astype(np.uint32) & ~np.uint32(n - 1)).astype(np.uint16)).astype(np.float64)
        up = O.as_half((ALL.astype(np.uint32) | np.uint32(n - 1)).astype(np.uint16)).astype(np.float64)
        with np.errstate(invalid="ignore"):
            width = np.abs(up - lo)
            err = np.abs(r - v)
        assert np.all(err[finite] <= (width[finite] / 2) * (1 + 1.0 / (n - 1)) + 1e-12)


def test_exponent_bits_exhaustive():
    e = O.exponent_bits(ALL)
    assert np.array_equal(e, ((ALL >> 10) & 0x1F).astype(np.uint8))
    assert O.exponent_bits(np.array([1.5, -2.0, 0.0, 65504.0], np.float16)).tolist() == [15, 16, 0, 30]


def test_c_half_conversions(oracle_c):
    L = oracle_c.lib()
    f = O.as_half(ALL).astype(np.float32)
    for h in list(range(0, 65536, 7)) + [0x7BFF, 0xFBFF, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7C00, 0xFC00]:
        got = L.akvo_half_to_float(h)
        if np.isnan(f[h]):
            assert np.isnan(got)
        else:
            assert got == f[h], hex(h)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                                  2.0 ** -25 * 1.0001, 2.0 ** -14, 6.1e-5, 5.96e-8, np.inf, -np.inf], np.float32)])
    # halfway cases exactly between two fp16 values
    hw = (O.as_half(ALL[:0x7BFF]).astype(np.float64) + O.as_half(ALL[1:0x7C00]).astype(np.float64)) / 2
    x = np.concatenate([x, hw.astype(np.float32), -hw.astype(np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.akvo_float_to_half(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)


def _k_brute(first_8, mid_4, last_4, k_new_u8, bsz, H, n_blocks, n_max_blocks, D, cb, start_pos, seqlen):
    """Flat-index loops transcribed from the expressions of the K prefill kernel."""
    f8, m4, l4 = first_8.reshape(-1), mid_4.reshape(-1), last_4.reshape(-1)
    kn = k_new_u8.reshape(-1)
    sd = cb >> 1
    sb_ = sd * D
    sh = sb_ * n_max_blocks
    sB = sh * H
    nh, ns = D, D * H
    nB = ns * seqlen
    for bx in range(bsz):
        for by in range(H):
            for bz in range(n_blocks):
                for tx in range(D):
                    t0 = bz * cb
                    for seq in range(t0, min(t0 + cb, seqlen)):
                        j = seq - t0
                        base = bx * sB + by * sh + (bz + start_pos // cb) * sb_ + tx * sd
                        src = (bx * nB + seq * ns + by * nh + tx) * 2
                        f8[base * 2 + j] = kn[src + 1]
                        m4[base + (j >> 1)] = (int(m4[base + (j >> 1)]) + ((int(kn[src]) & 0xF0) >> ((j & 1) << 2))) & 0xFF
                        l4[base + (j >> 1)] = (int(l4[base + (j >> 1)]) + ((int(kn[src]) & 0x0F) << (4 - ((j & 1) << 2)))) & 0xFF


@pytest.mark.parametrize("cb,S,start_blk", [(8, 24, 0), (8, 19, 0), (4, 4, 2), (64, 128, 0)])
def test_k_save_layout_bruteforce(oracle_c, cb, S, start_blk):
    rng = np.random.default_rng(cb * 100 + S)
    B, H, D = 2, 3, 4
    Lmax = 6 * cb
    kb = rng.integers(0, 65536, (B, S, H, D)).astype(np.uint16)
    n_blocks = S // cb
    start_pos = start_blk * cb
    planes_np = O.k_planes_alloc(B, H, Lmax, D, cb)
    planes_c = O.k_planes_alloc(B, H, Lmax, D, cb)
    planes_bf = O.k_planes_alloc(B, H, Lmax, D, cb)
    O.k_cache_save(*planes_np, kb, n_blocks, cb, start_pos, S)
    oracle_c.k_cache_save(*planes_c, kb, n_blocks, cb, start_pos, S)
    _k_brute(*planes_bf, kb.view(np.uint8), B, H, n_blocks, Lmax // cb, D, cb, start_pos, S)
    for a, b, c in zip(planes_np, planes_c, planes_bf):
        assert np.array_equal(a, c) and np.array_equal(b, c)
    # semantic read-back: token p, channel d lives at [blk, d, j]; even j in the high nibble
    hi, mid, last = O.split_fp16(kb)
    for p in range(n_blocks * cb):
        blk, j = start_blk + p // cb, p % cb
        assert np.array_equal(planes_np[0][:, :, blk, :, j], hi[:, p])
        nib = planes_np[1][:, :, blk, :, j >> 1]
        assert np.array_equal((nib >> 4) if j % 2 == 0 else (nib & 0xF), mid[:, p])
        nib = planes_np[2][:, :, blk, :, j >> 1]
        assert np.array_equal((nib >> 4) if j % 2 == 0 else (nib & 0xF), last[:, p])
    # untouched blocks stay zero
    touched = np.zeros(Lmax // cb, bool)
    touched[start_blk:start_blk + n_blocks] = True
    assert not planes_np[0][:, :, ~touched].any()


def test_k_save_single_token_branch(oracle_c):
    # seqlen == 1 at a position that is not a block start takes the decoding kernel
    rng = np.random.default_rng(5)
    B, H, D, cb = 2, 2, 4, 8
    planes_np = O.k_planes_alloc(B, H, 32, D, cb)
    planes_c = O.k_planes_alloc(B, H, 32, D, cb)
    toks = rng.integers(0, 65536, (11, B, 1, H, D)).astype(np.uint16)
    for p in range(1, 11):
        O.k_cache_save(*planes_np, toks[p], 0, cb, p, 1)
        oracle_c.k_cache_save(*planes_c, toks[p], 0, cb, p, 1)
    for a, b in zip(planes_np, planes_c):
        assert np.array_equal(a, b)
    hi, mid, last = O.k_planes_fields(*planes_np, 2)
    for p in range(1, 11):
        want = O.reconstruct(hi[:, :, p // cb, :, p % cb], mid[:, :, p // cb, :, p % cb],
                             last[:, :, p // cb, :, p % cb], 0)
        assert np.array_equal(want, toks[p][:, 0])


def _v_brute(first_8, mid_4, last_4, v_new_u8, bsz, H, Lmax, D, start_pos, seq_len, S):
    f8, m4, l4 = first_8.reshape(-1), mid_4.reshape(-1), last_4.reshape(-1)
    vn = v_new_u8.reshape(-1)
    ss = D >> 1
    sh = ss * Lmax
    sB = sh * H
    nh, ns = D, D * H
    nB = ns * S
    for bx in range(bsz):
        for by in range(H):
            for tx in range(D // 2):
                for pos in range(seq_len):
                    dst = bx * sB + by * sh + (pos + start_pos) * ss + tx
                    s0 = (bx * nB + pos * ns + by * nh + tx * 2) * 2
                    s1 = (bx * nB + pos * ns + by * nh + tx * 2 + 1) * 2
                    f8[dst * 2] = vn[s0 + 1]
                    f8[dst * 2 + 1] = vn[s1 + 1]
                    m4[dst] = (int(vn[s0]) & 0xF0) + ((int(vn[s1]) & 0xF0) >> 4)
                    l4[dst] = ((int(vn[s0]) & 0x0F) << 4) + (int(vn[s1]) & 0x0F)


@pytest.mark.parametrize("S,seq_len,start_pos", [(9, 9, 0), (13, 8, 0), (8, 8, 16), (5, 0, 0)])
def test_v_save_layout_bruteforce(oracle_c, S, seq_len, start_pos):
    rng = np.random.default_rng(S)
    B, H, D, Lmax = 2, 3, 6, 32
    vb = rng.integers(0, 65536, (B, S, H, D)).astype(np.uint16)
    pn, pc, pb = (O.v_planes_alloc(B, H, Lmax, D) for _ in range(3))
    O.v_cache_save(*pn, vb, start_pos, seq_len)
    oracle_c.v_cache_save(*pc, vb, start_pos, seq_len)
    _v_brute(*pb, vb.view(np.uint8), B, H, Lmax, D, start_pos, seq_len, S)
    for a, b, c in zip(pn, pc, pb):
        assert np.array_equal(a, c) and np.array_equal(b, c)
    hi, mid, last = O.v_planes_fields(*pn, Lmax)
    got = O.reconstruct(hi, mid, last, 0)[:, :, start_pos:start_pos + seq_len]
    assert np.array_equal(got, vb[:, :seq_len].transpose(0, 2, 1, 3))


def test_k_levels_exhaustive_table():
    mx, sm = np.meshgrid(np.arange(63), np.arange(63), indexing="ij")
    lv = O.k_levels(sm.astype(np.uint8).reshape(1, 1, 63, 63).transpose(0, 1, 2, 3),
                    mx[:, :1].astype(np.uint8).reshape(1, 1, 63, 1))
    for m in range(63):
        for s in range(63):
            d = (m - s) & 0xFF
            want = 2 if d >= 8 else (1 if d >= 4 else 0)
            assert lv[0, m, s] == want
    # the host always has sum <= max, so the table collapses to thresholds on the exponent gap
    assert lv[0, 20, 20] == 0 and lv[0, 20, 17] == 0 and lv[0, 20, 16] == 1 and lv[0, 20, 13] == 1 and lv[0, 20, 12] == 2


def test_v_levels_exhaustive_vs_twos_complement(oracle_c):
    amin = np.arange(256, dtype=np.uint8)
    s = ALL
    lv = O.v_levels(amin.reshape(1, 256), np.broadcast_to(s, (1, 256, 65536)))
    # independent formulation with explicit modular arithmetic on Python-style integers
    A = (amin.astype(np.int64) << 10) % 65536
    A = np.where(A >= 32768, A - 65536, A)
    sb = s.astype(np.int64)
    sb = np.where(sb >= 32768, sb - 65536, sb)
    diff = (A[:, None] - sb[None, :] + 32768) % 65536 - 32768
    want = np.where(diff >= 0x800, 2, np.where(diff >= 0x400, 1, 0)).astype(np.uint8)
    assert np.array_equal(lv[0], want)
    # and the C loop, which uses real `short` arithmetic
    f8, m4, l4 = O.v_planes_alloc(1, 256, 65536, 2)
    _, lv_c = oracle_c.v_cache_compute(f8, m4, l4, np.ascontiguousarray(np.broadcast_to(s, (1, 256, 1, 65536))),
                                       amin.reshape(1, 256), 65536)
    assert np.array_equal(lv_c[0], want)
    # sanity on meaning: for a positive probability p with exponent field e, amin - e >= 2 -> level 2
    p = np.array([0x3C00, 0x3800, 0x3400, 0x3000], np.uint16)   # 1, .5, .25, .125 -> e = 15,14,13,12
    assert O.v_levels(np.array([[15]], np.uint8), p.reshape(1, 1, 4)).reshape(-1).tolist() == [0, 1, 2, 2]
