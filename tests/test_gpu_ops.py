"""GPU parity of the five ops, called through `cuda_module` (ctypes -> C ABI -> HIP kernels), against
the CPU oracle on the same seeded inputs.  Integer outputs (planes, fetch levels) must be
bit-exact; fp16 outputs of the fp32-accumulating kernels must be within 1 fp16 ulp of the oracle
(summation order differs) and within 1e-3 absolute where the magnitudes make that meaningful."""
import math

import numpy as np
import pytest
import torch

from oracle import akv_oracle as O
from tests.common import assert_close_fp16, make_qkv

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mod():
    from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module
    assert torch.cuda.is_available()
    return cuda_module


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def u8(a):
    return dev(a).view(torch.uint8)


def k_planes_dev(B, H, Lmax, D, cb):
    return [dev(p) for p in O.k_planes_alloc(B, H, Lmax, D, cb)]


def v_planes_dev(B, H, Lmax, D):
    return [dev(p) for p in O.v_planes_alloc(B, H, Lmax, D)]


@pytest.mark.parametrize("B,H,D,cb,S,start_blk", [
    (2, 4, 128, 64, 256, 0), (1, 4, 128, 64, 200, 0), (2, 2, 128, 64, 64, 3),
    (2, 3, 8, 8, 24, 0), (1, 2, 64, 64, 128, 1), (1, 1, 256, 64, 64, 0), (1, 2, 20, 16, 48, 0),
    (1, 2, 128, 256, 512, 0), (1, 2, 64, 256, 768, 1), (1, 2, 256, 256, 512, 0), (1, 2, 72, 128, 384, 0),
    (2, 2, 128, 128, 384, 1), (1, 1, 24, 192, 384, 0), (1, 3, 328, 256, 256, 0)])
def test_k_cache_save_bit_exact(mod, B, H, D, cb, S, start_blk):
    rng = np.random.default_rng(S + D)
    kb = rng.integers(0, 65536, (B, S, H, D)).astype(np.uint16)
    Lmax = (start_blk + S // cb + 2) * cb
    want = O.k_planes_alloc(B, H, Lmax, D, cb)
    O.k_cache_save(*want, kb, S // cb, cb, start_blk * cb, S)
    got = k_planes_dev(B, H, Lmax, D, cb)
    mod.k_cache_save(*got, u8(kb), B, H, S // cb, Lmax // cb, D, cb, start_blk * cb, S)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


def test_k_cache_save_from_a_source_that_is_not_16_byte_aligned(mod):
    """The vector kernel wants 16-byte aligned tokens; any other source takes the general kernel, same bytes."""
    B, H, D, cb, S = 1, 2, 128, 64, 128
    rng = np.random.default_rng(5)
    kb = rng.integers(0, 65536, (B, S, H, D)).astype(np.uint16)
    want = O.k_planes_alloc(B, H, 4 * cb, D, cb)
    O.k_cache_save(*want, kb, S // cb, cb, 0, S)
    buf = torch.zeros(kb.nbytes + 8, dtype=torch.uint8, device="cuda")
    src = buf[8:]
    assert src.data_ptr() % 16 == 8
    src.copy_(torch.from_numpy(kb.view(np.uint8).reshape(-1)))
    got = k_planes_dev(B, H, 4 * cb, D, cb)
    mod.k_cache_save(*got, src, B, H, S // cb, 4, D, cb, 0, S)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


def test_k_cache_save_tiles_inside_256_token_blocks(mod):
    """Planes with d_block = 256 filled 64 tokens at a time: a prefill that ends inside a block, then appended tiles
    (defined by the oracle as single-token saves of the reference's decoding branch)."""
    B, H, D, cb = 2, 3, 128, 256
    rng = np.random.default_rng(7)
    kb = rng.integers(0, 65536, (B, 1024, H, D)).astype(np.uint16)
    want = O.k_planes_alloc(B, H, 1024, D, cb)
    got = k_planes_dev(B, H, 1024, D, cb)
    O.k_cache_save(*want, kb[:, :576], 3, cb, 0, 576)                      # 2 blocks + one 64-token tile
    mod.k_cache_save(*got, u8(kb[:, :576]), B, H, 3, 4, D, cb, 0, 576)
    for start, n in ((576, 64), (640, 128), (768, 64)):
        O.k_cache_save(*want, kb[:, start:start + n], 1, cb, start, n, tile_append=True)
        mod.k_cache_save(*got, u8(kb[:, start:start + n]), B, H, 1, 4, D, cb, start, n)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


def test_k_cache_save_single_token_branch(mod):
    rng = np.random.default_rng(1)
    B, H, D, cb = 2, 4, 128, 64
    want = O.k_planes_alloc(B, H, 3 * cb, D, cb)
    got = k_planes_dev(B, H, 3 * cb, D, cb)
    for p in [1, 2, 3, 63, 65, 70, 127, 129]:
        tok = rng.integers(0, 65536, (B, 1, H, D)).astype(np.uint16)
        O.k_cache_save(*want, tok, 0, cb, p, 1)
        mod.k_cache_save(*got, u8(tok), B, H, 0, 3, D, cb, p, 1)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("B,H,D,S,seq_len,start_pos", [
    (2, 4, 128, 256, 256, 0), (2, 4, 128, 100, 64, 0), (1, 3, 128, 64, 64, 192), (2, 3, 6, 13, 8, 5),
    (1, 2, 64, 40, 40, 0), (1, 2, 128, 5, 0, 0)])
def test_v_cache_save_bit_exact(mod, B, H, D, S, seq_len, start_pos):
    rng = np.random.default_rng(S)
    vb = rng.integers(0, 65536, (B, S, H, D)).astype(np.uint16)
    Lmax = start_pos + S + 3
    want = O.v_planes_alloc(B, H, Lmax, D)
    O.v_cache_save(*want, vb, start_pos, seq_len)
    got = v_planes_dev(B, H, Lmax, D)
    mod.v_cache_save(*got, u8(vb), B, H, Lmax, D, start_pos, seq_len)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


def _k_case(B, H, D, L, cb, seed, k_kind="outlier"):
    q, k, _ = make_qkv(B, L, H, D, seed, k_kind, n_outliers=min(4, D // 4))
    planes = O.k_planes_alloc(B, H, L + cb, D, cb)
    O.k_cache_save(*planes, O.as_bits(k), L // cb, cb, 0, L)
    ksum, kmax = O.k_sum_and_max(q, O.colmax_prefill(k))
    return q, planes, ksum, kmax


@pytest.mark.parametrize("reference", [False, True])
@pytest.mark.parametrize("B,H,D,L,cb", [(2, 4, 128, 512, 64), (1, 8, 128, 1024, 64), (3, 2, 128, 320, 64),
                                        (2, 4, 64, 256, 64), (1, 2, 256, 192, 64), (2, 3, 16, 64, 16),
                                        (1, 2, 128, 512, 128), (2, 4, 128, 1024, 256), (1, 3, 64, 768, 256),
                                        (3, 2, 128, 256, 256)])
def test_k_cache_compute_parity(mod, B, H, D, L, cb, reference):
    q, planes, ksum, kmax = _k_case(B, H, D, L, cb, L + D)
    nb = L // cb
    want, want_lv = O.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), nb, cb, 1 / math.sqrt(D), reference, True)
    lv = torch.full((B, H, D), 255, dtype=torch.uint8, device="cuda")
    s = mod.k_cache_compute(*[dev(p) for p in planes], dev(ksum), dev(kmax), u8(q), B, H, nb, planes[0].shape[2], D, cb,
                            L, 1 / math.sqrt(D), reference, levels_out=lv)
    assert s.shape == (B, H, 1, (nb + 1) * cb * 2) and s.dtype == torch.uint8
    got = s.view(torch.half).cpu().numpy()[..., :L]
    assert np.array_equal(lv.cpu().numpy(), want_lv)                         # fetch-decision mask: bit exact
    # terms k*q reach ~1e2 before scaling: fp32 summation-order noise is ~1e-4 on scores near zero
    assert_close_fp16(got, want[..., :L], 3e-4)


def test_k_cache_compute_each_level_isolated(mod):
    # one head per forced level: sum == max (0), max-4 (1), max-8 (2) for every channel but one
    B, H, D, L, cb = 1, 3, 128, 128, 64
    q, planes, _, _ = _k_case(B, H, D, L, cb, 3)
    ksum = np.zeros((B, 1, H, D), np.uint8)
    kmax = np.full((B, 1, H, 1), 20, np.uint8)
    for h, gap in enumerate((0, 4, 8)):
        ksum[0, 0, h] = 20 - gap
    want, want_lv = O.k_cache_compute(*planes, ksum, kmax, O.as_bits(q), 2, cb, 0.1, False, True)
    assert [int(want_lv[0, h, 0]) for h in range(3)] == [0, 1, 2]
    lv = torch.empty((B, H, D), dtype=torch.uint8, device="cuda")
    s = mod.k_cache_compute(*[dev(p) for p in planes], dev(ksum), dev(kmax), u8(q), B, H, 2, 3, D, cb, L, 0.1, False,
                            levels_out=lv)
    assert np.array_equal(lv.cpu().numpy(), want_lv)
    assert_close_fp16(s.view(torch.half).cpu().numpy()[..., :L], want[..., :L], 3e-4)


def test_k_cache_compute_zero_blocks_and_untouched_tail(mod):
    B, H, D, cb = 1, 4, 128, 64
    q, planes, ksum, kmax = _k_case(B, H, D, 128, cb, 5)
    s = mod.k_cache_compute(*[dev(p) for p in planes], dev(ksum), dev(kmax), u8(q), B, H, 0, 3, D, cb, 0, 0.1, False)
    assert s.shape == (B, H, 1, cb * 2)


@pytest.mark.parametrize("B,H,D,L,K", [(2, 4, 128, 256, 32), (1, 3, 8, 96, 32), (2, 2, 64, 64, 16)])
def test_v_cache_test_compute_parity(mod, B, H, D, L, K):
    rng = np.random.default_rng(L)
    _, _, v = make_qkv(B, L, H, D, 7)
    planes = O.v_planes_alloc(B, H, L, D)
    O.v_cache_save(*planes, O.as_bits(v), 0, L)
    p = O.softmax_fp32_to_half(rng.standard_normal((B, H, 1, L)).astype(np.float16) * 2)
    tv, ti = O.bucket_max(p, L, K)
    want = O.v_cache_test_compute(planes[0], O.as_bits(tv), ti, K)
    got = mod.v_cache_test_compute(*[dev(x) for x in planes], u8(tv), u8(ti), B, H, L, D, K)
    assert got.shape == (B, H, 1, 2 * D)
    assert_close_fp16(got.view(torch.half).cpu().numpy(), want, 2e-5)


@pytest.mark.parametrize("reference", [False, True])
@pytest.mark.parametrize("B,H,D,L,n_tok,extra", [(2, 4, 128, 512, 512, 64), (1, 8, 128, 1024, 960, 64),
                                                 (2, 2, 128, 300, 257, 0), (2, 3, 64, 256, 192, 64),
                                                 (1, 2, 256, 128, 128, 64), (2, 3, 6, 50, 37, 3),
                                                 (1, 2, 128, 64, 0, 64), (1, 32, 128, 4096, 4096, 64)])
def test_v_cache_compute_parity(mod, B, H, D, L, n_tok, extra, reference, require_all_levels=True):
    rng = np.random.default_rng(L + n_tok)
    _, _, v = make_qkv(B, L, H, D, 8)
    planes = O.v_planes_alloc(B, H, L + 5, D)
    O.v_cache_save(*planes, O.as_bits(v), 0, L)
    W = n_tok + extra
    p = O.softmax_fp32_to_half(rng.standard_normal((B, H, 1, max(W, 1))).astype(np.float16) * 3)
    # thresholds around the typical probability exponent so that all three levels occur
    amin = rng.integers(6, 14, (B, H)).astype(np.uint8)
    want, want_lv = O.v_cache_compute(*planes, O.as_bits(p), amin, n_tok, reference, True)
    if require_all_levels and not reference and n_tok >= 128 and D >= 64:
        assert len(np.unique(want_lv)) == 3      # (the hand-picked shapes exercise every level)
    pd = dev(p)
    s_cut = pd[:, :, :, :n_tok]                       # sliced view, row stride W (the reference passes this)
    lv = torch.full((B, H, max(n_tok, 1)), 255, dtype=torch.uint8, device="cuda")
    o = mod.v_cache_compute(*[dev(x) for x in planes], s_cut.view(torch.uint8), dev(amin), B, H, L + 5, D,
                            s_cut.stride(-2), n_tok, reference, levels_out=lv)
    assert o.shape == (B, H, 1, 2 * D)
    got = o.view(torch.half).cpu().numpy()
    if n_tok:
        assert np.array_equal(lv.cpu().numpy()[:, :, :n_tok], want_lv)       # fetch-decision mask: bit exact
    assert_close_fp16(got, want, 2e-5)
    assert np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))) <= 1e-3


def test_v_cache_compute_is_deterministic(mod):
    B, H, D, L = 2, 4, 128, 2048
    rng = np.random.default_rng(0)
    _, _, v = make_qkv(B, L, H, D, 9)
    planes = O.v_planes_alloc(B, H, L, D)
    O.v_cache_save(*planes, O.as_bits(v), 0, L)
    pl = [dev(x) for x in planes]
    p = u8(O.softmax_fp32_to_half(rng.standard_normal((B, H, 1, L)).astype(np.float16)))
    amin = dev(np.full((B, H), 9, np.uint8))
    outs = [mod.v_cache_compute(*pl, p, amin, B, H, L, D, L, L, False).cpu() for _ in range(3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_argument_errors_are_raised_before_launch(mod):
    B, H, D, cb = 1, 4, 128, 64
    planes = k_planes_dev(B, H, 128, D, cb)
    k = torch.zeros((B, 64, H, D), dtype=torch.half, device="cuda")
    with pytest.raises(RuntimeError, match="uint8"):
        mod.k_cache_save(*planes, k, B, H, 1, 2, D, cb, 0, 64)
    with pytest.raises(RuntimeError, match="bytes"):
        mod.k_cache_save(*planes, k.view(torch.uint8), B, H, 1, 4, D, cb, 0, 64)       # planes too small for 4 blocks
    with pytest.raises(RuntimeError, match="exceed n_max_blocks"):
        mod.k_cache_save(*planes, k.view(torch.uint8), B, H, 1, 2, D, cb, 128, 64)
    with pytest.raises(RuntimeError, match="GPU|cpu"):
        mod.k_cache_save(*planes, k.cpu().view(torch.uint8), B, H, 1, 2, D, cb, 0, 64)
    vp = v_planes_dev(B, H, 64, D)
    with pytest.raises(RuntimeError, match="outside the plane"):
        mod.v_cache_save(*vp, k.view(torch.uint8), B, H, 64, D, 32, 64)
