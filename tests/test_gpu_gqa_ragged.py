"""Grouped-query heads and per-sequence lengths in the fused step.  The oracle is the multi-head oracle run
per sequence on `repeat_kv`-ed keys and values: per query head the algorithm is the reference's."""
import numpy as np
import pytest
import torch

from oracle import akv_oracle as O
from tests.common import assert_step_output, assert_step_stagewise, make_qkv

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("B,Hq,Hkv,lens,steps,D", [(3, 8, 2, [130, 64, 7], 70, 128), (2, 4, 4, [200, 255], 3, 128),
                                                   (4, 16, 2, [63, 127, 128, 1], 66, 128), (2, 8, 1, [300, 190], 5, 128),
                                                   (2, 8, 2, [500, 321], 4, 64), (2, 12, 4, [260, 700], 3, 64),
                                                   (2, 8, 2, [450, 130], 4, 256), (1, 6, 2, [1100], 2, 128),
                                                   (2, 40, 2, [200, 330], 2, 128),
                                                   # K plane blocks of 256 tokens (negative head_dim marks them)
                                                   (3, 8, 2, [130, 64, 7], 70, -128), (2, 16, 1, [700, 255], 66, -128),
                                                   (2, 12, 4, [260, 900], 3, -64), (2, 4, 4, [200, 600], 70, -128)])
def test_gqa_ragged_step_matches_per_sequence_oracle(B, Hq, Hkv, lens, steps, D):
    _ragged_case_against_oracle(B, Hq, Hkv, lens, steps, D)


@pytest.mark.parametrize("listed", [256, -1])
@pytest.mark.parametrize("B,Hq,Hkv,lens,steps,D", [(3, 8, 2, [530, 64, 257], 8, 128), (2, 16, 1, [700, 255], 8, -128),
                                                   (2, 12, 4, [260, 900], 8, -64)])
def test_grouped_v_pass_with_every_pair_listed_and_with_none(monkeypatch, listed, B, Hq, Hkv, lens, steps, D):
    """AKV_TUNE_V_LISTED: up to how many (token, head) pairs below level 2 a wave lists and corrects in tiles of their
    own (256: whatever fits its list, many tiles one after the other; -1: never, the loop that corrects tile by tile)."""
    from alignedkv_amd import load_library
    lib = load_library()
    monkeypatch.setenv("AKV_TUNE_V_LISTED", str(listed))
    lib.akv_reload_tuning()
    try:
        _ragged_case_against_oracle(B, Hq, Hkv, lens, steps, D)
    finally:
        monkeypatch.delenv("AKV_TUNE_V_LISTED")
        lib.akv_reload_tuning()


def _ragged_case_against_oracle(B, Hq, Hkv, lens, steps, D):
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    kb = 256 if D < 0 else 64
    D = abs(D)
    G = Hq // Hkv
    Lmax = max(lens) + steps + 5
    _, k, v = make_qkv(B, Lmax, Hkv, D, seed=sum(lens), n_outliers=4)
    rng = np.random.default_rng(Hq)
    cache = RaggedGQACache(1, B, Lmax, Hq, Hkv, D, k_block=kb)
    cache.record_levels = True
    oracles = []
    for b in range(B):
        cache.prefill(0, b, dev(k[b:b + 1, :lens[b]]), dev(v[b:b + 1, :lens[b]]))
        oc = O.OracleCache(1, Lmax, Hq, D, k_block=kb)
        oc.save(np.repeat(k[b:b + 1, :lens[b]], G, axis=2), np.repeat(v[b:b + 1, :lens[b]], G, axis=2), 0, lens[b])
        oracles.append(oc)
    flips = total = 0
    for s in range(steps):
        # sharper, flat and in-between attention in turn: few, all and some of the tokens below level 2
        q = (rng.standard_normal((B, 1, Hq, D)) * (1.0, 0.0, 0.3, 0.05)[s % 4]).astype(np.float16)
        kn = np.stack([k[b, lens[b] + s] for b in range(B)])[:, None]
        vn = np.stack([v[b, lens[b] + s] for b in range(B)])[:, None]
        out = cache.decode(0, dev(q), dev(kn), dev(vn)).cpu().numpy()
        for b in range(B):
            oc = oracles[b]
            want = oc.decode(q[b:b + 1], np.repeat(kn[b:b + 1], G, axis=2), np.repeat(vn[b:b + 1], G, axis=2))
            L = lens[b] + s + 1
            probs_equal = bool(np.array_equal(O.as_bits(cache.probs[b, :, :L].cpu().numpy()),
                                              O.as_bits(np.ascontiguousarray(oc.last["probs"][0, :, 0, :L]))))
            def stagewise(b=b, oc=oc):
                R_ = oc.rest_start
                return assert_step_stagewise(out[b:b + 1], cache.scores[b:b + 1].cpu().numpy(), cache.probs[b:b + 1].cpu().numpy(), oc, D,
                                             cache.last_alignment_min[b].cpu().numpy() if R_ else None,
                                             cache.last_v_levels[b:b + 1].cpu().numpy() if R_ else None, False, f"step {s} sequence {b}")
            assert_step_output(out[b:b + 1], want, f"ragged grouped step (D={D}, k_block={kb})", probs_equal, stagewise)
            R = oc.rest_start
            if R:
                assert np.array_equal(cache.last_k_levels[b].cpu().numpy(), oc.last["k_levels"][0]), f"K levels, step {s} seq {b}"
                got = cache.last_v_levels[b, :, :R].cpu().numpy()
                flips += int((got != oc.last["v_levels"][0]).sum())
                total += got.size
                # exact for the probabilities and the threshold the kernels produced
                pk = cache.probs[b, :, :R].cpu().numpy()
                amin = cache.last_alignment_min[b].cpu().numpy()
                assert np.array_equal(got, O.v_levels(amin[None], O.as_bits(pk)[None])[0])
        assert cache.seq_lens[0].cpu().tolist() == [l + s + 1 for l in lens]
    assert flips <= max(2, 0.002 * total)
    # planes of every KV head hold what the oracle holds for the query heads of its group
    for b in range(B):
        oc = oracles[b]
        nb = O.cdiv(oc.rest_start, kb)
        for i in range(3):
            got = cache.k_planes[0][i][b, :, :nb].cpu().numpy()
            assert np.array_equal(got, oc.k_planes[i][0, ::G, :nb])
            gotv = cache.v_planes[0][i][b, :, :oc.rest_start].cpu().numpy()
            assert np.array_equal(gotv, oc.v_planes[i][0, ::G, :oc.rest_start])
        assert np.array_equal(cache.k_colmax[0][b, 0].cpu().numpy(), oc.k_colmax[0, 0, ::G])


@pytest.mark.parametrize("k_block", [64, 256])
def test_gqa_reads_each_kv_chunk_for_all_query_heads_consistently(k_block):
    """Uniform lengths through the same entry point (seq_lens=None): grouped heads against the multi-head
    cache fed with repeated keys and values."""
    from types import SimpleNamespace
    from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module as m
    from alignedkv_amd.model.KVCache_AlignedKV import QuantizedCache_AlignedKV
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    B, Hq, Hkv, D, L = 2, 8, 2, 128, 1024
    G = Hq // Hkv
    q, k, v = make_qkv(B, L + 1, Hkv, D, seed=5)
    q = np.random.default_rng(1).standard_normal((B, 1, Hq, D)).astype(np.float16)
    g = RaggedGQACache(1, B, L + 64, Hq, Hkv, D, k_block=k_block)
    for b in range(B):
        g.prefill(0, b, dev(k[b:b + 1, :L]), dev(v[b:b + 1, :L]))
    out_g = g.decode(0, dev(q), dev(k[:, L:]), dev(v[:, L:]))
    cfg = SimpleNamespace(num_hidden_layers=1, num_attention_heads=Hq, num_key_value_heads=Hq, hidden_size=Hq * D,
                          max_position_embeddings=L + 64)
    mha = QuantizedCache_AlignedKV(cfg, B, L + 64, "cuda", torch.half)
    kr, vr = np.repeat(k, G, axis=2), np.repeat(v, G, axis=2)
    mha.key_cache[0].save(dev(kr[:, :L]), 0, L)
    mha.value_cache[0].save(dev(vr[:, :L]), 0, L)
    out_m = mha.auto_compute(dev(q), dev(kr[:, L:]), dev(vr[:, L:]), 0, None)
    # the grouped passes sum in another order (matrix cores): same tolerance as against the oracle
    assert (out_g.float() - out_m.float()).abs().max().item() <= 1e-3


def _as_64_token_blocks(plane, kb):
    """K plane [1, H, NB, D, w * kb / 64 ...] laid out in blocks of kb tokens -> the same bytes in blocks of 64 tokens."""
    if kb == 64:
        return plane
    one, H, NB, D, row = plane.shape
    sub = kb // 64
    return np.ascontiguousarray(plane.reshape(one, H, NB, D, sub, row // sub).transpose(0, 1, 2, 4, 3, 5)).reshape(
        one, H, NB * sub, D, row // sub)


@pytest.mark.parametrize("k_block", [64, 256])
def test_grouped_heads_with_one_length_for_all_sequences_match_the_per_sequence_call(k_block):
    """seq_lens = None (every sequence has cur_len tokens: the token is appended by the middle stage, a full rest buffer
    flushed by the save kernels, no task maps) against the same steps with a length per sequence on the device."""
    from alignedkv_amd.extension._plane_cache import column_block
    from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    B, Hq, Hkv, D, L, steps = 2, 8, 2, 128, 700, 70
    _, k, v = make_qkv(B, L + steps, Hkv, D, seed=11, n_outliers=4)
    rng = np.random.default_rng(2)
    caches = [RaggedGQACache(1, B, L + steps + 64, Hq, Hkv, D, k_block=k_block) for _ in range(2)]
    for c in caches:
        for b in range(B):
            c.prefill(0, b, dev(k[b:b + 1, :L]), dev(v[b:b + 1, :L]))
    u = caches[1]
    for t in range(L, L + steps):
        q = dev(rng.standard_normal((B, 1, Hq, D)).astype(np.float16))
        kn, vn = dev(k[:, t:t + 1]), dev(v[:, t:t + 1])
        want = caches[0].decode(0, q, kn, vn)
        out = torch.empty_like(q)
        cuda_module.decode_step_gqa(u.k_planes[0], u.v_planes[0], u.k_colmax[0], u.v_colmax[0], u.restk[0].view(torch.uint8),
                                    u.restv[0].view(torch.uint8), q.view(torch.uint8), kn.view(torch.uint8),
                                    vn.view(torch.uint8), None, out.view(torch.uint8), u.scores.view(torch.uint8),
                                    u.probs.view(torch.uint8), B, Hq, Hkv, u.n_max_blocks, u.max_seq_len, D, column_block, 32,
                                    t, None, False, None, None, None, k_block=k_block)
        assert torch.equal(out, want), f"step at {t} tokens"
    for a, b_ in zip(caches[0].k_planes[0] + caches[0].v_planes[0], u.k_planes[0] + u.v_planes[0]):
        assert torch.equal(a, b_)
    assert torch.equal(caches[0].restk[0], u.restk[0]) and torch.equal(caches[0].k_colmax[0], u.k_colmax[0])


@pytest.mark.parametrize("k_block", [64, 256])
def test_config3_full_size_against_c_oracle(k_block):
    """C3: 32 query heads over 8 KV heads, head_dim 128, batch 32, lengths uniform in [2048, 8192], K with 4
    outlier channels per KV head x10, V ~ N(0, 0.5).  Every sequence is checked against the C restatement of
    the ops run on its own planes with the KV heads repeated (K planes in blocks of 256 tokens are first rearranged
    into the blocks of 64 the restatement works on)."""
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    from tests.common import oracle_decode_step_c
    B, Hq, Hkv, D, cb = 32, 32, 8, 128, 64
    G = Hq // Hkv
    Lmax = 8192 + cb
    lens = np.random.default_rng(3).integers(2048, 8193, B)
    lens[:4] = [2048, 8191, 4159, 8192]          # block-aligned, two that complete a block with the append, the maximum
    cache = RaggedGQACache(1, B, Lmax, Hq, Hkv, D, k_block=k_block)
    cache.record_levels = True
    gen = torch.Generator(device="cuda").manual_seed(33)
    tails = []
    for b in range(B):
        S = int(lens[b])
        k = torch.randn((1, S, Hkv, D), device="cuda", generator=gen)
        for h in range(Hkv):
            ch = torch.randperm(D, generator=torch.Generator().manual_seed(1000 + h))[:4].cuda()
            k[:, :, h, ch] *= 10.0
        k = k.half()
        v = (0.5 * torch.randn((1, S, Hkv, D), device="cuda", generator=gen)).half()
        cache.prefill(0, b, k, v)
        t = S % cb
        tails.append((k[:, S - t:].cpu().numpy(), v[:, S - t:].cpu().numpy()))
    colmax_k = cache.k_colmax[0].cpu().numpy()
    colmax_v = cache.v_colmax[0].cpu().numpy()
    q = torch.randn((B, 1, Hq, D), device="cuda", generator=gen).half()
    kn = torch.randn((B, 1, Hkv, D), device="cuda", generator=gen).half()
    vn = (0.5 * torch.randn((B, 1, Hkv, D), device="cuda", generator=gen)).half()
    out = cache.decode(0, q, kn, vn).cpu().numpy()
    assert cache.seq_lens[0].cpu().tolist() == [int(l) + 1 for l in lens]
    qh, knh, vnh = q.cpu().numpy(), kn.cpu().numpy(), vn.cpu().numpy()
    worst = 0.0
    flips = total = 0
    moved = dense = 0.0
    for b in range(B):
        L = int(lens[b]) + 1
        R = L // cb * cb
        rk = np.concatenate([tails[b][0], knh[b:b + 1]], axis=1)
        rv = np.concatenate([tails[b][1], vnh[b:b + 1]], axis=1)
        kpl = [_as_64_token_blocks(p[b:b + 1].cpu().numpy(), k_block)[:, :, :R // cb] for p in cache.k_planes[0]]
        vpl = [p[b:b + 1, :, :R].cpu().numpy() for p in cache.v_planes[0]]
        if rk.shape[1] == cb:
            # the append completed a block: what the step wrote into the planes must be the NumPy split of it
            blk = R // cb - 1
            ref_k = O.k_planes_alloc(1, Hkv, cb, D)
            O.k_cache_save(*ref_k, O.as_bits(rk), 1, cb, 0, cb)
            ref_v = O.v_planes_alloc(1, Hkv, cb, D)
            O.v_cache_save(*ref_v, O.as_bits(rv), 0, cb)
            for i in range(3):
                assert np.array_equal(kpl[i][:, :, blk], ref_k[i][:, :, 0]), f"flushed K block, plane {i}, sequence {b}"
                assert np.array_equal(vpl[i][:, :, R - cb:], ref_v[i]), f"flushed V block, plane {i}, sequence {b}"
            rk, rv = rk[:, :0], rv[:, :0]
        rep = lambda a, ax: np.ascontiguousarray(np.repeat(a, G, axis=ax))
        want, klv, vlv, amin, p = oracle_decode_step_c([rep(x, 1) for x in kpl], [rep(x, 1) for x in vpl],
                                                       rep(colmax_k[b:b + 1], 2), rep(colmax_v[b:b + 1], 2), qh[b:b + 1],
                                                       rep(knh[b:b + 1], 2), rep(vnh[b:b + 1], 2), R,
                                                       rest_k=rep(rk, 2), rest_v=rep(rv, 2))
        assert np.array_equal(cache.last_k_levels[b].cpu().numpy(), klv[0]), f"K levels, sequence {b}"
        assert np.array_equal(cache.last_alignment_min[b].cpu().numpy(), amin.reshape(-1)), f"threshold, sequence {b}"
        got_v = cache.last_v_levels[b, :, :R].cpu().numpy()
        got_p = cache.probs[b, :, :R].cpu().numpy()
        assert np.array_equal(got_v, O.v_levels(amin.reshape(1, Hq), O.as_bits(got_p)[None])[0])
        flips += int((got_v != vlv[0]).sum())
        total += got_v.size
        worst = max(worst, float(np.max(np.abs(out[b:b + 1].astype(np.float32) - want.astype(np.float32)))))
        moved += R * ((klv < 3).sum() + 0.5 * (klv < 2).sum() + 0.5 * (klv == 0).sum()) / G \
            + D * ((vlv < 3).sum() + 0.5 * (vlv < 2).sum() + 0.5 * (vlv == 0).sum()) / G
        dense += 2 * Hkv * R * D * 2
    assert worst <= 1e-3, f"max abs err {worst}"
    assert flips <= 1e-3 * total
    print(f"C3: max err {worst:.2e}, V level flips {flips}/{total}, plane bytes per query group {moved / dense:.3f} of dense")


def test_unsupported_combinations_are_refused_before_launch():
    from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module as m
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    B, Hq, Hkv, D = 2, 8, 2, 128
    c = RaggedGQACache(1, B, 256, Hq, Hkv, D)
    q = torch.zeros((B, 1, Hq, D), dtype=torch.half, device="cuda")
    kv = torch.zeros((B, 1, Hkv, D), dtype=torch.half, device="cuda")
    out = torch.empty_like(q)

    def step(**kw):
        args = dict(k_block=None, seq_lens=c.seq_lens[0], cur_len=0)
        args.update(kw)
        m.decode_step_gqa(c.k_planes[0], c.v_planes[0], c.k_colmax[0], c.v_colmax[0], c.restk[0].view(torch.uint8),
                          c.restv[0].view(torch.uint8), q.view(torch.uint8), kv.view(torch.uint8), kv.view(torch.uint8), None,
                          out.view(torch.uint8), c.scores.view(torch.uint8), c.probs.view(torch.uint8), B, Hq, Hkv,
                          c.n_max_blocks, c.max_seq_len, D, 64, 32, args["cur_len"], args["seq_lens"], False,
                          k_block=args["k_block"])

    with pytest.raises(RuntimeError, match="seq_lens"):
        step(seq_lens=c.seq_lens[0].long())
    with pytest.raises(RuntimeError, match="cache full"):
        step(cur_len=256)
    # 256-token K blocks are for multi-head caches; the plane size check of the wrapper comes first for other sizes
    with pytest.raises(RuntimeError):
        step(k_block=256)
    with pytest.raises(RuntimeError):
        step(k_block=128)
    step()   # and the supported call goes through
    assert c.seq_lens[0].cpu().tolist() == [1, 1]
    # 256-token K blocks: up to 16 query heads per KV head, head_dim up to 128
    for hq, d in ((40, 128), (8, 256)):
        c2 = RaggedGQACache(1, B, 256, hq, Hkv, d, k_block=256)
        q2 = torch.zeros((B, 1, hq, d), dtype=torch.half, device="cuda")
        kv2 = torch.zeros((B, 1, Hkv, d), dtype=torch.half, device="cuda")
        with pytest.raises(RuntimeError, match="k_block|K plane blocks"):
            c2.decode(0, q2, kv2, kv2)


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (8, 2)])
def test_captured_step_replays_like_the_eager_step(Hq, Hkv):
    """The step with per-sequence lengths has constant arguments: captured once in a HIP graph and replayed with
    eager work and synchronisations in between, every replay must equal the eager step on a twin cache."""
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    B, D, lens, steps = 3, 128, [190, 62, 700], 8
    Lmax = 1024
    _, k, v = make_qkv(B, Lmax, Hkv, D, seed=3)
    rng = np.random.default_rng(2)
    eager, graphed = RaggedGQACache(1, B, Lmax, Hq, Hkv, D), RaggedGQACache(1, B, Lmax, Hq, Hkv, D)
    for c in (eager, graphed):
        for b in range(B):
            c.prefill(0, b, dev(k[b:b + 1, :lens[b]]), dev(v[b:b + 1, :lens[b]]))
    graph, gq, gk, gv, gout = graphed.capture_decode(0)
    for s in range(steps):
        q = dev(rng.standard_normal((B, 1, Hq, D)).astype(np.float16))
        kn = dev(np.stack([k[b, lens[b] + s] for b in range(B)])[:, None])
        vn = dev(np.stack([v[b, lens[b] + s] for b in range(B)])[:, None])
        want = eager.decode(0, q, kn, vn)
        torch.cuda.synchronize()
        gq.copy_(q); gk.copy_(kn); gv.copy_(vn)
        graph.replay()
        torch.cuda.synchronize()
        # the eager step sizes its launches by the longest sequence, the graph by the capacity: same results
        assert (gout.float() - want.float()).abs().max().item() <= 1e-3, f"replay {s}"
        assert torch.equal(graphed.seq_lens[0], eager.seq_lens[0])
    for i in range(3):
        assert torch.equal(graphed.k_planes[0][i], eager.k_planes[0][i]) and torch.equal(graphed.v_planes[0][i], eager.v_planes[0][i])
