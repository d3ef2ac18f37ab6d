"""Grouped-query heads and per-sequence lengths in the fused step.  The oracle is the multi-head oracle run
per sequence on `repeat_kv`-ed keys and values: per query head the algorithm is the reference's."""
import numpy as np
import pytest
import torch

from oracle import akv_oracle as O
from tests.common import make_qkv

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("B,Hq,Hkv,lens,steps", [(3, 8, 2, [130, 64, 7], 70), (2, 4, 4, [200, 255], 3),
                                                 (4, 16, 2, [63, 127, 128, 1], 66), (2, 8, 1, [300, 190], 5)])
def test_gqa_ragged_step_matches_per_sequence_oracle(B, Hq, Hkv, lens, steps):
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    D, G = 128, Hq // Hkv
    Lmax = max(lens) + steps + 5
    _, k, v = make_qkv(B, Lmax, Hkv, D, seed=sum(lens), n_outliers=4)
    rng = np.random.default_rng(Hq)
    cache = RaggedGQACache(1, B, Lmax, Hq, Hkv, D)
    cache.record_levels = True
    oracles = []
    for b in range(B):
        cache.prefill(0, b, dev(k[b:b + 1, :lens[b]]), dev(v[b:b + 1, :lens[b]]))
        oc = O.OracleCache(1, Lmax, Hq, D)
        oc.save(np.repeat(k[b:b + 1, :lens[b]], G, axis=2), np.repeat(v[b:b + 1, :lens[b]], G, axis=2), 0, lens[b])
        oracles.append(oc)
    flips = total = 0
    for s in range(steps):
        q = rng.standard_normal((B, 1, Hq, D)).astype(np.float16)
        kn = np.stack([k[b, lens[b] + s] for b in range(B)])[:, None]
        vn = np.stack([v[b, lens[b] + s] for b in range(B)])[:, None]
        out = cache.decode(0, dev(q), dev(kn), dev(vn)).cpu().numpy()
        for b in range(B):
            oc = oracles[b]
            want = oc.decode(q[b:b + 1], np.repeat(kn[b:b + 1], G, axis=2), np.repeat(vn[b:b + 1], G, axis=2))
            err = np.max(np.abs(out[b:b + 1].astype(np.float32) - want.astype(np.float32)))
            assert err <= 2e-3, f"step {s} sequence {b}: max abs err {err}"
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
        nb = oc.rest_start // 64
        for i in range(3):
            got = cache.k_planes[0][i][b, :, :nb].cpu().numpy()
            assert np.array_equal(got, oc.k_planes[i][0, ::G, :nb])
            gotv = cache.v_planes[0][i][b, :, :oc.rest_start].cpu().numpy()
            assert np.array_equal(gotv, oc.v_planes[i][0, ::G, :oc.rest_start])
        assert np.array_equal(cache.k_colmax[0][b, 0].cpu().numpy(), oc.k_colmax[0, 0, ::G])


def test_gqa_reads_each_kv_chunk_for_all_query_heads_consistently():
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
    g = RaggedGQACache(1, B, L + 64, Hq, Hkv, D)
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
    assert torch.equal(out_g, out_m)
