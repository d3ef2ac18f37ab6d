"""The committed vectors of tests/golden (made by tests/golden/make_fixtures.py from the NumPy oracle) against
(a) the NumPy oracle as it is now, (b) the C restatement of the ops, and -- marked gpu -- (c) the HIP path through
the host classes.  Planes, column maxima, fetch levels and thresholds are compared bit for bit, attention outputs
within 1e-3 (fp32 accumulation, summation order differs between the implementations)."""
import math
import os
from types import SimpleNamespace

import numpy as np
import pytest

from oracle import akv_oracle as O
from tests.common import assert_step_output

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "akv_small_cases.npz"))
NAMES = sorted({k.split("/")[0] for k in FIX.files})


def case(name):
    B, H, D, prefill, steps, kb, lit = (int(x) for x in FIX[name + "/shape"])
    g = lambda key: FIX[name + "/" + key]
    return SimpleNamespace(B=B, H=H, D=D, prefill=prefill, steps=steps, kb=kb, lit=bool(lit), k=O.as_half(g("k")),
                           v=O.as_half(g("v")), q=O.as_half(g("q")), out=O.as_half(g("out")), g=g)


def replay_oracle(c):
    oc = O.OracleCache(c.B, c.prefill + c.steps + 64, c.H, c.D, k_block=c.kb, literal_broadcast=c.lit)
    oc.save(c.k[:, :c.prefill], c.v[:, :c.prefill], 0, c.prefill)
    outs = [oc.decode(c.q[s], c.k[:, c.prefill + s:c.prefill + s + 1], c.v[:, c.prefill + s:c.prefill + s + 1])
            for s in range(c.steps)]
    return oc, np.stack(outs)


@pytest.mark.parametrize("name", NAMES)
def test_numpy_oracle_reproduces_the_fixture(name):
    c = case(name)
    oc, outs = replay_oracle(c)
    nkb = O.cdiv(oc.rest_start, c.kb)
    for i in range(3):
        assert np.array_equal(oc.k_planes[i][:, :, :nkb], c.g(f"k_plane{i}"))
        assert np.array_equal(oc.v_planes[i][:, :, :oc.rest_start], c.g(f"v_plane{i}"))
    assert np.array_equal(oc.k_colmax, c.g("k_colmax")) and np.array_equal(oc.v_colmax, c.g("v_colmax"))
    assert np.array_equal(oc.last["k_levels"], c.g("k_levels")) and np.array_equal(oc.last["v_levels"], c.g("v_levels"))
    assert np.array_equal(oc.last["amin"], c.g("amin"))
    assert np.array_equal(O.as_bits(outs), c.g("out"))


@pytest.mark.parametrize("name", NAMES)
def test_c_restatement_reproduces_the_fixture(name, oracle_c):
    """The literal-loop C ops on the fixture's planes: levels bit exact, scores and outputs within tolerance."""
    c = case(name)
    oc, _ = replay_oracle(c)          # state after the last step (planes are checked above)
    q = c.q[-1]
    R = oc.rest_start
    if R == 0:
        pytest.skip("no flushed block in this case")
    ksum, kmax = O.k_sum_and_max(q, oc.k_colmax)
    s, klv = oracle_c.k_cache_compute(*oc.k_planes, ksum, kmax, O.as_bits(q), O.cdiv(R, c.kb), c.kb, 1 / math.sqrt(c.D), False)
    assert np.array_equal(klv, c.g("k_levels"))
    want_s = oc.last["scores"][..., :R].astype(np.float32)
    assert np.max(np.abs(s[..., :R].astype(np.float32) - want_s)) <= 2e-3
    p = oc.last["probs"]
    o, vlv = oracle_c.v_cache_compute(*oc.v_planes, O.as_bits(np.ascontiguousarray(p[..., :R])), c.g("amin"), R, False)
    assert np.array_equal(vlv, c.g("v_levels"))
    o = (o + O.rest_output(p[..., R:R + oc.rest_len], oc.restv, oc.rest_len)).astype(np.float16) if oc.rest_len else o
    assert np.max(np.abs(o.reshape(c.B, 1, c.H, c.D).astype(np.float32) - c.out[-1].astype(np.float32))) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_reproduces_the_fixture(name, fused):
    import torch
    from alignedkv_amd.model.KVCache_AlignedKV import QuantizedCache_AlignedKV
    c = case(name)
    cfg = SimpleNamespace(num_hidden_layers=1, num_attention_heads=c.H, num_key_value_heads=c.H, hidden_size=c.H * c.D,
                          max_position_embeddings=c.prefill + c.steps + 64)
    cache = QuantizedCache_AlignedKV(cfg, c.B, c.prefill + c.steps + 64, "cuda", torch.half, literal_broadcast=c.lit, k_block=c.kb)
    cache.fused = fused
    kc, vc = cache.key_cache[0], cache.value_cache[0]
    kc.record_levels = vc.record_levels = True
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    kc.save(dev(c.k[:, :c.prefill]), 0, c.prefill)
    vc.save(dev(c.v[:, :c.prefill]), 0, c.prefill)
    for s in range(c.steps):
        t = c.prefill + s
        out = cache.auto_compute(dev(c.q[s]), dev(c.k[:, t:t + 1]), dev(c.v[:, t:t + 1]), 0, None)
        assert_step_output(out.cpu().numpy(), c.out[s], f"golden fixture {name} (fused={fused})")
    R = kc.reststartpos
    nkb = O.cdiv(R, c.kb)
    got_k = [kc.k_cache_first_8, kc.k_cache_mid_4, kc.k_cache_last_4]
    got_v = [vc.v_cache_first_8, vc.v_cache_mid_4, vc.v_cache_last_4]
    for i in range(3):
        assert np.array_equal(got_k[i][:, :, :nkb].cpu().numpy(), c.g(f"k_plane{i}"))
        assert np.array_equal(got_v[i][:, :, :R].cpu().numpy(), c.g(f"v_plane{i}"))
    assert np.array_equal(kc._colmax.cpu().numpy(), c.g("k_colmax"))
    assert np.array_equal(vc._colmax.cpu().numpy(), c.g("v_colmax"))
    if R:
        assert np.array_equal(kc.last_levels.cpu().numpy(), c.g("k_levels"))
        # V levels depend on the probabilities: a level can flip where one sits on a rounding boundary
        assert (vc.last_levels.cpu().numpy() != c.g("v_levels")).mean() <= 0.01


# ---- grouped-query heads with a length per sequence ---------------------------------------------------------------
GQA = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "akv_gqa_cases.npz"))
GQA_NAMES = sorted({k.split("/")[0] for k in GQA.files})


def gqa_case(name):
    Hq, Hkv, D, steps, kb = (int(x) for x in GQA[name + "/shape"])
    g = lambda key: GQA[name + "/" + key]
    return SimpleNamespace(Hq=Hq, Hkv=Hkv, D=D, steps=steps, kb=kb, lens=[int(x) for x in g("lens")], k=O.as_half(g("k")),
                           v=O.as_half(g("v")), q=O.as_half(g("q")), out=O.as_half(g("out")), g=g)


@pytest.mark.parametrize("name", GQA_NAMES)
def test_numpy_oracle_reproduces_the_grouped_fixture(name):
    from tests.golden.make_fixtures import replay_gqa
    c = gqa_case(name)
    outs, klv, amin = replay_gqa(c.Hq, c.Hkv, c.D, c.lens, c.steps, c.kb, c.k, c.v, c.q)
    assert np.array_equal(O.as_bits(outs), c.g("out"))
    assert np.array_equal(klv, c.g("k_levels")) and np.array_equal(amin, c.g("amin"))


@pytest.mark.gpu
@pytest.mark.parametrize("name", GQA_NAMES)
def test_hip_path_reproduces_the_grouped_fixture(name):
    import torch
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    c = gqa_case(name)
    B = len(c.lens)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    cache = RaggedGQACache(1, B, max(c.lens) + c.steps + 64, c.Hq, c.Hkv, c.D, k_block=c.kb)
    cache.record_levels = True
    for b in range(B):
        cache.prefill(0, b, dev(c.k[b:b + 1, :c.lens[b]]), dev(c.v[b:b + 1, :c.lens[b]]))
    for s in range(c.steps):
        kn = np.stack([c.k[b, c.lens[b] + s] for b in range(B)])[:, None]
        vn = np.stack([c.v[b, c.lens[b] + s] for b in range(B)])[:, None]
        out = cache.decode(0, dev(c.q[s]), dev(kn), dev(vn)).cpu().numpy()
        assert_step_output(out, c.out[s], f"golden grouped fixture {name}")
    for b in range(B):
        if (c.lens[b] + c.steps) // 64:
            assert np.array_equal(cache.last_k_levels[b].cpu().numpy(), c.g("k_levels")[b])
            assert np.array_equal(cache.last_alignment_min[b].cpu().numpy(), c.g("amin")[b])
