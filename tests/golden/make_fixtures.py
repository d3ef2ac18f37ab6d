"""Writes tests/golden/akv_small_cases.npz: small seeded decode cases with everything the NumPy oracle derives
from them (planes, fetch levels, threshold, probabilities, outputs), and tests/golden/akv_gqa_cases.npz: grouped-query
heads with a length per sequence (outputs, K levels and thresholds of every sequence run on its own with repeated KV heads).

The reference ships no tests, golden vectors or fixtures, and its kernels are CUDA (nothing of it can run in this
image), so these vectors come from this repository's own oracle (oracle/akv_oracle.py), whose functions are pinned
by tests/test_oracle_*.py.  They freeze that behaviour: the C restatement, the NumPy oracle of any later state of
the repository and the HIP path are all compared with the same committed numbers.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import akv_oracle as O          # noqa: E402
from tests.common import make_qkv           # noqa: E402

CASES = {   # name: (B, H, D, prefill, steps, k_block, literal_broadcast)
    "mha_d64": (1, 1, 64, 130, 2, 64, False),
    "mha_d128_flush": (1, 1, 128, 62, 3, 64, False),      # the second step fills the rest buffer
    "mha_kblock256": (1, 1, 64, 200, 2, 256, False),
    "mha_literal_broadcast": (2, 2, 64, 64, 1, 64, True),
}


GQA_CASES = {   # name: (Hq, Hkv, D, lengths per sequence, steps, k_block)
    "gqa_g4_kblock256": (4, 1, 128, (270, 130), 2, 256),    # the first sequence has a block of 256 and a tile of the next
    "gqa_g3_d64": (6, 2, 64, (130, 63), 2, 64),             # the second fills its rest buffer with the first step
}


def replay_gqa(Hq, Hkv, D, lens, steps, kb, k, v, q):
    """Grouped-query heads with a length per sequence, as the reference's algorithm defines them: every sequence on its
    own, the KV heads repeated for the query heads of their group.  Returns outputs [steps, B, 1, Hq, D] and, after
    the last step, K levels [B, Hq, D] and thresholds [B, Hq]."""
    G = Hq // Hkv
    B = len(lens)
    outs = np.zeros((steps, B, 1, Hq, D), np.float16)
    klv = np.zeros((B, Hq, D), np.uint8)
    amin = np.zeros((B, Hq), np.uint8)
    for b in range(B):
        oc = O.OracleCache(1, max(lens) + steps + 64, Hq, D, k_block=kb)
        rep = lambda a: np.repeat(a, G, axis=2)
        oc.save(rep(k[b:b + 1, :lens[b]]), rep(v[b:b + 1, :lens[b]]), 0, lens[b])
        for s in range(steps):
            t = lens[b] + s
            outs[s, b] = oc.decode(q[s, b:b + 1], rep(k[b:b + 1, t:t + 1]), rep(v[b:b + 1, t:t + 1]))[0]
        klv[b] = oc.last["k_levels"][0]
        amin[b] = np.asarray(oc.last["amin"]).reshape(-1)
    return outs, klv, amin


def main_gqa():
    out = {}
    for name, (Hq, Hkv, D, lens, steps, kb) in GQA_CASES.items():
        B = len(lens)
        _, k, v = make_qkv(B, max(lens) + steps, Hkv, D, seed=len(name) + sum(lens), n_outliers=4)
        q = np.random.default_rng(sum(lens)).standard_normal((steps, B, 1, Hq, D)).astype(np.float16)
        outs, klv, amin = replay_gqa(Hq, Hkv, D, lens, steps, kb, k, v, q)
        out[name + "/shape"] = np.array([Hq, Hkv, D, steps, kb], np.int32)
        out[name + "/lens"] = np.array(lens, np.int32)
        out[name + "/k"], out[name + "/v"], out[name + "/q"] = O.as_bits(k), O.as_bits(v), O.as_bits(q)
        out[name + "/out"] = O.as_bits(outs)
        out[name + "/k_levels"], out[name + "/amin"] = klv, amin
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "akv_gqa_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


def main():
    out = {}
    for name, (B, H, D, prefill, steps, kb, lit) in CASES.items():
        _, k, v = make_qkv(B, prefill + steps, H, D, seed=len(name) + prefill)
        rng = np.random.default_rng(prefill)
        q = rng.standard_normal((steps, B, 1, H, D)).astype(np.float16)
        c = O.OracleCache(B, prefill + steps + 64, H, D, k_block=kb, literal_broadcast=lit)
        c.save(k[:, :prefill], v[:, :prefill], 0, prefill)
        outs = []
        for s in range(steps):
            outs.append(c.decode(q[s], k[:, prefill + s:prefill + s + 1], v[:, prefill + s:prefill + s + 1]))
        out[name + "/shape"] = np.array([B, H, D, prefill, steps, kb, int(lit)], np.int32)
        out[name + "/k"], out[name + "/v"], out[name + "/q"] = O.as_bits(k), O.as_bits(v), O.as_bits(q)
        out[name + "/out"] = O.as_bits(np.stack(outs))
        nkb = O.cdiv(c.rest_start, kb)
        for i, p in enumerate(c.k_planes):
            assert not p[:, :, nkb:].any()
            out[name + f"/k_plane{i}"] = p[:, :, :nkb]           # the blocks that hold tokens; the rest is zero
        for i, p in enumerate(c.v_planes):
            assert not p[:, :, c.rest_start:].any()
            out[name + f"/v_plane{i}"] = p[:, :, :c.rest_start]
        out[name + "/k_colmax"], out[name + "/v_colmax"] = c.k_colmax, c.v_colmax
        out[name + "/k_levels"], out[name + "/v_levels"] = c.last["k_levels"], c.last["v_levels"]
        out[name + "/amin"] = c.last["amin"]
        out[name + "/probs"] = O.as_bits(c.last["probs"])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "akv_small_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
    main_gqa()
