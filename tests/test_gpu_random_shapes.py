"""Seeded random shapes through the stand-alone ops and the grouped ragged step: the case functions of the op tests and
of the grouped-step tests, called with shapes nobody picked by hand (odd batch and head counts, small and large head
dimensions, every K block length, lengths on both sides of the flush boundaries, listed and unlisted corrections)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _op_shapes(seed, n):
    rng = np.random.default_rng(seed)
    for _ in range(n):
        yield dict(B=int(rng.choice([1, 2, 3, 5])), H=int(rng.choice([1, 2, 3, 4, 8, 12])),
                   Dk=int(rng.choice([8, 16, 64, 128, 128, 256])), cb=int(rng.choice([16, 64, 64, 128, 256])),
                   nb=int(rng.integers(1, 12)), ref=bool(rng.random() < 0.3), Lv=int(rng.integers(1, 1500)),
                   frac=float(rng.random()), extra=int(rng.choice([0, 3, 64])), Dv=int(rng.choice([6, 16, 64, 128, 128, 256])),
                   S=int(rng.integers(1, 300)), start=int(rng.integers(0, 100)), Ds=int(rng.choice([8, 24, 64, 128, 256])),
                   cbs=int(rng.choice([8, 16, 64, 128, 256])), nbs=int(rng.integers(1, 6)), sb=int(rng.integers(0, 4)))


@pytest.mark.parametrize("c", list(_op_shapes(3, 16)), ids=lambda c: "B%d-H%d-D%d-cb%d" % (c["B"], c["H"], c["Dk"], c["cb"]))
def test_ops_on_random_shapes(c):
    import tests.test_gpu_ops as T
    from alignedkv_amd.extension.KV_cache_cpp_extention import cuda_module as mod
    B, H = c["B"], c["H"]
    T.test_k_cache_compute_parity(mod, B, H, c["Dk"], c["nb"] * c["cb"], c["cb"], c["ref"])
    T.test_v_cache_compute_parity(mod, B, H, c["Dv"], c["Lv"], int(c["frac"] * c["Lv"]), c["extra"], c["ref"], require_all_levels=False)
    T.test_v_cache_save_bit_exact(mod, B, H, c["Dv"], c["S"] + 5, c["S"], c["start"])
    T.test_k_cache_save_bit_exact(mod, B, H, c["Ds"], c["cbs"], c["nbs"] * c["cbs"], c["sb"])


def _grouped_shapes(seed, n):
    rng = np.random.default_rng(seed)
    for _ in range(n):
        Hkv, G, D = int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 3, 4, 8, 16])), int(rng.choice([64, 128, 128, 256]))
        kb = 256 if D <= 128 and rng.random() < 0.5 else 64
        B = int(rng.choice([1, 2, 3, 5]))
        lens = [int(x) for x in rng.integers(1, 1400, B)]
        steps = int(rng.choice([2, 4, 66]))
        if Hkv * G * D * max(lens) * B > 30e6:
            steps = 2
        yield dict(B=B, Hq=Hkv * G, Hkv=Hkv, D=D, kb=kb, lens=lens, steps=steps, listed=str(rng.choice(["", "256", "-1", "8"])))


@pytest.mark.parametrize("c", list(_grouped_shapes(7, 8)),
                         ids=lambda c: "B%d-%dover%d-D%d-kb%d-listed%s" % (c["B"], c["Hq"], c["Hkv"], c["D"], c["kb"], c["listed"] or "default"))
def test_grouped_ragged_step_on_random_shapes(monkeypatch, c):
    from alignedkv_amd import load_library
    from tests.test_gpu_gqa_ragged import _ragged_case_against_oracle
    lib = load_library()
    if c["listed"]:
        monkeypatch.setenv("AKV_TUNE_V_LISTED", c["listed"])
    lib.akv_reload_tuning()
    try:
        _ragged_case_against_oracle(c["B"], c["Hq"], c["Hkv"], c["lens"], c["steps"], -c["D"] if c["kb"] == 256 else c["D"])
    finally:
        monkeypatch.delenv("AKV_TUNE_V_LISTED", raising=False)
        lib.akv_reload_tuning()
