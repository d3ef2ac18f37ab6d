"""Seeded synthetic inputs shared by the tests, the smoke check and the benchmark."""
import numpy as np


def make_qkv(B, L, H, D, seed=0, k_kind="outlier", n_outliers=4):
    """fp16 inputs with the value distributions of the benchmark configurations:
    q ~ N(0,1); K ~ N(0,1) with `n_outliers` fixed channels per head scaled x10 ("outlier") or
    per-token log-normal scale ("lognormal"); V ~ N(0, 0.5).  Layout [B, L, H, D]."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, 1, H, D), dtype=np.float32)
    k = rng.standard_normal((B, L, H, D), dtype=np.float32)
    if k_kind == "outlier":
        for h in range(H):
            ch = np.random.default_rng(1000 + h).choice(D, size=min(n_outliers, D), replace=False)
            k[:, :, h, ch] *= 10.0
    elif k_kind == "lognormal":
        k *= np.exp(rng.standard_normal((B, L, 1, 1), dtype=np.float32))
    v = 0.5 * rng.standard_normal((B, L, H, D), dtype=np.float32)
    return q.astype(np.float16), k.astype(np.float16), v.astype(np.float16)


def ulp_diff_fp16(a, b):
    """Distance in units of fp16 representable values between two float16 arrays (finite)."""
    def key(x):
        u = np.asarray(x, np.float16).view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a) - key(b))


def assert_close_fp16(got, want, abs_floor):
    """|got - want| <= one fp16 spacing at |want| + abs_floor.  The floor covers the fp32
    accumulation-order noise of a dot product whose result is much smaller than its terms."""
    g = np.asarray(got, np.float16).astype(np.float64)
    w = np.asarray(want, np.float16).astype(np.float64)
    spacing = np.abs(np.spacing(np.asarray(want, np.float16))).astype(np.float64)
    err = np.abs(g - w)
    bad = err > spacing + abs_floor
    assert not bad.any(), f"max err {err.max():.3e} (allowed {float((spacing + abs_floor)[err.argmax()]):.3e}) at {int(bad.sum())} entries"
