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


# Worst end-to-end output error seen per comparison site, printed at the end of a test run (tests/conftest.py):
# the slack the limits below leave is measured, not assumed.
WORST_STEP_ERR = {}

STEP_TOL = 1e-3          # max-abs bound on attention outputs against the oracle (fp32 accumulate)
STEP_TOL_ROUNDED = 2e-3  # allowed only where the step's fp16 probabilities differ from the oracle's in some bit


def assert_step_output(got, want, label, probs_equal=None):
    """|got - want| <= 1e-3 for one decode step's output.  probs_equal=False (the fp16 probabilities the kernels produced
    differ from the oracle's somewhere: a score rounded to the neighbouring fp16 value under another summation order,
    which moves a sharp softmax row by up to ~0.4 %) widens the bound to 2e-3; probs_equal=True or None holds 1e-3."""
    g = np.asarray(got).astype(np.float32)
    w = np.asarray(want).astype(np.float32)
    err = float(np.max(np.abs(g - w))) if g.size else 0.0
    key = label + ("" if probs_equal is not False else " [probabilities differ]")
    WORST_STEP_ERR[key] = max(WORST_STEP_ERR.get(key, 0.0), err)
    limit = STEP_TOL_ROUNDED if probs_equal is False else STEP_TOL
    assert err <= limit, f"{label}: max abs err {err:.3e} > {limit:g} (probabilities equal: {probs_equal})"
    return err


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
    assert not bad.any(), f"max err {err.max():.3e} (allowed {float((spacing + abs_floor).flat[err.argmax()]):.3e}) at {int(bad.sum())} entries"


def oracle_decode_step_c(k_planes, v_planes, k_colmax, v_colmax, q, k_new, v_new, R, d_block=64, top_k=32,
                         reference=False, rest_k=None, rest_v=None):
    """One decode step with the C restatement of the ops + the NumPy host logic: R tokens in the planes and,
    after the append, the rest buffer given by rest_k/rest_v [B, n_rest, H, D] (default: only the appended
    token; n_rest may be 0 when the append completed a block that the planes already hold).  All arguments
    are NumPy arrays in the reference layouts.  Returns (out [B,1,H,D] float16, k_levels, v_levels, amin, probs)."""
    import math
    from oracle import akv_oracle as O
    from oracle import akv_oracle_c as OC
    B, _, H, D = q.shape
    nb = R // d_block
    kcm2 = O.colmax_update(k_colmax, k_new)
    vcm2 = O.colmax_update(v_colmax, v_new)
    ksum, kmax = O.k_sum_and_max(q, kcm2)
    s, klv = OC.k_cache_compute(*k_planes, ksum, kmax, O.as_bits(q), nb, d_block, 1.0 / math.sqrt(D), reference)
    s = s.copy()
    if rest_k is None:
        rest_k, rest_v = k_new, v_new
    n_rest = rest_k.shape[1]
    restk = np.zeros((B, d_block, H, D), np.float16)
    restv = np.zeros((B, d_block, H, D), np.float16)
    restk[:, :n_rest], restv[:, :n_rest] = rest_k, rest_v
    if n_rest:
        s[:, :, :, R:R + n_rest] = O.rest_scores(q, restk, n_rest, D)
    s[:, :, :, R + n_rest:] = -np.inf
    p = O.softmax_fp32_to_half(s)
    tv, ti = O.bucket_max(p[..., :R], R + n_rest, top_k)
    to = OC.v_cache_test_compute(v_planes[0], O.as_bits(tv), ti, top_k)
    amin = O.alignment_min(O.test_o_exponent(to), vcm2)
    o, vlv = OC.v_cache_compute(*v_planes, O.as_bits(np.ascontiguousarray(p)), amin, R, reference)
    if n_rest:
        o = (o + O.rest_output(p[..., R:R + n_rest], restv, n_rest)).astype(np.float16)
    return o.reshape(B, 1, H, D), klv, vlv, amin, p
