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


def assert_step_output(got, want, label, probs_equal=None, stagewise=None):
    """|got - want| <= 1e-3 for one decode step's output against the oracle's, end to end.

    The end-to-end difference is a property of the inputs as much as of the kernels: scores are fp16 (in the reference
    too), and a score that lands on the neighbouring fp16 value under another fp32 summation order moves a sharp softmax
    row by up to 0.8 %.  Where that happened (probs_equal=False: the fp16 probabilities the kernels produced differ from
    the oracle's in some bit) AND the end-to-end difference exceeds 1e-3, the step has to pass stage by stage instead:
    `stagewise()` (see assert_step_stagewise) checks every score within one fp16 value of the oracle's, the probabilities
    as the oracle's softmax of the kernel's own scores, and the output within 1e-3 of the oracle's V side applied to the
    kernel's own probabilities.  No bound above 1e-3 is ever applied to an output."""
    g = np.asarray(got).astype(np.float32)
    w = np.asarray(want).astype(np.float32)
    err = float(np.max(np.abs(g - w))) if g.size else 0.0
    if err <= STEP_TOL or probs_equal is not False or stagewise is None:
        WORST_STEP_ERR[label] = max(WORST_STEP_ERR.get(label, 0.0), err)
        assert err <= STEP_TOL, f"{label}: max abs err {err:.3e} > {STEP_TOL:g} (probabilities equal: {probs_equal})"
        return err
    v_side = stagewise()
    key = label + " [a score on the neighbouring fp16 value: V side on the kernel's own probabilities]"
    WORST_STEP_ERR[key] = max(WORST_STEP_ERR.get(key, 0.0), v_side)
    key = label + " [the same steps end to end, not asserted]"
    WORST_STEP_ERR[key] = max(WORST_STEP_ERR.get(key, 0.0), err)
    return err


def assert_step_stagewise(out, scores, probs, oc, D, amin=None, levels=None, literal_broadcast=False, what=""):
    """One decode step checked stage by stage against the oracle cache `oc` that has just decoded the same token
    (oracle.akv_oracle.OracleCache: oc.last, planes, column maxima and rest buffer are those of this step).
      out [B,1,H,D] fp16, scores / probs [B,H,>=L] fp16: what the kernels produced (mask-free step);
      amin [B,H] uint8 / levels [B,H,R] uint8 (optional): the threshold and V fetch levels the kernels used.
    Checks: every score within one fp16 value of the oracle's (two for the tail, which the reference rounds twice,
    extension/k_cache_file.py:156; 3e-4 per 128 channels where a dot product is much smaller than its terms); the
    probabilities equal to the oracle's softmax OF THESE SCORES (within one fp16 value, nearly all bit for bit); threshold
    and levels bit for bit for these probabilities; the output within 1e-3 of the oracle's V side applied to these
    probabilities.  Returns that last difference."""
    from oracle import akv_oracle as O
    B, _, H, _ = np.asarray(out).shape
    R, L = oc.rest_start, oc.rest_start + oc.rest_len
    sg = np.ascontiguousarray(np.asarray(scores)[:, :, :L])
    pg = np.ascontiguousarray(np.asarray(probs)[:, :, :L])
    so = oc.last["scores"][:, :, 0, :L]
    floor = 3e-4 * max(1, D // 128)
    values_off = ulp_diff_fp16(sg, so)
    finite = np.isfinite(so)
    beyond = np.abs(np.where(finite, sg, 0).astype(np.float32) - np.where(finite, so, 0).astype(np.float32)) > floor
    assert not ((values_off[:, :, :R] > 1) & beyond[:, :, :R]).any(), f"{what}: a score is more than one fp16 value off"
    assert not ((values_off[:, :, R:] > 2) & beyond[:, :, R:]).any(), f"{what}: a tail score is more than two fp16 values off"
    p_own = O.softmax_fp32_to_half(sg[:, :, None, :])[:, :, 0]
    du = ulp_diff_fp16(pg, p_own)
    assert du.max() <= 1 and (du != 0).sum() <= max(4, 0.002 * du.size), f"{what}: softmax of the kernel's scores differs"
    if R:
        tv, ti = O.bucket_max(np.ascontiguousarray(pg[:, :, None, :R]), L)
        to = O.v_cache_test_compute(oc.v_planes[0], O.as_bits(tv), ti)
        want_amin = O.alignment_min(O.test_o_exponent(to), oc.v_colmax, literal_broadcast)
        if amin is not None:
            # (the op sequence with the reference's broadcast hands the op [B,H,H,1]; the op reads the first B*H bytes)
            assert np.array_equal(np.asarray(amin).reshape(-1)[:B * H], want_amin.reshape(-1)), f"{what}: threshold differs"
        if levels is not None:
            assert np.array_equal(np.asarray(levels)[:, :, :R], O.v_levels(want_amin, O.as_bits(np.ascontiguousarray(pg[:, :, :R])))), \
                f"{what}: V levels differ for the kernel's own probabilities"
        o_own, _ = O.v_cache_compute(*oc.v_planes, O.as_bits(np.ascontiguousarray(pg[:, :, None, :R])), want_amin, R, False,
                                     return_levels=True)
    else:
        o_own = np.zeros((B, H, 1, D), np.float16)
    if oc.rest_len:
        o_own = (o_own + O.rest_output(np.ascontiguousarray(pg[:, :, None, R:L]), oc.restv, oc.rest_len)).astype(np.float16)
    v_side = float(np.abs(np.asarray(out).astype(np.float32) - o_own.reshape(B, 1, H, D).astype(np.float32)).max())
    assert v_side <= STEP_TOL, f"{what}: V side on the kernel's own probabilities: {v_side:.3e}"
    return v_side


def assert_outputs_agree(out_a, out_b, probs_a, probs_b, v_abs_max, label, what=""):
    """Two implementations of the same step (say the fused step and the op sequence) on the same cache contents:
    |out_a - out_b| <= 1e-3 + sum_t |p_a[t] - p_b[t]| * max|v| per (batch, head).  Equal probabilities leave the flat
    1e-3; where a probability differs (a score on the neighbouring fp16 value under another summation order, a softmax
    that adds the row up in another order) the outputs may differ by what those probabilities explain, since
    o = sum_t p[t] v[t], and by nothing more.  out_*: [B,1,H,D]; probs_*: [B,H,>=L] fp16 over the same L columns."""
    oa = np.asarray(out_a).astype(np.float32)
    ob = np.asarray(out_b).astype(np.float32)
    dp = np.abs(np.asarray(probs_a).astype(np.float32) - np.asarray(probs_b).astype(np.float32)).sum(-1)    # [B,H]
    limit = STEP_TOL + dp[:, None, :, None] * float(v_abs_max)
    err = np.abs(oa - ob)
    flat = float(err.max())
    WORST_STEP_ERR[label] = max(WORST_STEP_ERR.get(label, 0.0), float((err - (limit - STEP_TOL)).max()))
    assert (err <= limit).all(), f"{label} {what}: outputs differ by {flat:.3e}, probabilities explain {float(limit.max() - STEP_TOL):.3e}"
    return flat


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
                         reference=False, rest_k=None, rest_v=None, k_block=None):
    """One decode step with the C restatement of the ops + the NumPy host logic: R tokens in the planes and,
    after the append, the rest buffer given by rest_k/rest_v [B, n_rest, H, D] (default: only the appended
    token; n_rest may be 0 when the append completed a block that the planes already hold).  All arguments
    are NumPy arrays in the reference layouts; k_block: tokens per block of the K planes (the K op's d_block) when it
    is not the flush unit d_block.  Returns (out [B,1,H,D] float16, k_levels, v_levels, amin, probs)."""
    import math
    from oracle import akv_oracle as O
    from oracle import akv_oracle_c as OC
    B, _, H, D = q.shape
    k_block = d_block if k_block is None else k_block
    nb = (R + k_block - 1) // k_block     # the last block may be partly filled (its other slots are overwritten below)
    kcm2 = O.colmax_update(k_colmax, k_new)
    vcm2 = O.colmax_update(v_colmax, v_new)
    ksum, kmax = O.k_sum_and_max(q, kcm2)
    s, klv = OC.k_cache_compute(*k_planes, ksum, kmax, O.as_bits(q), nb, k_block, 1.0 / math.sqrt(D), reference)
    s = s.copy()
    if s.shape[-1] < R + d_block:
        s = np.concatenate([s, np.zeros(s.shape[:-1] + (R + d_block - s.shape[-1],), s.dtype)], axis=-1)
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
