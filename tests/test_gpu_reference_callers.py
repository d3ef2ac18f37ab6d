"""Drives the five ops through `extension.KV_cache_cpp_extention.cuda_module` with exactly the argument forms of the
reference's Python callers, against the oracle with the literal threshold broadcast:
  - prefill save of a sequence that is not a multiple of 64 tokens: the whole tensor is passed with n_blocks = seqlen // 64
    (extension/k_cache_file.py:79-90) and seq_len = seqlen - seqlen % 64 (extension/v_cache_file.py:82-91);
  - flush of the 64-token rest buffer (k_cache_file.py:103-114, v_cache_file.py:103-112);
  - k_cache_compute returns a tensor whose last 64 entries per row the op leaves alone and Python fills in place
    (k_cache_file.py:139-158);
  - the probabilities arrive as the uint8 view of a sliced, non-contiguous tensor together with its row stride, and the
    threshold as the [B,H,H,1] result of the [B,H,1,D] - [B,1,H,D] broadcast (v_cache_file.py:150-186)."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import akv_oracle as O
from tests.common import assert_step_output, assert_step_stagewise, make_qkv

pytestmark = pytest.mark.gpu

CB = 64
TOP = 32


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def exp_u8(x):
    return (x.view(torch.int16) >> 10).to(torch.uint8) & 0x1F


def new_state(B, Lmax, H, D):
    nmb = (Lmax + CB - 1) // CB
    z = lambda *shape: torch.zeros(shape, dtype=torch.uint8, device="cuda")
    return SimpleNamespace(B=B, H=H, D=D, Lmax=Lmax, nmb=nmb,
                           kf8=z(B, H, nmb, D, CB), km4=z(B, H, nmb, D, CB // 2), kl4=z(B, H, nmb, D, CB // 2),
                           vf8=z(B, H, Lmax, D), vm4=z(B, H, Lmax, D // 2), vl4=z(B, H, Lmax, D // 2),
                           kcm=z(B, 1, H, D), vcm=z(B, 1, H, D), restk=None, restv=None, restlen=0, reststart=0, cur=0)


def save_like_the_reference(m, st, new_k, new_v, start_pos, seqlen):
    B, H, D = st.B, st.H, st.D
    st.cur += seqlen
    if start_pos == 0:
        st.kcm = exp_u8(torch.max(new_k, dim=1, keepdim=True).values)
        st.vcm = exp_u8(torch.max(new_v, dim=1, keepdim=True).values)
        m.k_cache_save(st.kf8, st.km4, st.kl4, new_k.view(torch.uint8), B, H, seqlen // CB, st.nmb, D, CB, start_pos, seqlen)
        m.v_cache_save(st.vf8, st.vm4, st.vl4, new_v.view(torch.uint8), B, H, st.Lmax, D, start_pos, seqlen - seqlen % CB)
        st.restk = torch.zeros((B, CB, H, D), dtype=torch.half, device="cuda")
        st.restv = torch.zeros((B, CB, H, D), dtype=torch.half, device="cuda")
        st.restk[:, :seqlen % CB] = new_k[:, seqlen - seqlen % CB:]
        st.restv[:, :seqlen % CB] = new_v[:, seqlen - seqlen % CB:]
        st.restlen = seqlen % CB
        st.reststart = seqlen - st.restlen
        return
    st.kcm = torch.maximum(st.kcm, exp_u8(new_k))
    st.vcm = torch.maximum(st.vcm, exp_u8(new_v))
    st.restk[:, st.restlen:st.restlen + seqlen] = new_k
    st.restv[:, st.restlen:st.restlen + seqlen] = new_v
    st.restlen += seqlen
    if st.restlen == CB:
        m.k_cache_save(st.kf8, st.km4, st.kl4, st.restk.view(torch.uint8), B, H, 1, st.nmb, D, CB, st.reststart, CB)
        m.v_cache_save(st.vf8, st.vm4, st.vl4, st.restv.view(torch.uint8), B, H, st.Lmax, D, st.reststart, st.restlen)
        st.restlen = 0
        st.reststart += CB
        st.restk = torch.zeros_like(st.restk)
        st.restv = torch.zeros_like(st.restv)


def scores_like_the_reference(m, st, q, start_pos, seqlen, poison):
    B, H, D = st.B, st.H, st.D
    ksum = exp_u8(q) + st.kcm
    kmax = torch.max(ksum, dim=3, keepdim=True).values
    s = m.k_cache_compute(st.kf8, st.km4, st.kl4, ksum, kmax, q.view(torch.uint8), B, H, st.reststart // CB, st.nmb, D, CB,
                          st.reststart, 1.0 / math.sqrt(D), False)
    assert s.dtype == torch.uint8 and tuple(s.shape) == (B, H, 1, (st.reststart // CB + 1) * CB * 2)
    s = s.view(torch.half)
    if poison:
        # the op leaves the last 64 entries of a row to the caller: whatever they hold must not matter
        s[..., st.reststart:] = float("nan")
    s_rest = torch.matmul(q.transpose(1, 2), st.restk.transpose(1, 2).transpose(2, 3)[:, :, :, :st.restlen]) / math.sqrt(D)
    s[:, :, :, st.reststart:st.reststart + st.restlen] = s_rest
    s[:, :, :, start_pos + seqlen:] = float("-inf")
    return s


def output_like_the_reference(m, st, s, start_pos, seqlen):
    B, H, D = st.B, st.H, st.D
    R = st.reststart
    s_cut = s[:, :, :, :R]
    assert not s_cut.is_contiguous() or R == s.shape[-1]
    s_test = s_cut if R else s
    # the 32 residue classes: a [G, 32] view reduced over G (zero padding when the row ends at the valid length)
    if start_pos + seqlen == s_test.shape[-1]:
        groups = (start_pos + seqlen + TOP - 1) // TOP
        s_test = F.pad(s_test, (0, groups * TOP - start_pos - seqlen), "constant", 0)
    else:
        groups = s_test.shape[-1] // TOP
    tv, ti = torch.max(s_test.reshape(B, H, groups, TOP), dim=2, keepdim=True)
    ti = ti.to(torch.int32)
    test_o = m.v_cache_test_compute(st.vf8, st.vm4, st.vl4, tv.view(torch.uint8), ti.view(torch.uint8), B, H, st.Lmax, D, TOP)
    test_o_exp = (test_o.view(torch.half).view(torch.int16) >> 10).to(torch.uint8) & 0x1F - 1
    align = test_o_exp + (2 ** 4 - 1) - st.vcm                      # [B,H,1,D] with [B,1,H,D]: [B,H,H,D]
    amin = torch.min(align, dim=-1, keepdim=True).values            # [B,H,H,1]
    assert tuple(amin.shape) == (B, H, H, 1)
    o = m.v_cache_compute(st.vf8, st.vm4, st.vl4, s_cut.view(torch.uint8), amin, B, H, st.Lmax, D, s_cut.stride()[-2], R, False)
    o = o.view(torch.half)
    o += torch.matmul(s[:, :, :, R:start_pos + seqlen], st.restv.transpose(1, 2)[:, :, :st.restlen, :])
    return o, amin


@pytest.mark.parametrize("B,H,D,prefill,steps", [(2, 4, 128, 200, 70), (1, 8, 128, 130, 5), (3, 4, 64, 64, 66)])
def test_five_ops_with_the_reference_callers_argument_forms(B, H, D, prefill, steps):
    from extension.KV_cache_cpp_extention import cuda_module as m
    Lmax = prefill + steps + 10
    _, k, v = make_qkv(B, prefill + steps, H, D, seed=prefill + H)
    rng = np.random.default_rng(prefill)
    st = new_state(B, Lmax, H, D)
    oc = O.OracleCache(B, Lmax, H, D, literal_broadcast=True)
    save_like_the_reference(m, st, dev(k[:, :prefill]), dev(v[:, :prefill]), 0, prefill)
    oc.save(k[:, :prefill], v[:, :prefill], 0, prefill)
    for t in range(prefill, prefill + steps):
        qt = rng.standard_normal((B, 1, H, D)).astype(np.float16)
        q = dev(qt)
        save_like_the_reference(m, st, dev(k[:, t:t + 1]), dev(v[:, t:t + 1]), t, 1)
        s = scores_like_the_reference(m, st, q, t, 1, poison=True)
        p = F.softmax(s.float(), dim=-1).type_as(q)
        o, amin = output_like_the_reference(m, st, p, t, 1)
        out = o.view(B, 1, H, D).cpu().numpy()
        want = oc.decode(qt, k[:, t:t + 1], v[:, t:t + 1])
        assert st.reststart == oc.rest_start and st.restlen == oc.rest_len and st.cur == t + 1
        for got, ref in zip((st.kf8, st.km4, st.kl4, st.vf8, st.vm4, st.vl4), list(oc.k_planes) + list(oc.v_planes)):
            assert np.array_equal(got.cpu().numpy(), ref), f"planes differ after token {t}"
        assert np.array_equal(st.kcm.cpu().numpy(), oc.k_colmax) and np.array_equal(st.vcm.cpu().numpy(), oc.v_colmax)
        pn = p.cpu().numpy()
        probs_equal = bool(np.array_equal(O.as_bits(pn[..., :t + 1]), O.as_bits(np.ascontiguousarray(oc.last["probs"][..., :t + 1]))))
        if oc.rest_start:
            # the threshold entries the op reads (the first B*H bytes of the [B,H,H,1] tensor), for the GPU's own probabilities
            R = oc.rest_start
            tv, ti = O.bucket_max(pn[..., :R], t + 1)
            to = O.v_cache_test_compute(oc.v_planes[0], O.as_bits(tv), ti)
            want_amin = O.alignment_min(O.test_o_exponent(to), oc.v_colmax, True)
            assert np.array_equal(amin.reshape(-1)[:B * H].cpu().numpy().reshape(B, H), want_amin), f"threshold differs at token {t}"
        stagewise = lambda: assert_step_stagewise(out, s[:, :, 0].cpu().numpy(), pn[:, :, 0], oc, D,
                                                  amin.cpu().numpy() if oc.rest_start else None, None, True, f"token {t}")
        assert_step_output(out, want, f"reference callers' forms (D={D})", probs_equal, stagewise)
