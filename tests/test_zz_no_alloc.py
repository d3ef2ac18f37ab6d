"""The allocation-free entry point akv_decode_step_static against akv_decode_step, through the C ABI: two calls in a
row on the same GPU, the second on a smaller cache, each compared bit for bit (same kernels, same order of sums) with
the workspace-taking entry point run from an identical copy of the cache state.  That it allocates nothing is checked
on the device-wide free memory (hipMemGetInfo), which also sees a hipMalloc inside the library, once a first round of
the same calls has loaded the library's code objects and looked up the scratch array's address."""
import ctypes

import numpy as np
import pytest
import torch

from tests.common import make_qkv

pytestmark = pytest.mark.gpu

CB = 64


def _state(B, H, D, L, Lmax, seed, k_block=64):
    """A multi-head cache holding L tokens, filled through the library's own save entry points."""
    import alignedkv_amd
    from alignedkv_amd._lib import check
    lib = alignedkv_amd.load_library()
    q, k, v = make_qkv(B, L + 1, H, D, seed=seed)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    nmb = (Lmax + CB - 1) // CB
    z = lambda *shape: torch.zeros(shape, dtype=torch.uint8, device="cuda")
    st = dict(kf8=z(B, H, nmb, D, CB), km4=z(B, H, nmb, D, CB // 2), kl4=z(B, H, nmb, D, CB // 2),
              vf8=z(B, H, Lmax, D), vm4=z(B, H, Lmax, D // 2), vl4=z(B, H, Lmax, D // 2))
    R = L // CB * CB
    kd, vd = dev(k[:, :L]), dev(v[:, :L])
    stream = torch.cuda.current_stream().cuda_stream
    check(lib.akv_k_cache_save(st["kf8"].data_ptr(), st["km4"].data_ptr(), st["kl4"].data_ptr(), kd.data_ptr(), B, H, L // CB,
                               nmb, D, CB, 0, L, stream), lib)
    check(lib.akv_v_cache_save(st["vf8"].data_ptr(), st["vm4"].data_ptr(), st["vl4"].data_ptr(), vd.data_ptr(), B, H, Lmax, D,
                               0, R, L, stream), lib)
    exp = lambda x: ((x.view(torch.int16) >> 10).to(torch.uint8) & 0x1F)
    st["kcm"] = exp(kd).max(dim=1, keepdim=True).values.contiguous()
    st["vcm"] = exp(vd).max(dim=1, keepdim=True).values.contiguous()
    st["restk"] = torch.zeros((B, CB, H, D), dtype=torch.half, device="cuda")
    st["restv"] = torch.zeros((B, CB, H, D), dtype=torch.half, device="cuda")
    st["restk"][:, :L - R] = kd[:, R:]
    st["restv"][:, :L - R] = vd[:, R:]
    tok = dict(q=dev(q), k_new=dev(k[:, L:]), v_new=dev(v[:, L:]))
    torch.cuda.synchronize()
    return st, tok, nmb, R


def _run(static, st, tok, B, H, D, L, Lmax, nmb, R, literal, check_free=False):
    import alignedkv_amd
    from alignedkv_amd._lib import check
    lib = alignedkv_amd.load_library()
    width = (nmb + 1) * CB
    res = dict(out=torch.zeros((B, 1, H, D), dtype=torch.half, device="cuda"),
               scores=torch.zeros((B, H, width), dtype=torch.half, device="cuda"),
               probs=torch.zeros((B, H, width), dtype=torch.half, device="cuda"),
               klv=torch.zeros((B, H, D), dtype=torch.uint8, device="cuda"),
               vlv=torch.zeros((B, H, max(1, (L + 1) // CB * CB)), dtype=torch.uint8, device="cuda"),
               amin=torch.zeros((B, H), dtype=torch.uint8, device="cuda"))
    head = [st[n].data_ptr() for n in ("kf8", "km4", "kl4", "vf8", "vm4", "vl4", "kcm", "vcm", "restk", "restv")]
    head += [tok["q"].data_ptr(), tok["k_new"].data_ptr(), tok["v_new"].data_ptr(), None, 0, res["out"].data_ptr(),
             res["scores"].data_ptr(), res["probs"].data_ptr(), width]
    rec = [res["klv"].data_ptr(), res["vlv"].data_ptr(), res["amin"].data_ptr()]
    geo = [B, H, nmb, Lmax, D, CB, 32, L, R, L - R, 0, int(literal), torch.cuda.current_stream().cuda_stream]
    if static:
        # no torch allocation between here and the end of the call: the entry point itself must not need any, from
        # torch's allocator or from the device (free memory of the whole GPU, as hipMemGetInfo reports it)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = lib.akv_decode_step_static(*head, *rec, *geo)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        if check_free:
            free_after = torch.cuda.mem_get_info()[0]
            assert free_after == free_before, f"device free memory changed by {free_after - free_before} bytes across the call"
    else:
        need = lib.akv_decode_step_workspace_bytes(B, H, D, Lmax)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        res["ws"] = ws
        rc = lib.akv_decode_step(*head, ws.data_ptr(), ws.numel(), *rec, *geo)
    check(rc, lib)
    torch.cuda.synchronize()
    return res


def _compare(B, H, D, L, literal, seed, check_free=False):
    Lmax = L + 1 + CB
    got, want = {}, {}
    for static, dst in ((True, got), (False, want)):
        st, tok, nmb, R = _state(B, H, D, L, Lmax, seed)
        res = _run(static, st, tok, B, H, D, L, Lmax, nmb, R, literal, check_free)
        dst.update(res)
        dst.update({"state_" + k: v for k, v in st.items()})
    flushed = (L + 1) // CB * CB
    assert torch.equal(got["out"], want["out"]), "outputs differ"
    assert torch.isfinite(got["out"].float()).all() and got["out"].float().abs().max().item() > 0
    assert torch.equal(got["probs"][:, :, :L + 1], want["probs"][:, :, :L + 1])
    assert torch.equal(got["scores"][:, :, :L + 1], want["scores"][:, :, :L + 1])
    assert torch.equal(got["klv"], want["klv"])
    if flushed:
        assert torch.equal(got["vlv"][:, :, :flushed], want["vlv"][:, :, :flushed]) and torch.equal(got["amin"], want["amin"])
    for k in ("kf8", "km4", "kl4", "vf8", "vm4", "vl4", "kcm", "vcm", "restk", "restv"):
        assert torch.equal(got["state_" + k], want["state_" + k]), f"cache state {k} differs after the step"


def test_static_scratch_step_matches_the_workspace_step_twice_in_a_row():
    # first round: the library's code objects are loaded lazily and the scratch array's address is looked up on the first
    # call; second round: the same calls must leave the device's free memory untouched
    for check_free in (False, True):
        print(f"no-alloc step (free memory checked: {check_free}): 4 x 8 heads x 128, 1279 tokens (this step flushes a block), "
              "literal threshold indexing", flush=True)
        _compare(4, 8, 128, 1279, True, seed=31, check_free=check_free)   # four launches: partial sums go through the scratch array
        print("no-alloc step: 2 x 4 heads x 128, 200 tokens", flush=True)
        _compare(2, 4, 128, 200, False, seed=32, check_free=check_free)   # smaller, right after: one workgroup per (batch, head) row
        print("no-alloc step: 1 x 4 heads x 64, 70 tokens", flush=True)
        _compare(1, 4, 64, 70, False, seed=33, check_free=check_free)


def test_static_scratch_step_rejects_shapes_beyond_its_array():
    import alignedkv_amd
    lib = alignedkv_amd.load_library()
    B, H, D, Lmax = 64, 64, 128, 65536
    assert lib.akv_decode_step_workspace_bytes(B, H, D, Lmax) > (32 << 20)
    buf = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    rc = lib.akv_decode_step_static(*([p] * 13), None, 0, p, p, p, Lmax + 64, None, None, None, B, H, Lmax // 64, Lmax, D, 64, 32,
                                    100, 64, 36, 0, 0, None)
    assert rc == 1
    msg = lib.akv_last_error().decode()
    assert "built-in scratch array" in msg and "akv_decode_step" in msg, msg
