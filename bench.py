#!/usr/bin/env python3
"""Benchmark of the AlignedKV decode-attention hot path on one MI355X.

One "step" = one decode step of one layer at the headline configuration: batch 8, 32 heads x 128,
4096 cached tokens in the split-precision planes, append one K/V token per sequence and attend over
the 4097 tokens (K pass, softmax + probe, V pass, combine: one akv_decode_step call).  Inputs are
synthetic and resident in HBM before the timed region: q ~ N(0,1), K ~ N(0,1) with 4 fixed outlier
channels per head scaled x10, V ~ N(0,0.5), fp16 storage, fp32 accumulation.  Steps rotate over
several layers' caches so that no step finds its planes in the 256 MiB last-level cache.

Prints ONE JSON line (see the README of the harness contract): metric value = microseconds per step,
plus `roofline` for the dominant kernel (the K pass), `cpu_baseline` (the C restatement of the
algorithm on the host cores) and a few extra fields (effective bandwidth, bytes versus dense fp16,
the dense baselines).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X published HBM3E bandwidth

PROFILES = os.path.join(ROOT, "profiles")


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def profile_figures(name):
    """Per-kernel figures of a tracked rocprofv3 summary under profiles/ (`<name>_kernel_stats.txt`: average duration in
    us; `<name>_hbm_traffic.txt`: MiB fetched and written per dispatch, already scaled by the known-size copy kernel).
    Returns {kernel: {"avg_us", "fetch_mib", "write_mib"}}; empty when the summaries are not there.  The benchmark
    prints them beside what it measures itself, so a summary that no longer matches the kernels shows up as a mismatch."""
    out = {}
    try:
        for line in open(os.path.join(PROFILES, name + "_kernel_stats.txt")):
            f = line.split()
            if len(f) >= 5 and (line.startswith("akv::") or line.startswith("copy_probe")):
                kernel = line.rsplit(None, 4)[0].strip()     # (split from the right: the name's template arguments hold numbers too)
                out.setdefault(kernel, {})["avg_us"] = float(f[-3])
        for line in open(os.path.join(PROFILES, name + "_hbm_traffic.txt")):
            f = line.split()
            if len(f) >= 6 and (line.startswith("akv::") or line.startswith("copy_probe")):
                kernel = line.rsplit(None, 5)[0].strip()
                out.setdefault(kernel, {}).update(fetch_mib=float(f[-3]), write_mib=float(f[-1]))
    except (OSError, ValueError):
        pass
    return out


def roofline_entry(kernel, algorithmic_bytes, event_us, event_pair_us, prof):
    """Roofline of one kernel: algorithmic bytes per launch over its average launch duration.  The duration is
    measured live with HIP events on the step's stream (interval minus the interval of an empty event pair); when the
    tracked rocprofv3 summary has this kernel, the longer of the two durations is used, so `frac` never exceeds what the
    committed profile supports.  `traffic` = HBM bytes per launch from the tracked FETCH_SIZE / WRITE_SIZE summary."""
    live = max(event_us - event_pair_us, 1e-3)
    prof_us = prof.get("avg_us")
    used = max(live, prof_us) if prof_us else live
    achieved = algorithmic_bytes / (used * 1e-6) / 1e9
    traffic = None
    if "fetch_mib" in prof:
        traffic = int((prof["fetch_mib"] + prof.get("write_mib", 0.0)) * (1 << 20))
    return {"kernel": kernel, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
            "algorithmic_bytes_per_launch": int(algorithmic_bytes), "avg_launch_us": round(used, 2),
            "duration_source": "rocprofv3 summary under profiles/ (longer than the live measurement)" if used != live
            else "HIP events on the step's stream minus an empty event pair",
            "hip_event_interval_us": round(event_us, 2), "event_pair_overhead_us": round(event_pair_us, 2),
            "rocprof_avg_launch_us": prof_us}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--cache-len", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=4, help="caches the steps rotate over")
    ap.add_argument("--k-kind", default="outlier", choices=["outlier", "lognormal"])
    ap.add_argument("--k-block", type=int, default=256, choices=[64, 256],
                    help="tokens per block of the K planes (the ops' d_block): 256 (default) = a nibble row is a whole "
                         "128-byte line, 64 = the block length the reference's Python classes use")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-steps", type=int, default=10)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--q-scale", type=float, default=1.0,
                    help="c2 only: factor on the query (0 or 0.05: flat attention rows, many V tokens below level 2; "
                         "1: the headline workload)")
    ap.add_argument("--extra-capacity", type=int, default=0,
                    help="tokens of cache capacity beyond cache-len + 64 (changes the pitch of the plane rows)")
    ap.add_argument("--workload", default="c2", choices=["c2", "c3"],
                    help="c2: the headline configuration (shape flags apply); c3: grouped-query heads (32 over 8), batch 32, "
                         "lengths uniform in [2048, 8192] -- an extra line, not the headline metric")
    ap.add_argument("--c3-q-heads", type=int, default=32, help="c3 only: query heads over the 8 KV heads")
    ap.add_argument("--c3-len", type=int, default=0, help="c3 only: one length for every sequence instead of U[2048, 8192]")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the short runs of the other workloads (C1, C3, C4) that the headline line carries along")
    ap.add_argument("--profile-run", action="store_true",
                    help="for runs under rocprofv3: leave out the long steady-state loop and the loop through the host API")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB copy kernel (known size, for scaling hardware byte counters)")
    a = ap.parse_args()
    return a


def make_layer_inputs(torch, B, L, H, D, seed, k_kind):
    g = torch.Generator(device="cuda").manual_seed(seed)
    k = torch.randn((B, L, H, D), device="cuda", generator=g)
    if k_kind == "outlier":
        for h in range(H):
            ch = torch.randperm(D, generator=torch.Generator().manual_seed(1000 + h))[:4].cuda()
            k[:, :, h, ch] *= 10.0
    else:
        k *= torch.exp(torch.randn((B, L, 1, 1), device="cuda", generator=g))
    v = 0.5 * torch.randn((B, L, H, D), device="cuda", generator=g)
    return k.half(), v.half()


class StepRunner:
    """Pre-marshalled akv_decode_step_gqa call (multi-head, uniform length) for one layer at a fixed state
    (cur_len = cache_len)."""

    def __init__(self, torch, lib, cache, layer, q, k_new, v_new, out, reference, record, record_probs=True):
        # record_probs False: AKV_STEP_NO_PROBS_RECORD, the probabilities are not copied to memory where the step keeps them on
        # chip (a caller that never reads `probs`); the headline figure is measured with the default, the record kept
        from alignedkv_amd.extension._plane_cache import column_block
        self.lib = lib
        kc, vc = cache.key_cache[layer], cache.value_cache[layer]
        B, H, D = cache.max_batch_size, cache.num_key_value_heads, cache.head_dim
        width = (kc.n_max_blocks + 1) * column_block
        self.scores = torch.empty((B, H, width), dtype=torch.half, device="cuda")
        self.probs = torch.empty((B, H, width), dtype=torch.half, device="cuda")
        need = lib.akv_decode_step_workspace_bytes(B, H, D, cache.max_cache_len)
        self.ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        R = kc.reststartpos
        self.k_levels = torch.empty((B, H, D), dtype=torch.uint8, device="cuda") if record else None
        self.v_levels = torch.empty((B, H, R), dtype=torch.uint8, device="cuda") if record else None
        self.amin = torch.empty((B, H), dtype=torch.uint8, device="cuda") if record else None
        p = lambda t: None if t is None else t.data_ptr()
        self.keep = (q, k_new, v_new, out, kc, vc)
        self.args = [p(kc.k_cache_first_8), p(kc.k_cache_mid_4), p(kc.k_cache_last_4), p(vc.v_cache_first_8),
                     p(vc.v_cache_mid_4), p(vc.v_cache_last_4), p(kc._colmax), p(vc._colmax), p(kc._rest), p(vc._rest),
                     p(q), p(k_new), p(v_new), None, 0, p(out), p(self.scores), p(self.probs), width, p(self.ws),
                     self.ws.numel(), p(self.k_levels), p(self.v_levels), p(self.amin), B, H, H, kc.k_n_max_blocks,
                     cache.max_cache_len, D, column_block, kc.k_block, vc.top_max_k, kc.current_cache_len, None,
                     int(reference), 0 if record_probs else 2, torch.cuda.current_stream().cuda_stream]

        self.cur_len_index = len(self.args) - 5

    def at_length(self, cur_len):
        self.args[self.cur_len_index] = cur_len
        return self

    def __call__(self):
        rc = self.lib.akv_decode_step_gqa(*self.args)
        if rc != 0:
            raise RuntimeError(self.lib.akv_last_error().decode())


def time_steps(torch, runners, steps, warmup):
    n = len(runners)
    for i in range(warmup):
        runners[i % n]()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        runners[i % n]()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_api_path(torch, cache, q, k_new, v_new, L, steps):
    """us/step through the host API the reference's callers use, QuantizedCache_AlignedKV.auto_compute(q, k, v, layer)
    (reference: model/KVCache_AlignedKV.py:126-135), layers rotated: the cache grows token by token from L (no flush of
    the rest buffers inside the timed region), then the host counters go back to L and it starts over.  Returns
    (us per step by the wall clock, host microseconds per call with the device left to run behind)."""
    layers = len(cache.key_cache)
    grow = 60

    def rewind():
        for c in list(cache.key_cache) + list(cache.value_cache):
            c.__dict__["current_cache_len"] = L
            c.__dict__["_restlen"] = 0

    def run(n):
        done = 0
        while done < n:
            for s in range(grow):
                for layer in range(layers):
                    cache.auto_compute(q, k_new, v_new, layer)
                done += layers
                if done >= n:
                    break
            rewind()
        return done

    run(max(steps // 10, 2 * layers))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = run(steps)
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    rewind()
    return (t2 - t0) / n * 1e6, (t1 - t0) / n * 1e6


def step_percentiles(torch, runners, steps, batch=20):
    """us/step over batches of `batch` consecutive steps (events on the current stream between the batches, one
    synchronisation at the end): p10 / median / p90 of the batch means."""
    n = len(runners)
    nb = max(steps // batch, 5)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(nb + 1)]
    ev[0].record()
    k = 0
    for b in range(nb):
        for _ in range(batch):
            runners[k % n]()
            k += 1
        ev[b + 1].record()
    torch.cuda.synchronize()
    us = sorted(ev[b].elapsed_time(ev[b + 1]) * 1e3 / batch for b in range(nb))
    pick = lambda f: us[min(len(us) - 1, int(f * len(us)))]
    return {"p10": round(pick(0.1), 2), "median": round(pick(0.5), 2), "p90": round(pick(0.9), 2),
            "sample": "%d batches of %d consecutive steps, HIP events between batches" % (nb, batch)}


def phase_times(torch, lib, runners, steps):
    """Average duration (us) of the four kernels of the step, HIP events on the step's stream."""
    import ctypes
    lib.akv_profile_enable(1)
    buf = (ctypes.c_float * 4)()
    empty = ctypes.c_float()
    acc = [0.0] * 5
    n = len(runners)
    for i in range(8):
        runners[i % n]()
    torch.cuda.synchronize()
    for i in range(steps):
        runners[i % n]()
        if lib.akv_profile_read(buf) != 0 or lib.akv_profile_read_empty(ctypes.byref(empty)) != 0:
            raise RuntimeError(lib.akv_last_error().decode())
        for j in range(4):
            acc[j] += buf[j] * 1e3
        acc[4] += empty.value * 1e3
    lib.akv_profile_enable(0)
    # raw intervals, and what an event pair around nothing measures (a few microseconds)
    return [a / steps for a in acc[:4]], acc[4] / steps


def algorithmic_bytes(k_levels, v_levels, B, H, D, R, L, top_k=32):
    """Bytes one decode step has to move given the fetch levels (0: all planes, 1: no last_4, 2: high byte
    only): per plane element 1 + 1/2 [level < 2] + 1/2 [level == 0] bytes, plus the fp16 tail, q, the
    score row written by the K side and one row of the same size read by the V side (the scores, where the
    probabilities stay on chip; the probabilities, where a kernel of its own turns the scores into them) and the
    probe rows.  Dense fp16 reads 2 bytes per K and per V element."""
    tail = L - R
    k_plane = float(R) * (k_levels.size + 0.5 * (k_levels < 2).sum() + 0.5 * (k_levels == 0).sum())
    v_plane = float(D) * (v_levels.size + 0.5 * (v_levels < 2).sum() + 0.5 * (v_levels == 0).sum())
    k_other = B * H * tail * D * 2 + B * H * D * 3 + B * H + B * H * L * 2
    v_other = B * H * top_k * D + B * H * L * 2 + B * H * tail * D * 2 + B * H * D * 2
    return dict(k_plane=k_plane, v_plane=v_plane, total=k_plane + v_plane + k_other + v_other,
                dense=float(2 * B * H * L * D * 2),
                f_mid_k=float((k_levels < 2).mean()), f_last_k=float((k_levels == 0).mean()),
                f_mid_v=float((v_levels < 2).mean()), f_last_v=float((v_levels == 0).mean()))


def cpu_baseline(torch, cache, q, k_new, v_new, n_steps):
    """The C restatement of the algorithm (oracle/akv_oracle.c, OpenMP) on the host cores, same inputs:
    one full-size decode step (planes already flushed, one tail token), timed n_steps times."""
    import numpy as np
    from oracle import akv_oracle as O
    from oracle import akv_oracle_c as OC
    kc, vc = cache.key_cache[0], cache.value_cache[0]
    B, H, D = cache.max_batch_size, cache.num_key_value_heads, cache.head_dim
    R, cb, kb = kc.reststartpos, 64, kc.k_block
    nb = (R + kb - 1) // kb
    kp = [t.cpu().numpy() for t in (kc.k_cache_first_8, kc.k_cache_mid_4, kc.k_cache_last_4)]
    vp = [t.cpu().numpy() for t in (vc.v_cache_first_8, vc.v_cache_mid_4, vc.v_cache_last_4)]
    kcm, vcm = kc._colmax.cpu().numpy(), vc._colmax.cpu().numpy()
    qn, kn, vn = (t.cpu().numpy() for t in (q, k_new, v_new))
    OC.lib()
    times = []
    out = None
    for _ in range(n_steps):
        t0 = time.perf_counter()
        kcm2 = O.colmax_update(kcm, kn)
        vcm2 = O.colmax_update(vcm, vn)
        ksum, kmax = O.k_sum_and_max(qn, kcm2)
        s, klv = OC.k_cache_compute(*kp, ksum, kmax, O.as_bits(qn), nb, kb, 1.0 / math.sqrt(D), False)
        s = s.copy()
        restk = np.zeros((B, cb, H, D), np.float16)
        restv = np.zeros((B, cb, H, D), np.float16)
        restk[:, :1], restv[:, :1] = kn, vn
        s[:, :, :, R:R + 1] = O.rest_scores(qn, restk, 1, D)
        s[:, :, :, R + 1:] = -np.inf
        p = O.softmax_fp32_to_half(s)
        tv, ti = O.bucket_max(p[..., :R], R + 1)
        to = OC.v_cache_test_compute(vp[0], O.as_bits(tv), ti, 32)
        amin = O.alignment_min(O.test_o_exponent(to), vcm2)
        o, vlv = OC.v_cache_compute(*vp, O.as_bits(np.ascontiguousarray(p)), amin, R, False)
        o = (o + O.rest_output(p[..., R:R + 1], restv, 1)).astype(np.float16)
        times.append(time.perf_counter() - t0)
        out = o
    return min(times), out.reshape(B, 1, H, D), klv, vlv, OC.num_threads()


def cpu_dense_torch(torch, B, H, D, L, n_steps=10, warm=3):
    """Dense attention as the reference's model file computes it (model/Llama_AlignedKV.py:119-140: fp16
    tensors, fp32 softmax) with torch on the host cores, one step over L tokens.  Returns (seconds, threads)."""
    g = torch.Generator().manual_seed(1)
    q = torch.randn((B, 1, H, D), generator=g).half()
    k = torch.randn((B, L, H, D), generator=g).half()
    v = torch.randn((B, L, H, D), generator=g).half()
    kt, vt = k.permute(0, 2, 3, 1), v.transpose(1, 2)
    times = []
    for i in range(warm + n_steps):
        t0 = time.perf_counter()
        s = torch.matmul(q.transpose(1, 2), kt) / math.sqrt(D)
        pr = torch.softmax(s.float(), dim=-1).type_as(q)
        torch.matmul(pr, vt).transpose(1, 2).contiguous()
        if i >= warm:
            times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], torch.get_num_threads()


def bench_c3(a):
    """Grouped-query, ragged-length decode step (akv_decode_step_gqa) at batch 32, 32 query heads over 8 KV
    heads x 128, lengths uniform in [2048, 8192].  In the timed loop the lengths advance by themselves as in a decode
    loop (the step increments them on the device, sequences whose rest buffer fills flush it); every `grow` steps of
    a layer they are set back to the drawn lengths, so the workload stays the one named."""
    import numpy as np
    import torch
    import alignedkv_amd
    from alignedkv_amd.model.ragged_gqa_cache import RaggedGQACache
    lib = alignedkv_amd.load_library()
    B, Hq, Hkv, D, cb = 32, a.c3_q_heads, 8, 128, 64
    Lmax = 8192 + cb + a.extra_capacity
    lens = np.random.default_rng(a.seed + 3).integers(2048, 8193, B)
    if a.c3_len:
        lens[:] = a.c3_len
    cache = RaggedGQACache(a.layers, B, Lmax, Hq, Hkv, D, k_block=a.k_block)
    for layer in range(a.layers):
        for b in range(B):
            k, v = make_layer_inputs(torch, 1, int(lens[b]), Hkv, D, a.seed + 100 * layer + b, "outlier")
            cache.prefill(layer, b, k, v)
    g = torch.Generator(device="cuda").manual_seed(a.seed + 999)
    q = torch.randn((B, 1, Hq, D), device="cuda", generator=g).half()
    k_new = torch.randn((B, 1, Hkv, D), device="cuda", generator=g).half()
    v_new = (0.5 * torch.randn((B, 1, Hkv, D), device="cuda", generator=g)).half()
    lens0 = torch.from_numpy(lens.astype(np.int32)).cuda()
    bound = int(lens.max())
    cache.record_levels = True

    grow = 32       # steps of a layer between two resets of its lengths (the longest sequence stays inside the capacity)

    def run(reference, steps, warmup):
        cache.reference = reference
        t0 = 0.0
        for i in range(warmup + steps):
            if i == warmup:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
            layer = i % a.layers
            if (i // a.layers) % grow == 0:
                cache.seq_lens[layer].copy_(lens0)
                cache.len_bound[layer] = bound
            cache.decode(layer, q, k_new, v_new)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    cache.record_levels = True
    cache.seq_lens[0].copy_(lens0)
    cache.len_bound[0] = bound
    cache.decode(0, q, k_new, v_new)
    klv = cache.last_k_levels.cpu().numpy()
    vlv = cache.last_v_levels.cpu().numpy()
    cache.record_levels = False
    kv_bytes = dense = 0.0
    for b in range(B):
        R = (int(lens[b]) + 1) // cb * cb
        # a KV element is fetched at the finest level any query head of its group asks for
        kl = klv[b].reshape(Hkv, Hq // Hkv, D).min(1)
        vl = vlv[b, :, :R].reshape(Hkv, Hq // Hkv, R).min(1)
        kv_bytes += R * (kl.size + 0.5 * (kl < 2).sum() + 0.5 * (kl == 0).sum())
        kv_bytes += D * (vl.size + 0.5 * (vl < 2).sum() + 0.5 * (vl == 0).sum())
        dense += 2 * Hkv * (int(lens[b]) + 1) * D * 2
    sec = run(False, a.steps, a.warmup)
    sec_ref = run(True, max(a.steps // 2, 20), 10)
    cache.reference = False
    lib.akv_profile_enable(1)
    import ctypes
    buf = (ctypes.c_float * 4)()
    empty = ctypes.c_float()
    acc = [0.0] * 4
    acc_raw = [0.0] * 4
    empty_us = 0.0
    n = min(a.steps, 100)
    for i in range(n + 4):
        layer = i % a.layers
        cache.seq_lens[layer].copy_(lens0)
        cache.len_bound[layer] = bound
        cache.decode(layer, q, k_new, v_new)
        lib.akv_profile_read(buf)
        lib.akv_profile_read_empty(ctypes.byref(empty))
        if i >= 4:
            for j in range(4):
                acc[j] += max(buf[j] - empty.value, 0.0) * 1e3 / n
                acc_raw[j] += buf[j] * 1e3 / n
            empty_us += empty.value * 1e3 / n
    lib.akv_profile_enable(0)
    # bytes of the K pass per launch: plane rows at the finest level any query head of the group asks for, q, column
    # maxima, new keys, scores written
    k_plane_bytes = 0.0
    for b in range(B):
        R = (int(lens[b]) + 1) // cb * cb
        kl = klv[b].reshape(Hkv, Hq // Hkv, D).min(1)
        k_plane_bytes += R * (kl.size + 0.5 * (kl < 2).sum() + 0.5 * (kl == 0).sum())
    k_pass_bytes = k_plane_bytes + B * Hq * D * 2 + B * Hkv * D * 3 + sum((int(l) + 1) // cb * cb for l in lens) * Hq * 2
    prof = profile_figures("decode_step_c3_gqa") if (a.c3_q_heads == 32 and not a.c3_len and a.k_block == 256) else {}
    k_kernel = "akv::mfma_k_pass_kernel<%d, false" % D
    k_prof = next((v for k, v in prof.items() if k.startswith(k_kernel)), {})
    res = {"metric": "decode-attn us/step, grouped-query 32 over 8 heads x 128, batch 32, lengths U[2048,8192]",
           "value": round(sec * 1e6, 2), "unit": "us/step", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "ms_per_step": round(sec * 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic",
           "config": {"workload": "C3: batch 32, 32 query heads over 8 KV heads x 128, %d cached tokens in total, "
                                  "%d layers rotated, K plane blocks of %d tokens" % (int(lens.sum()), a.layers, a.k_block)},
           "kv_plane_bytes_union_of_group_levels": int(kv_bytes), "dense_fp16_bytes": int(dense),
           "bytes_vs_dense": round(kv_bytes / dense, 4),
           "effective_hbm_gbps": round(kv_bytes / sec / 1e9, 1), "pct_hbm_peak": round(100 * kv_bytes / sec / 1e9 / HBM_PEAK_GBPS, 1),
           "kernel_us": {"k_pass": round(acc[0], 2), "middle": round(acc[1], 2), "v_pass": round(acc[2], 2),
                         "combine": round(acc[3], 2)},
           "dense_in_planes_us": round(sec_ref * 1e6, 2), "speedup_vs_dense_in_planes": round(sec_ref / sec, 3),
           "roofline": roofline_entry(k_kernel, k_pass_bytes, acc_raw[0], empty_us, k_prof),
           "roofline_step": {"bound": "hbm", "achieved": round(kv_bytes / sec / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                             "frac": round(kv_bytes / sec / 1e9 / HBM_PEAK_GBPS, 4), "algorithmic_bytes_per_step": int(kv_bytes),
                             "us_per_step": round(sec * 1e6, 2), "duration_source": "wall clock around the timed steps"}}
    if not a.no_cpu:
        res.update(cpu_baseline_c3(torch, cache, lens, q, k_new, v_new, lens0, bound))
    print(json.dumps(res))


def cpu_baseline_c3(torch, cache, lens, q, k_new, v_new, lens0, bound):
    """The C restatement of the ops (OpenMP) + the NumPy host logic on the host cores for the grouped-query workload: every
    sequence on its own planes with the KV heads repeated per query head, one full-size step of layer 0 (what the
    reference's multi-head algorithm does for each query head).  Also the parity of the GPU step against it."""
    import numpy as np
    from oracle import akv_oracle_c as OC
    from tests.common import oracle_decode_step_c
    B, Hq, Hkv, D, cb, kb = cache.bsz, cache.n_q_heads, cache.n_kv_heads, cache.head_dim, 64, cache.k_block
    G = Hq // Hkv
    cache.record_levels = True
    cache.seq_lens[0].copy_(lens0)
    cache.len_bound[0] = bound
    out = cache.decode(0, q, k_new, v_new).cpu().numpy()
    klv_gpu = cache.last_k_levels.cpu().numpy()
    cache.record_levels = False
    OC.lib()
    rep = lambda x, ax: np.ascontiguousarray(np.repeat(x, G, axis=ax))

    def as_64(plane):      # K plane in blocks of kb tokens -> the same bytes in blocks of 64 tokens
        if kb == 64:
            return plane
        one, H, NB, D_, row = plane.shape
        sub = kb // 64
        return np.ascontiguousarray(plane.reshape(one, H, NB, D_, sub, row // sub).transpose(0, 1, 2, 4, 3, 5)).reshape(
            one, H, NB * sub, D_, row // sub)

    qh, knh, vnh = q.cpu().numpy(), k_new.cpu().numpy(), v_new.cpu().numpy()
    kcm, vcm = cache.k_colmax[0].cpu().numpy(), cache.v_colmax[0].cpu().numpy()
    restk, restv = cache.restk[0].cpu().numpy(), cache.restv[0].cpu().numpy()
    seconds, worst, k_equal = 0.0, 0.0, True
    for b in range(B):
        Lb = int(lens[b]) + 1
        R = Lb // cb * cb
        n_rest = Lb - R
        kpl = [rep(as_64(p[b:b + 1].cpu().numpy())[:, :, :R // cb], 1) for p in cache.k_planes[0]]
        vpl = [rep(p[b:b + 1, :, :R].cpu().numpy(), 1) for p in cache.v_planes[0]]
        args = (kpl, vpl, rep(kcm[b:b + 1], 2), rep(vcm[b:b + 1], 2), qh[b:b + 1], rep(knh[b:b + 1], 2), rep(vnh[b:b + 1], 2), R)
        rk, rv = rep(restk[b:b + 1, :n_rest], 2), rep(restv[b:b + 1, :n_rest], 2)
        t0 = time.perf_counter()
        want, klv, vlv, amin, p = oracle_decode_step_c(*args, rest_k=rk, rest_v=rv)
        seconds += time.perf_counter() - t0
        worst = max(worst, float(np.max(np.abs(out[b:b + 1].astype(np.float32) - want.astype(np.float32)))))
        k_equal = k_equal and bool(np.array_equal(klv_gpu[b], klv[0]))
    return {"cpu_baseline": {"value": round(seconds * 1e6, 1), "unit": "us/step", "cores": OC.num_threads(), "kind": "port",
                             "cpu_model": cpu_model(), "host_cores": os.cpu_count(),
                             "sample": "one full-size step of layer 0, sequence by sequence (C restatement with OpenMP + NumPy "
                                       "host logic, KV heads repeated per query head; copies to the host not timed)"},
            "parity": {"max_abs_err_vs_oracle": worst, "k_levels_equal": k_equal}}


def other_workloads(a):
    """Short runs of the configurations that are not the headline (C1, C4: the multi-head step at other shapes; C3:
    grouped-query heads with a length per sequence), each in a process of its own: us/step and per-kernel times for the
    same line.  A run that fails is reported as such and does not touch the headline figure."""
    import subprocess
    # (step counts that outlast the few milliseconds after an idle period in which the device runs slower)
    runs = {"c1": ["--batch", "1", "--cache-len", "1024", "--k-block", "64", "--steps", "3000", "--warmup", "500"],
            "c3": ["--workload", "c3", "--steps", "300", "--warmup", "60"],
            "c4": ["--batch", "4", "--cache-len", "32768", "--k-kind", "lognormal", "--steps", "200", "--warmup", "40"]}
    out = {}
    for name, extra in runs.items():
        cmd = [sys.executable, os.path.abspath(__file__), "--no-cpu", "--no-extras", "--seed", str(a.seed)] + extra
        try:
            r = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
            d = json.loads(r.stdout.strip().splitlines()[-1])
            out[name] = {"us_per_step": d["value"], "workload": d["config"]["workload"], "kernel_us": d.get("kernel_us"),
                         "pct_hbm_peak": d.get("pct_hbm_peak"), "bytes_vs_dense": d.get("bytes_vs_dense"),
                         "k_pass_roofline_frac": d["roofline"]["frac"], "steps": d["steps"],
                         "dense_baseline_us": d.get("dense_fp16_hip_us", d.get("dense_in_planes_us")),
                         "us_per_step_via_auto_compute": d.get("us_per_step_via_auto_compute"),
                         "host_us_per_auto_compute_call": d.get("host_us_per_auto_compute_call"),
                         "command": "python bench.py --no-cpu " + " ".join(extra)}
        except Exception as e:      # noqa: BLE001 (reported in the line)
            out[name] = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
    out["c5"] = workload_c5()
    return out


def workload_c5():
    """Config 5 end to end: the random-init Llama-2-7B-shaped decoder (32 layers, d = 4096, 32 heads, fp16 weights), batch 8,
    a 128-token prompt and 256 greedy decode steps, once with dense torch attention and once with the AlignedKV cache in
    every layer through QuantizedCache_AlignedKV.auto_compute (reference loop: model/KVCache_AlignedKV.py:92-135), teacher
    forced with the first run's tokens.  Whole-model wall clock: the GEMMs are torch's."""
    import re
    import subprocess
    cmd = [sys.executable, "-m", "alignedkv_amd.model.decoder_harness", "--kinds", "dense_torch,alignedkv,alignedkv_graph",
           "--k-block", "256"]
    try:
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=400, cwd=ROOT)
        out = {"workload": "C5: 32-layer Llama-2-7B-shaped decoder, batch 8, 128-token prompt + 256 greedy steps",
               "command": "python -m alignedkv_amd.model.decoder_harness --kinds dense_torch,alignedkv,alignedkv_graph --k-block 256",
               "kinds": "dense_torch: dense torch attention; alignedkv: QuantizedCache_AlignedKV.auto_compute, launched eagerly; "
                        "alignedkv_graph: the step with lengths on the device, the whole decoder step replayed from a HIP graph"}
        for line in r.stdout.splitlines():
            m = re.match(r"(\w+)\s+([\d.]+) s\s+([\d.]+) tok/s(.*)", line.strip())
            if m:
                out[m.group(1)] = {"seconds": float(m.group(2)), "tokens_per_s": float(m.group(3))}
                alone = re.search(r"alone ([\d.]+) ms/step = ([\d.]+) tok/s", m.group(4))
                if alone:
                    out[m.group(1)].update(decode_ms_per_step=float(alone.group(1)), decode_tokens_per_s=float(alone.group(2)))
                extra = re.search(r"agreement.*?([\d.]+) %\s+max \|dlogit\| ([\d.]+)", m.group(4))
                if extra:
                    out[m.group(1)].update(greedy_agreement_pct=float(extra.group(1)), max_abs_dlogit=float(extra.group(2)))
        if "alignedkv" not in out:
            out["error"] = (r.stderr or r.stdout)[-300:]
        return out
    except Exception as e:      # noqa: BLE001 (reported in the line)
        return {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if a.workload == "c3":
        return bench_c3(a)
    import numpy as np
    import torch
    import alignedkv_amd
    from alignedkv_amd.model.KVCache_AlignedKV import QuantizedCache_AlignedKV
    from types import SimpleNamespace

    lib = alignedkv_amd.load_library()
    B, H, D, L = a.batch, a.heads, a.head_dim, a.cache_len
    if D > 128:
        a.k_block = 64      # the 256-token layout is built for head_dim 64 and 128
    assert L % 64 == 0, "the cache length of the benchmark must be a multiple of the 64-token flush block"
    cfg = SimpleNamespace(num_hidden_layers=a.layers, num_attention_heads=H, num_key_value_heads=H, hidden_size=H * D,
                          max_position_embeddings=L + 64 + a.extra_capacity)
    cache = QuantizedCache_AlignedKV(cfg, B, L + 64 + a.extra_capacity, "cuda", torch.half, k_block=a.k_block)
    for layer in range(a.layers):
        k, v = make_layer_inputs(torch, B, L, H, D, a.seed + layer, a.k_kind)
        cache.key_cache[layer].save(k, 0, L)
        cache.value_cache[layer].save(v, 0, L)
        del k, v
    g = torch.Generator(device="cuda").manual_seed(a.seed + 999)
    q = (a.q_scale * torch.randn((B, 1, H, D), device="cuda", generator=g)).half()
    k_new = torch.randn((B, 1, H, D), device="cuda", generator=g).half()
    v_new = (0.5 * torch.randn((B, 1, H, D), device="cuda", generator=g)).half()
    out = torch.empty_like(q)
    torch.cuda.synchronize()

    copy_gbps = None
    if a.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        st = torch.cuda.current_stream().cuda_stream
        for _ in range(3):
            lib.akv_copy_probe(dst.data_ptr(), src.data_ptr(), src.numel(), st)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            lib.akv_copy_probe(dst.data_ptr(), src.data_ptr(), src.numel(), st)
        torch.cuda.synchronize()
        copy_gbps = 2 * src.numel() * 20 / (time.perf_counter() - t0) / 1e9
        del src, dst

    runners = [StepRunner(torch, lib, cache, i, q, k_new, v_new, out, False, i == 0) for i in range(a.layers)]
    sec = time_steps(torch, runners, a.steps, a.warmup)
    us = sec * 1e6
    # The same loop long enough for its fixed costs not to matter (the first launch after the idle device, the host
    # noticing the end: about 25 us per timed region, and a few milliseconds of slower steps that follow 2-3 ms after an
    # idle period): what a decode loop that keeps the device busy sees per step.
    steady_steps = max(a.steps, 2000 if B * L <= 8 * 8192 else 400)
    if a.profile_run:
        steady_steps = a.steps
    sec_steady = time_steps(torch, runners, steady_steps, max(a.warmup, steady_steps // 6))
    pct = step_percentiles(torch, runners, a.steps)
    runners[0]()
    torch.cuda.synchronize()
    out_aligned = out.clone()            # layer 0's output
    k_levels = runners[0].k_levels.cpu().numpy()
    v_levels = runners[0].v_levels.cpu().numpy()

    # bytes the algorithm has to move for this input (from the fetch decisions the kernels took)
    R = L
    by = algorithmic_bytes(k_levels, v_levels, B, H, D, R, L + 1)
    eff_gbps = by["total"] / sec / 1e9

    # per-kernel durations (HIP events on the stream) -> roofline of the step's kernels
    ph_raw, event_pair_us = phase_times(torch, lib, runners, min(a.steps, 200))
    ph = [max(x - event_pair_us, 0.0) for x in ph_raw]
    k_pass_bytes = by["k_plane"] + B * H * D * (2 + 1 + 2) + B * H * R * 2     # planes + q, column max, new key + scores
    v_pass_bytes = by["v_plane"] + B * H * R * 2 + B * H * D * 2 + B * H * (R // 256) * D * 4
    # everything after the K pass: scores and probabilities, probe rows, V planes, the token's fp16 rows, the output
    tail_bytes = by["total"] - k_pass_bytes
    # With one row of (batch, head) pairs per compute unit the library runs everything after the K pass as one
    # launch: the second interval then covers it and the last two are empty
    one_launch_tail = ph[2] < 0.5 and ph[3] < 0.5
    if one_launch_tail:
        kernel_us = {"k_pass": round(ph[0], 2), "middle_v_pass_sum": round(ph[1], 2)}
        v_pass_gbps = None
    else:
        kernel_us = {"k_pass": round(ph[0], 2), "middle": round(ph[1], 2), "v_pass": round(ph[2], 2), "combine": round(ph[3], 2)}
        v_pass_gbps = round(v_pass_bytes / (ph[2] * 1e-6) / 1e9, 1)

    # dense-in-planes baseline: same kernels, every plane read (the reference's `reference=True` mode)
    ref_runners = [StepRunner(torch, lib, cache, i, q, k_new, v_new, out, True, False) for i in range(a.layers)]
    sec_ref = time_steps(torch, ref_runners, max(a.steps // 2, 20), 10)

    # the same step with the other K plane block length (same inputs)
    other = None
    if D <= 128:      # (head_dim 256 has the 64-token layout only)
        other_kb = 64 if a.k_block == 256 else 256
        cache2 = QuantizedCache_AlignedKV(cfg, B, L + 64 + a.extra_capacity, "cuda", torch.half, k_block=other_kb)
        for layer in range(a.layers):
            k, v = make_layer_inputs(torch, B, L, H, D, a.seed + layer, a.k_kind)
            cache2.key_cache[layer].save(k, 0, L)
            cache2.value_cache[layer].save(v, 0, L)
            del k, v
        out2 = torch.empty_like(q)
        runners2 = [StepRunner(torch, lib, cache2, i, q, k_new, v_new, out2, False, False) for i in range(a.layers)]
        sec_other = time_steps(torch, runners2, max(a.steps // 2, 20), 10)
        runners2[0]()
        torch.cuda.synchronize()
        # summation order differs, levels do not (both: layer 0)
        other = {"k_block": other_kb, "us_per_step": round(sec_other * 1e6, 2),
                 "max_abs_diff_of_outputs": float((out2.float() - out_aligned.float()).abs().max())}
        del cache2, runners2

    # figures of the tracked rocprofv3 summaries for this exact workload (none for other shapes)
    default_workload = (B, H, D, L, a.k_kind) == (8, 32, 128, 4096, "outlier")
    prof = profile_figures("decode_step_c2" + ("" if a.k_block == 256 else "_k_block64")) if default_workload else {}
    if a.k_block == 64:
        k_kernel = "akv::fused_k_pass_kernel<%d, false, true, true>" % D if D <= 128 else "akv::fused_k_pass_kernel<%d, false, false, false>" % D
    else:
        k_kernel = "akv::fused_k_pass256_split_kernel<%d, false, 4, true>" % D
    tail_kernel = "akv::tail_step_kernel<%d, 512, 2, false>" % D
    res = {
        "metric": "decode-attn us/step (+ effective HBM GB/s, %% of peak), B=%d L=%d %dx%d" % (B, L, H, D),
        "value": round(us, 2), "unit": "us/step", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(us / 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: batch %d, %d heads x %d, cache %d + 1 appended token, K %s, %d layers rotated, K plane blocks of %d tokens"
                               % ({(8, 32, 128, 4096): "C2", (1, 32, 128, 1024): "C1", (4, 32, 128, 32768): "C4"}.get((B, H, D, L), "other shape")
                                  if a.q_scale == 1.0 else "other queries (q x %g)" % a.q_scale,
                                  B, H, D, L, a.k_kind, a.layers, a.k_block)},
        "us_per_step_percentiles": pct,
        "steady_state": {"us_per_step": round(sec_steady * 1e6, 2), "steps": steady_steps,
                         "effective_hbm_gbps": round(by["total"] / sec_steady / 1e9, 1),
                         "frac_of_hbm_peak": round(by["total"] / sec_steady / 1e9 / HBM_PEAK_GBPS, 4),
                         "note": "same loop and clock as `value`, over more steps after a longer warm-up"},
        "effective_hbm_gbps": round(eff_gbps, 1), "pct_hbm_peak": round(100 * eff_gbps / HBM_PEAK_GBPS, 1),
        "algorithmic_bytes": int(by["total"]), "dense_fp16_bytes": int(by["dense"]),
        "bytes_vs_dense": round(by["total"] / by["dense"], 4),
        "level_fractions": {"k_mid": round(by["f_mid_k"], 4), "k_last": round(by["f_last_k"], 4),
                            "v_mid": round(by["f_mid_v"], 4), "v_last": round(by["f_last_v"], 4)},
        "kernel_us": kernel_us,
        "v_pass_gbps": v_pass_gbps,
        "k_block": a.k_block, "other_k_block_us": other,
        "dense_in_planes_us": round(sec_ref * 1e6, 2),
        "speedup_vs_dense_in_planes": round(sec_ref / sec, 3),
        # the dominant kernel (the K pass), the step's other kernel, and the step as a whole
        "roofline": roofline_entry(k_kernel, k_pass_bytes, ph_raw[0], event_pair_us, prof.get(k_kernel, {})),
        "roofline_step": {"bound": "hbm", "achieved": round(eff_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                          "frac": round(eff_gbps / HBM_PEAK_GBPS, 4), "algorithmic_bytes_per_step": int(by["total"]),
                          "us_per_step": round(us, 2), "duration_source": "wall clock around the timed steps"},
    }
    if one_launch_tail:
        res["roofline_tail"] = roofline_entry(tail_kernel, tail_bytes, ph_raw[1], event_pair_us, prof.get(tail_kernel, {}))
    if copy_gbps is not None:
        res["copy_probe_gbps_read_plus_write"] = round(copy_gbps, 1)
    try:
        from alignedkv_amd import dense_baseline
        res.update(dense_baseline.bench(torch, lib, B, H, D, L + 1, a.layers, max(a.steps // 2, 20), sec))
    except ImportError:
        pass
    if not a.no_cpu:
        cpu_sec, cpu_out, cklv, cvlv, threads = cpu_baseline(torch, cache, q, k_new, v_new, a.cpu_steps)
        runners[0]()
        torch.cuda.synchronize()
        err = float(np.max(np.abs(out.cpu().numpy().astype(np.float32) - cpu_out.astype(np.float32))))
        res["cpu_baseline"] = {"value": round(cpu_sec * 1e6, 1), "unit": "us/step", "cores": threads, "kind": "port",
                               "cpu_model": cpu_model(), "host_cores": os.cpu_count(),
                               "sample": "%d full-size steps of layer 0 (min), C restatement with OpenMP + NumPy host logic"
                                         % a.cpu_steps}
        dsec, dthreads = cpu_dense_torch(torch, B, H, D, L + 1)
        res["cpu_dense_torch"] = {"value": round(dsec * 1e6, 1), "unit": "us/step", "cores": dthreads,
                                  "sample": "median of 10 dense fp16 attention steps (fp32 softmax) with torch on the host"}
        res["parity"] = {"max_abs_err_vs_oracle": err, "k_levels_equal": bool(np.array_equal(cklv, k_levels)),
                         "v_level_mismatches": int((cvlv != v_levels).sum()), "v_levels_total": int(v_levels.size)}
    # 64 consecutive decode steps per layer (the cache grows from L to L + 64: the rest buffer fills up and is
    # flushed once), averaged: what a generation loop sees, against `value` which repeats the first of them
    if L % 64 == 0:
        grow = [StepRunner(torch, lib, cache, i, q, k_new, v_new, out, False, False) for i in range(a.layers)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for sidx in range(64):
            for r in grow:
                r.at_length(L + sidx)()
        torch.cuda.synchronize()
        res["avg_us_over_64_growing_steps"] = round((time.perf_counter() - t0) / (64 * a.layers) * 1e6, 2)
    # the same steps through the reference's host API (QuantizedCache_AlignedKV.auto_compute), beside the raw C-ABI figure
    res["probabilities_recorded"] = True       # (the C ABI's default; the figure without the record follows)
    if not a.profile_run:
        lean = [StepRunner(torch, lib, cache, i, q, k_new, v_new, out, False, False, record_probs=False) for i in range(a.layers)]
        sec_lean = time_steps(torch, lean, steady_steps, max(a.warmup, steady_steps // 6))
        res["steady_state_without_probability_record"] = {
            "us_per_step": round(sec_lean * 1e6, 2), "frac_of_hbm_peak": round(by["total"] / sec_lean / 1e9 / HBM_PEAK_GBPS, 4),
            "note": "AKV_STEP_NO_PROBS_RECORD: a caller that never reads `probs`; same loop as steady_state"}
        api_us, api_host_us = time_api_path(torch, cache, q, k_new, v_new, L, max(a.steps, 400))
        res["us_per_step_via_auto_compute"] = round(api_us, 2)
        res["host_us_per_auto_compute_call"] = round(api_host_us, 2)
    if not a.no_extras and not a.no_cpu and (B, H, D, L) == (8, 32, 128, 4096):
        res["other_workloads"] = other_workloads(a)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
