#!/usr/bin/env python3
"""Benchmark of the fused AdamW + clip + bf16-twin optimizer step on one MI355X.

A "step" is one pass of the optimizer over the whole parameter set of the named workload:
the global sum of squares of the gradients (clip norm) and the fused update.  Inputs are
synthetic and already resident in HBM when the timed region starts: parameters ~N(0, 0.02),
zero moments, and one fresh gradient flat ~N(0, 1e-3) per step (steps+warmup gradient slots of the arena,
generated on the device), scaled so that about half the steps clip.  The learning rate follows
a 100-step warmup + cosine schedule.

Prints ONE JSON line.  `value` is whole-step algorithmic HBM throughput (bytes the step must
move per parameter x parameters / step time); `roofline` is the update kernel alone, timed
with HIP events on the library's compute stream; `cpu_baseline` is the same step on the host
cores of this box (multithreaded restatement of the reference's loop) on a bounded sample.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# name: (size, grad_type, moment_type, bytes/param of the norm pass, bytes/param of the update)
WORKLOADS = {
    "185m": ("185m", 0, 0, 4, 34),          # benchmark configuration 2
    "555m": ("555m", 0, 0, 4, 34),          # benchmark configuration 3 (headline)
    "555m-bf16": ("555m", 1, 1, 2, 22),     # benchmark configuration 4
    "1p4b-fp8": ("1p4b", 2, 0, 1, 28),      # benchmark configuration 5
    "1p4b": ("1p4b", 0, 0, 4, 34),          # the 1.4B set in the all-f32 mode (comparison only)
}
ELEM = {0: 4, 1: 2, 2: 1}
# HBM bytes per launch of the update kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled
# by what the counter reads for a plain copy kernel of known size: profiles/traffic.json, written
# together with the summaries under profiles/ (per workload: scaled bytes read and written, the
# scale factors, and a digest of the kernel sources the profiled library was built from).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
KERNEL_SOURCES = ["adam_kernels.hip", "adam_kernels.h", "adam_math.h"]


def kernel_sources_digest():
    import hashlib
    h = hashlib.sha1()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "anni_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic(workload):
    """(bytes per launch, digest of the profiled kernel sources, do today's sources match)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)[workload]
    except (OSError, KeyError, ValueError):
        return None, None, None
    return (int(t["fetch_bytes"] + t["write_bytes"]), t.get("kernel_sources_sha1"),
            t.get("kernel_sources_sha1") == kernel_sources_digest())


STORAGE = {"185m": "f32 p/g/m/v + bf16 twin", "555m": "f32 p/g/m/v + bf16 twin",
           "555m-bf16": "f32 p, bf16 g/m/v + bf16 twin",
           "1p4b-fp8": "f32 p/m/v, fp8-e4m3 g with per-tensor scale + bf16 twin",
           "1p4b": "f32 p/g/m/v + bf16 twin"}


QUANT_MS = []        # wall time of every anni_adam_quantize_grads call of fill_grad_slots (fp8 workloads)


def fill_grad_slots(L, opt, tensors, count, grad_type, seed, first_step=0):
    """Fills the arena's first `count` gradient slots for the steps first_step .. first_step + count - 1,
    each ~N(0, 1e-3) in the workload's storage type (a fresh random stream per step).
    Returns the slot pointers and, for fp8, one per-tensor scale array per slot."""
    from anni_amd.lm_adam import DeviceBuffer
    n = opt.n
    ptrs, scales = [], []
    stage = DeviceBuffer(n * 4) if grad_type != 0 else None
    for k in range(count):
        slot = opt.grad_slot(k)
        assert slot
        dst = slot if grad_type == 0 else stage.ptr
        assert L.anni_fill_normal_f32(dst, n, seed, 1000 + first_step + k, 0.0, 1e-3) == 0
        sc = None
        if grad_type == 1:
            assert L.anni_f32_to_bf16(slot, stage.ptr, n) == 0
        elif grad_type == 2:
            # the multi-tensor quantiser writes the bound flat and the bound scale array
            sc = DeviceBuffer(len(tensors) * 4)
            opt.bind_grad(slot)
            opt.o.d_gscale = sc.ptr
            assert L.gpu_stream_sync() == 0
            t0 = time.perf_counter()
            assert L.anni_adam_quantize_grads(opt.h, stage.ptr) == 0
            assert L.gpu_stream_sync() == 0
            QUANT_MS.append((time.perf_counter() - t0) * 1e3)
        assert L.gpu_stream_sync() == 0
        ptrs.append(slot)
        scales.append(sc)
    if stage is not None:
        stage.free()
    return ptrs, scales


def short_leg(L, workload, layout, steps=6, warmup=2, slots=4):
    """A second arena in the same process (after the first was freed): `steps` timed steps of
    `workload` on an arena of the given layout, HIP events per kernel, any storage mode."""
    from anni_amd import layout as lay
    from anni_amd import lm_adam
    from anni_amd.lm_adam import LmAdam
    size, gt, mt, norm_bpp, upd_bpp = WORKLOADS[workload]
    tensors = lay.tensors(size, "baseline")
    t_create = time.perf_counter()
    opt = LmAdam(tensors, grad_type=gt, moment_type=mt, twins=True, skip_nonfinite=True, grad_slots=slots,
                 layout={"auto": 0, "compact": 1, "split": 2}[layout],
                 beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    t_create = (time.perf_counter() - t_create) * 1e3
    n = opt.n
    own_gscale = opt.o.d_gscale
    assert L.anni_fill_normal_f32(opt.o.d_param, n, 20260101, 1, 0.0, 0.02) == 0
    opt.seed_twins()
    unit = 1.0 / (math.sqrt(n) * 1e-3)
    tot = [0.0, 0.0, 0.0]
    wall = 0.0
    done = 0
    old_scales = []
    while done < warmup + steps:
        count = min(slots, warmup + steps - done)
        ring, scales = fill_grad_slots(L, opt, tensors, count, gt, 20260101, done)
        for sc in old_scales:
            if sc is not None:
                sc.free()
        old_scales = scales
        lr = [lm_adam.step_lr(3e-4, done + i, 100, 1000, "cosine") for i in range(count)]
        gs = [unit * (1.7 if (done + i) % 2 else 0.6) for i in range(count)]
        timed = [i for i in range(count) if done + i >= warmup]

        def run(first, k, per_kernel):
            """Steps first .. first + k - 1 of this batch; fp8: one call per step, each flat has scales of its own."""
            ms, sa, sb = C.c_float(0), C.c_float(0), C.c_float(0)
            groups = [(first + i, 1) for i in range(k)] if gt == 2 else [(first, k)]
            out = [0.0, 0.0, 0.0]
            for g0, gk in groups:
                if gt == 2:
                    opt.o.d_gscale = scales[g0].ptr
                rc = L.anni_adam_time_steps(opt.h, gk, (C.c_void_p * gk)(*ring[g0:g0 + gk]), gk,
                                            (C.c_double * gk)(*lr[g0:g0 + gk]),
                                            (C.c_double * gk)(*gs[g0:g0 + gk]), C.byref(ms),
                                            C.byref(sa) if per_kernel else None,
                                            C.byref(sb) if per_kernel else None)
                assert rc == 0, L.gpu_debug_last_error()
                out = [out[0] + ms.value, out[1] + sa.value, out[2] + sb.value]
            return out
        if len(timed) < count:                           # the warm-up part of this batch
            run(0, count - len(timed), False)
        if timed:
            L.gpu_device_sync()
            t0 = time.perf_counter()
            got = run(timed[0], len(timed), True)
            L.gpu_device_sync()
            wall += (time.perf_counter() - t0) * 1e3
            tot = [tot[0] + got[0], tot[1] + got[1], tot[2] + got[2]]
        done += count
    st = opt.sync_stats()
    assert opt.t == warmup + steps and math.isfinite(st.last_grad_norm)
    # fp8: a step per call, so the wall clock carries a launch and a wait per step; the events do not
    ms_step = (tot[0] if gt == 2 else wall) / steps
    upd_ms = tot[2] / steps
    walked, place_ms, _timed = opt.placement_cost
    _traffic, _digest, current = profiled_traffic(workload)
    out = {"workload": workload, "storage": STORAGE[workload], "params": n, "steps": steps, "warmup": warmup,
           "layout": "split" if opt.split else "compact",
           "placement_apart_ratio": round(opt.apart_ratio, 3),
           "placement_walked_GiB": round(walked, 1), "placement_ms": round(place_ms, 1),
           "arena_create_ms": round(t_create, 1),
           "arena_bytes": opt.arena_bytes, "resident_bytes": opt.resident_bytes,
           "ms_per_step": round(ms_step, 4),
           "ms_per_step_timed_by": "events around each step" if gt == 2 else "wall clock around the run",
           "GBps": round(n * (norm_bpp + upd_bpp) / ms_step / 1e6, 1),
           "frac": round(n * (norm_bpp + upd_bpp) / ms_step / 1e6 / HBM_PEAK_GBPS, 4),
           "update_ms": round(upd_ms, 4), "sumsq_ms": round(tot[1] / steps, 4),
           "update_frac": round(n * upd_bpp / upd_ms / 1e6 / HBM_PEAK_GBPS, 4),
           "profile_matches_these_sources": current}
    opt.o.d_gscale = own_gscale
    for sc in old_scales:
        if sc is not None:
            sc.free()
    opt.free()
    return out


def placement_cost_leg(L):
    """What the search for the arena's second block costs, and what it leaves behind for the next
    allocation: creation of a 555M arena (GiB requested and held during the walk, milliseconds),
    then hipMalloc + first touch of 64 GiB; first on the device as this process found it, then again
    after 150 GiB were allocated, touched and freed.  Run with ANNI_PLACE_LOG=1 to see every candidate."""
    from anni_amd import layout as lay
    from anni_amd.lm_adam import LmAdam
    hip = C.CDLL("libamdhip64.so")
    hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    hip.hipFree.argtypes = [C.c_void_p]
    tensors = lay.tensors("555m", "baseline")

    def malloc_and_touch(gib):
        p = C.c_void_p()
        L.gpu_device_sync()
        t0 = time.perf_counter()
        assert hip.hipMalloc(C.byref(p), gib << 30) == 0
        t1 = time.perf_counter()
        assert L.gpu_memset(p.value, 0, gib << 30) == 0
        L.gpu_device_sync()
        t2 = time.perf_counter()
        assert hip.hipFree(p) == 0
        L.gpu_device_sync()
        return {"GiB": gib, "hipMalloc_ms": round((t1 - t0) * 1e3, 1), "first_fill_ms": round((t2 - t1) * 1e3, 1),
                "hipFree_ms": round((time.perf_counter() - t2) * 1e3, 1)}

    def create():
        fr, tt = C.c_size_t(0), C.c_size_t(0)
        L.gpu_mem_info(C.byref(fr), C.byref(tt))
        t0 = time.perf_counter()
        opt = LmAdam(tensors, twins=True, skip_nonfinite=True, grad_slots=13, beta2=0.95,
                     weight_decay=0.1, grad_clip=1.0)
        ms = (time.perf_counter() - t0) * 1e3
        walked, place_ms, timed = opt.placement_cost
        out = {"free_GiB_before": round(fr.value / (1 << 30), 1), "create_ms": round(ms, 1),
               "search_ms": round(place_ms, 1), "walked_GiB": round(walked, 1), "candidates_timed": timed,
               "apart_ratio": round(opt.apart_ratio, 3), "probe_GBps": round(opt.probe_gbps, 1),
               "arena_GiB": round(opt.arena_bytes / (1 << 30), 2)}
        opt.free()
        return out
    out = {"untouched_device": {"arena_create": create(), "then_64GiB": malloc_and_touch(64),
                                "64GiB_again": malloc_and_touch(64)}}
    blocks = []
    for _ in range(150 // 15):
        p = C.c_void_p()
        assert hip.hipMalloc(C.byref(p), 15 << 30) == 0
        assert L.gpu_memset(p.value, 1, 15 << 30) == 0
        blocks.append(p)
    L.gpu_device_sync()
    for p in blocks:
        assert hip.hipFree(p) == 0
    out["after_150GiB_allocated_touched_freed"] = {"arena_create": create(), "then_64GiB": malloc_and_touch(64)}
    return out


def cpu_baselines(size_name, norm_bpp, upd_bpp, budget_s, full=False):
    """The step on the host cores of this box: (multithreaded port, single-thread reference).
    full: the multithreaded leg runs on the workload's whole parameter count instead of a
    48 Mi sample (about 10 GB of host memory and half a minute more at 555M)."""
    from anni_amd import layout
    from oracle import binding as ob
    ob.lib()
    threads = min(ob.lib().oracle_max_threads(), len(os.sched_getaffinity(0)))
    n_full = layout.param_count(size_name)
    bpp = norm_bpp + upd_bpp
    rng = np.random.default_rng(0)

    def sample(n):
        p = (rng.standard_normal(n, dtype=np.float32) * np.float32(0.02))
        g0 = (rng.standard_normal(n, dtype=np.float32) * np.float32(1e-3))
        return p, g0

    # multithreaded restatement, SoA, all cores; norm by ordered partials
    n = n_full if full else min(n_full, 48 << 20)
    p, g0 = sample(n)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    simd = ob.cpu_simd()
    O = ob.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, threads=threads,
                  norm_threads=threads, simd=simd)
    g = g0.copy()
    O.step(p, g, m, v, 3e-6, 1.0 / (math.sqrt(n) * 1e-3) * 1.7)      # warm the pages
    times = []
    t_end = time.perf_counter() + budget_s * 0.5
    k = 0
    while k < 3 or (time.perf_counter() < t_end and k < 12):
        g[:] = g0
        gs = 1.0 / (math.sqrt(n) * 1e-3) * (1.7 if k % 2 else 0.6)
        t0 = time.perf_counter()
        O.step(p, g, m, v, 3e-6 * (k + 2), gs)
        times.append(time.perf_counter() - t0)
        k += 1
    mt = float(np.median(times))
    mt_out = {
        "value": round(n * bpp / mt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "simd": simd,
        "sample": ("all" if n == n_full else "first") + " %d of %d params of the workload, %d timed steps (median), fp32 state, "
                  "clip 1.0 + decay 0.1, OpenMP over %d threads, %s build (gcc -O3 auto-vectorised, "
                  "no FMA contraction: bit-identical to the serial loop)"
                  % (n, n_full, len(times), threads, simd),
        "params_per_s": round(n / mt, 1), "ms_per_step_sample": round(mt * 1e3, 3),
        "ms_per_step_extrapolated": round(mt * 1e3 * n_full / n, 1),
    }
    del p, g, g0, m, v

    # the reference's own serial loop (compiled reference if it travelled, else the slot-layout port)
    n = min(n_full, 12 << 20)
    p, g0 = sample(n)
    g = g0.copy()
    if ob.ref_available():
        R = ob.RefAdam(p, g, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
        kind = "reference"

        def one(k):
            R.step(3e-6 * (k + 1), 1.0 / (math.sqrt(n) * 1e-3) * (1.7 if k % 2 else 0.6))
    else:
        kind = "port"
        slots = np.zeros(n, dtype=[("param", np.uint64), ("grad", np.uint64), ("m", np.float32),
                                   ("v", np.float32)])
        slots["param"] = p.ctypes.data + 4 * np.arange(n, dtype=np.uint64)
        slots["grad"] = g.ctypes.data + 4 * np.arange(n, dtype=np.uint64)

        def one(k):
            ob.lib().oracle_adam_step_slots(
                slots.ctypes.data, n, k + 1, 0.9, 0.95, 1e-8, 0.1, 1.0, 3e-6 * (k + 1),
                1.0 / (math.sqrt(n) * 1e-3) * (1.7 if k % 2 else 0.6))
    one(0)
    times = []
    for k in range(1, 4):
        g[:] = g0
        t0 = time.perf_counter()
        one(k)
        times.append(time.perf_counter() - t0)
    st = float(np.median(times))
    serial_out = {
        "value": round(n * bpp / st / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind,
        "sample": "first %d of %d params, 3 timed steps (median), the reference's serial "
                  "24-byte-slot loop" % (n, n_full),
        "params_per_s": round(n / st, 1), "ns_per_param": round(st / n * 1e9, 3),
        "ms_per_step_extrapolated": round(st * 1e3 * n_full / n, 1),
    }
    return mt_out, serial_out


def reference_caller_leg(L, size="185m", call_trace=False):
    """The reference's own lm + lm_adam_create + lm_adam_step_scaled (compiled from the reference
    tree, linked against this backend) timed wall-clock per step: at its compile-time size
    (oracle/_ref/libanni_ref_hip.so: untied 16384-token embedding) or, size "555m", at the sizes of
    its 555M run with the tied 100000-token embedding (oracle/_ref/libanni_ref_555m_hip.so).
    call_trace: the flavours with the call-timing interposer in front of the backend
    (oracle/gputrace.c); the last step's calls are reported as a host-side timeline.
    None when that library did not travel."""
    from oracle import binding as ob
    have = ob.ref_trace_available() if call_trace else \
        (ob.ref_hip_available() if size == "185m" else ob.ref_hip_555m_available())
    if not have:
        return None
    suffix = "_trace" if call_trace else ""
    if size == "185m":
        make = lambda: ob.RefModelOnBackend(16384, beta2=0.95, weight_decay=0.1, grad_clip=1.0,
                                            backend="hip" + suffix)
    else:
        make = lambda: ob.RefModelOnBackend(100000, beta2=0.95, weight_decay=0.1, grad_clip=1.0,
                                            backend="hip555m" + suffix, tied=True)
    L.gpu_set_compute_prec(1)
    used0, dropped0 = C.c_long(0), C.c_long(0)
    L.anni_early_sum_stats(C.byref(used0), C.byref(dropped0))
    vsteps0, vserved0 = C.c_long(0), C.c_long(0)
    L.anni_vectors_first_stats(C.byref(vsteps0), C.byref(vserved0))
    M = make()
    n = M.n
    vec_bytes = 4 * sum(cnt for _off, cnt, is_mat in M.segs() if not is_mat)
    rng = np.random.default_rng(1)
    # 16 Mi normal deviates, repeated: what the step costs does not depend on the values, and
    # drawing 5.6e8 of them would take longer than all the timed steps together
    block = rng.standard_normal(1 << 24, dtype=np.float32) * np.float32(1e-3)
    g = np.tile(block, -(-n // block.size))[:n]
    unit = 1.0 / (math.sqrt(n) * 1e-3)
    times = []
    last = 12
    for t in range(1, last + 1):
        M.set_grads(g)
        L.gpu_device_sync()
        if call_trace and t == last:
            ob.gputrace().gputrace_start()
        t0 = time.perf_counter()
        M.step(3e-6 * t, unit * (1.7 if t % 2 else 0.6))
        times.append((time.perf_counter() - t0) * 1e3)
        if call_trace:
            ob.gputrace().gputrace_stop()
    n_segs = M.n_segs
    events = ob.gputrace_events() if call_trace else None
    used, dropped = C.c_long(0), C.c_long(0)
    L.anni_early_sum_stats(C.byref(used), C.byref(dropped))
    vsteps, vserved = C.c_long(0), C.c_long(0)
    L.anni_vectors_first_stats(C.byref(vsteps), C.byref(vserved))
    M.close()
    L.gpu_set_compute_prec(0)
    L.gpu_adam_set_weight_decay(0.0)
    ms = float(np.median(times[1:]))
    out = {"what": "unchanged lang/lm_adam.c (lm_adam_step_scaled, device path) on this backend: "
                   "matrices aliased into the flats, bias/LayerNorm vectors host-resident (uploaded "
                   "before and read back after every step by the caller), norm read back by the caller",
           "params": n, "segments": n_segs, "host_vector_bytes": vec_bytes,
           "ms_per_step": round(ms, 3), "min_ms": round(min(times[1:]), 3),
           "first_step_ms_with_arena_init": round(times[0], 1),
           "ms_of_steps_2_to_4_while_the_callers_pattern_is_learned": [round(x, 3) for x in times[1:4]],
           "GBps_algorithmic": round(n * 38 / ms / 1e6, 1),
           "frac": round(n * 38 / ms / 1e6 / HBM_PEAK_GBPS, 4),
           "steps": last,
           "sums_begun_at_the_first_upload_and_used": used.value - used0.value,
           "sums_begun_early_and_dropped": dropped.value - dropped0.value,
           "steps_with_the_vectors_updated_and_read_back_first": vsteps.value - vsteps0.value,
           "read_backs_served_that_way": vserved.value - vserved0.value,
           "a_stream_that_runs_beside_the_compute_stream_was_found":
               {-1: "not looked for", 0: "no", 1: "yes"}[L.anni_second_stream_state()]}
    if events:
        out["call_trace_of_the_last_step"] = call_timeline(events, times[-1])
    return out


def call_timeline(ev, wall_ms):
    """Host-side timeline of one lm_adam_step_scaled from the interposer's records (microseconds)."""
    base = ev[0][1]
    per = {}
    for nm, a, b, by in ev:
        k = per.setdefault(nm, [0, 0.0, 0])
        k[0] += 1
        k[1] += b - a
        k[2] += by

    def first(nm):
        return next(i for i, e in enumerate(ev) if e[0] == nm)
    i_ss, i_st = first("gpu_grad_sumsq"), first("gpu_adam_step_dev_bf16")
    i_sy = max(i for i, e in enumerate(ev) if e[0] == "gpu_stream_sync")
    r = lambda x: round(x, 1)
    return {
        "wall_ms_with_interposer": round(wall_ms, 3), "calls": len(ev),
        "per_entry_point_us": {nm: {"calls": c, "total_us": r(us), "bytes": by}
                               for nm, (c, us, by) in sorted(per.items(), key=lambda kv: -kv[1][1]) if us >= 0.05},
        "callers_own_time_between_calls_us": r(sum(ev[i + 1][1] - ev[i][2] for i in range(len(ev) - 1))),
        "phases_us": {
            "gather: step start .. gpu_grad_sumsq called (the caller stages its vectors; on the device "
            "the copy pieces and, once the pattern is learned, the sum begun at the first upload)":
                r(ev[i_ss][1] - base),
            "gpu_grad_sumsq (last copy piece, rest of the sum, its last stage, result read from "
            "page-locked memory)": r(ev[i_ss][2] - ev[i_ss][1]),
            "norm on the host .. update launched (in two parts once the read-backs are learned)":
                r(ev[i_st][2] - ev[i_ss][2]),
            "the caller's read-back calls": r(ev[i_sy][1] - ev[i_st][2]),
            "gpu_stream_sync (the vectors handed over while the update runs, then the wait for it)":
                r(ev[i_sy][2] - ev[i_sy][1]),
            "after": r(ev[-1][2] - ev[i_sy][2])},
        "calls_over_10us": [{"entry": nm, "at_us": r(a - base), "us": r(b - a), "bytes": by}
                            for nm, a, b, by in ev if b - a > 10.0]}


def colsum_leg(L, rows, shapes=((6272, False), (1536, False), (1536, True))):
    """anni_colsum_add at the 555M model's shapes: db1 (rows x 6272), db2 / dbeta (rows x 1536),
    dgamma (rows x 1536, product of two matrices); 20 launches each, wall clock around them."""
    from anni_amd.lm_adam import DeviceBuffer
    out = []
    for cols, prod in shapes:
        n = rows * cols
        x, y, acc = DeviceBuffer(n * 4), DeviceBuffer(n * 4), DeviceBuffer(cols * 4)
        assert L.anni_fill_normal_f32(x.ptr, n, 5, 1, 0.0, 1e-2) == 0
        assert L.anni_fill_normal_f32(y.ptr, n, 5, 2, 0.0, 1.0) == 0
        assert L.gpu_memset(acc.ptr, 0, cols * 4) == 0
        for _ in range(3):
            assert L.anni_colsum_add(acc.ptr, x.ptr, y.ptr if prod else None, rows, cols) == 0
        L.gpu_device_sync()
        t0 = time.perf_counter()
        for _ in range(20):
            assert L.anni_colsum_add(acc.ptr, x.ptr, y.ptr if prod else None, rows, cols) == 0
        L.gpu_device_sync()
        ms = (time.perf_counter() - t0) * 1e3 / 20
        nbytes = n * 4 * (2 if prod else 1)
        out.append({"rows": rows, "cols": cols, "product": prod, "ms": round(ms, 4),
                    "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                    "ns_per_row": round(ms * 1e6 / rows, 2)})
        for b in (x, y, acc):
            b.free()
    # the six sums of one 555M block (b1, b2, two LayerNorms) as one batch
    from anni_amd import lib
    shapes = [(6272, False), (1536, False), (1536, False), (1536, True), (1536, False), (1536, True)]
    bufs, jobs = [], []
    for k, (cols, prod) in enumerate(shapes):
        n = rows * cols
        x, y, acc = DeviceBuffer(n * 4), DeviceBuffer(n * 4 if prod else 4), DeviceBuffer(cols * 4)
        assert L.anni_fill_normal_f32(x.ptr, n, 6, k, 0.0, 1e-2) == 0
        if prod:
            assert L.anni_fill_normal_f32(y.ptr, n, 7, k, 0.0, 1.0) == 0
        assert L.gpu_memset(acc.ptr, 0, cols * 4) == 0
        bufs += [x, y, acc]
        jobs.append(lib.Colsum(acc.ptr, x.ptr, y.ptr if prod else None, rows, cols))
    arr = (lib.Colsum * len(jobs))(*jobs)
    for _ in range(3):
        assert L.anni_colsum_add_batch(arr, len(jobs)) == 0
    L.gpu_device_sync()
    t0 = time.perf_counter()
    for _ in range(20):
        assert L.anni_colsum_add_batch(arr, len(jobs)) == 0
    L.gpu_device_sync()
    ms = (time.perf_counter() - t0) * 1e3 / 20
    nbytes = sum(rows * c * 4 * (2 if p else 1) for c, p in shapes)
    out.append({"batch": "b1 + b2 + 2 x (dbeta, dgamma) of one 555M block", "rows": rows,
                "ms": round(ms, 4), "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1)})
    for b in bufs:
        b.free()
    return out


def ckpt_leg(L, size="555m"):
    """The optimizer block of a checkpoint (has_adam, epoch, step, t, n + n interleaved (m, v)
    pairs) written from and read into the arena: to /dev/null (device side + host link alone)
    and through a file on tmpfs."""
    import tempfile
    from anni_amd import layout
    from anni_amd.lm_adam import LmAdam
    opt = LmAdam(layout.tensors(size), twins=False, grad_slots=1)
    n = opt.n
    assert L.anni_fill_normal_f32(opt.o.d_m, n, 8, 1, 0.0, 1e-3) == 0
    assert L.anni_fill_normal_f32(opt.o.d_v, n, 8, 2, 1e-6, 1e-7) == 0
    L.gpu_device_sync()
    nbytes = 20 + 8 * n
    out = {"workload": size, "slots": n, "block_bytes": nbytes}
    fd = os.open("/dev/null", os.O_WRONLY)
    opt.write_state(fd, 1, 2)                                       # warm the staging buffers
    t0 = time.perf_counter()
    opt.write_state(fd, 1, 2)
    dt = time.perf_counter() - t0
    os.close(fd)
    out["write_to_devnull"] = {"ms": round(dt * 1e3, 1), "GBps": round(nbytes / dt / 1e9, 2)}
    d = "/dev/shm" if os.path.isdir("/dev/shm") else None
    with tempfile.NamedTemporaryFile(dir=d) as f:
        t0 = time.perf_counter()
        opt.write_state(f.fileno(), 1, 2)
        dt = time.perf_counter() - t0
        out["write_to_tmpfs"] = {"ms": round(dt * 1e3, 1), "GBps": round(nbytes / dt / 1e9, 2)}
        os.lseek(f.fileno(), 0, os.SEEK_SET)
        t0 = time.perf_counter()
        opt.read_state(f.fileno())
        L.gpu_device_sync()
        dt = time.perf_counter() - t0
        out["read_from_tmpfs"] = {"ms": round(dt * 1e3, 1), "GBps": round(nbytes / dt / 1e9, 2)}
    opt.free()
    return out


def sections_leg(L, n=555848096, region_gib=16):
    """How device memory is organised, measured: free memory is taken as physical blocks of 16 GiB
    (HIP virtual memory management: each a naturally aligned block while memory is free, handed
    out from the highest address down), each mapped at its own address; the flat-ABI update
    (gpu_adam_step_dev_bf16, all-zero state, which it leaves zero) then runs with its five flats
    in chosen blocks.  Reports the update's GB/s for every window of five consecutive blocks, the
    runs of blocks ("sections") those windows reveal, and for a few placements."""
    hip = C.CDLL("libamdhip64.so")

    class Loc(C.Structure):
        _fields_ = [("type", C.c_int), ("id", C.c_int)]

    class Prop(C.Structure):                      # hipMemAllocationProp
        _fields_ = [("type", C.c_int), ("handle_type", C.c_int), ("location", Loc),
                    ("win32", C.c_void_p), ("compression", C.c_ubyte), ("rdma", C.c_ubyte),
                    ("usage", C.c_ushort)]

    class Access(C.Structure):                    # hipMemAccessDesc
        _fields_ = [("location", Loc), ("flags", C.c_int)]
    hip.hipMemCreate.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.POINTER(Prop), C.c_ulonglong]
    hip.hipMemAddressReserve.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.c_size_t, C.c_void_p,
                                         C.c_ulonglong]
    hip.hipMemMap.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_ulonglong]
    hip.hipMemSetAccess.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(Access), C.c_size_t]
    hip.hipMemUnmap.argtypes = [C.c_void_p, C.c_size_t]
    hip.hipMemRelease.argtypes = [C.c_void_p]
    hip.hipMemAddressFree.argtypes = [C.c_void_p, C.c_size_t]
    prop = Prop(1, 0, Loc(1, 0), None, 0, 0, 0)   # pinned device memory of device 0
    acc = Access(Loc(1, 0), 3)                    # read-write
    size = region_gib << 30
    fr, tt = C.c_size_t(0), C.c_size_t(0)
    blocks = []
    while L.gpu_mem_info(C.byref(fr), C.byref(tt)) == 0 and fr.value >= size + (3 << 30):
        h, va = C.c_void_p(), C.c_void_p()
        if hip.hipMemCreate(C.byref(h), size, C.byref(prop), 0) != 0:
            break
        assert hip.hipMemAddressReserve(C.byref(va), size, 0, None, 0) == 0
        assert hip.hipMemMap(va, size, 0, h, 0) == 0
        assert hip.hipMemSetAccess(va, size, C.byref(acc), 1) == 0
        assert L.gpu_memset(va.value, 0, 10 << 30) == 0       # what the flats below touch
        blocks.append((h, va.value))
    L.gpu_device_sync()
    K = len(blocks)
    L.gpu_set_compute_prec(1)
    L.gpu_adam_set_weight_decay(0.1)

    def run(places, reps=4):
        """places: (block, offset GiB) of p, m, v, twin, g -> GB/s of algorithmic traffic."""
        p, m, v, tw, g = [blocks[b][1] + int(off * (1 << 30)) for b, off in places]
        args = (p, tw, g, m, v, n, 1e-3, 0.9, 0.95, 1e-8, 3, 1.0)
        assert L.gpu_adam_step_dev_bf16(*args) == 0
        L.gpu_device_sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            L.gpu_adam_step_dev_bf16(*args)
        L.gpu_device_sync()
        return round(n * 34 * reps / (time.perf_counter() - t0) / 1e9, 1)
    out = {"blocks_of_GiB": region_gib, "blocks": K, "params": n,
           "free_GiB_before": round((fr.value + K * size) / (1 << 30), 1)}
    win = [run([(b + i, 0) for i in range(5)]) for b in range(K - 4)]
    out["window_of_five_consecutive_blocks_GBps"] = win
    # a window inside one section is slow; the first fast window b means a boundary behind block b+3
    cut = (max(win) + min(win)) / 2
    sec, cur, b = [0] * K, 0, 0
    bounds = []
    while b < K - 4:
        if win[b] > cut:
            bounds.append(b + 4)
            b += 4
        else:
            b += 1
    for i in range(K):
        sec[i] = sum(1 for x in bounds if i >= x)
    out["section_of_block"] = sec
    members = [[i for i in range(K) if sec[i] == s] for s in range(max(sec) + 1)]
    out["blocks_per_section"] = [len(m) for m in members]
    if len(members) >= 3 and min(len(m) for m in members[:3]) >= 5:
        A, B_, C_ = members[0], members[1], members[2]
        out["placements_GBps"] = {
            "all five flats in ONE block (3 GiB apart)": run([(A[0], 3 * i) for i in range(5)]),
            "five blocks of section A": run([(A[i], 0) for i in range(5)]),
            "five blocks of section B, not consecutive": run([(B_[i], 0) for i in (0, 1, 3, 4, 5)] if len(B_) > 5 else [(B_[i], 0) for i in range(5)]),
            "p m | v twin g (two sections, as the split arena)": run([(A[0], 0), (A[1], 0), (B_[0], 0), (B_[1], 0), (B_[2], 0)]),
            "p m | v twin g, each side inside ONE block": run([(A[0], 0), (A[0], 4), (B_[0], 0), (B_[0], 4), (B_[0], 7)]),
            "p m v twin | g": run([(A[0], 0), (A[1], 0), (A[2], 0), (A[3], 0), (B_[0], 0)]),
            "p | m v twin g": run([(A[0], 0), (B_[0], 0), (B_[1], 0), (B_[2], 0), (B_[3], 0)]),
            "p g | m v | twin (three sections)": run([(A[0], 0), (B_[0], 0), (B_[1], 0), (C_[0], 0), (A[1], 0)]),
            "p twin g | m v": run([(A[0], 0), (B_[0], 0), (B_[1], 0), (A[1], 0), (A[2], 0)]),
        }
    L.gpu_set_compute_prec(0)
    L.gpu_adam_set_weight_decay(0.0)
    for h, va in blocks:
        hip.hipMemUnmap(va, size)
        hip.hipMemRelease(h)
        hip.hipMemAddressFree(va, size)
    return out


def ceilings(L, nbytes=8 << 30):
    """What this box delivers to the simplest kernels of the library: write-only (fill), copy
    (16-byte vectors, read + write: the grid-stride loop of the counter calibration, and one
    workgroup per 16 KiB as the update does it, with and without non-temporal hints) and read-only
    (the sum of squares), for comparison with the update's mixed stream.  The two blocks come from
    gpu_malloc's two pools, i.e. from different memory sections, like the halves of an arena."""
    a, b = L.gpu_malloc(nbytes), L.gpu_malloc(nbytes)
    assert a and b
    assert L.gpu_memset(a, 1, nbytes) == 0 and L.gpu_memset(b, 0, nbytes) == 0
    L.gpu_device_sync()

    def timed(f, reps=10):
        f()
        L.gpu_device_sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            f()
        L.gpu_device_sync()
        return (time.perf_counter() - t0) / reps
    ss = C.c_double(0)
    n = min(nbytes // 4, (1 << 31) - 4096)
    out = {"bytes": nbytes,
           "write_only_GBps": round(nbytes / timed(lambda: L.gpu_memset(b, 3, nbytes)) / 1e9, 1),
           "copy_read_plus_write_GBps":
               round(2 * nbytes / timed(lambda: L.anni_copy_bytes(b, a, nbytes)) / 1e9, 1),
           "copy_in_the_updates_shape_GBps":
               round(2 * nbytes / timed(lambda: L.anni_copy_bytes_tiled(b, a, nbytes, 0)) / 1e9, 1),
           "copy_in_the_updates_shape_nontemporal_GBps":
               round(2 * nbytes / timed(lambda: L.anni_copy_bytes_tiled(b, a, nbytes, 1)) / 1e9, 1),
           "read_only_GBps":
               round(n * 4 / timed(lambda: L.gpu_grad_sumsq(a, n, C.byref(ss))) / 1e9, 1)}
    L.gpu_free(a)
    L.gpu_free(b)
    return out


def copy_calibration(L, nbytes):
    """Ten launches of the plain copy kernel: each reads nbytes and writes nbytes exactly."""
    from anni_amd.lm_adam import DeviceBuffer
    nbytes = nbytes // 16 * 16
    src, dst = DeviceBuffer(nbytes), DeviceBuffer(nbytes)
    assert L.gpu_memset(src.ptr, 1, nbytes) == 0 and L.gpu_memset(dst.ptr, 0, nbytes) == 0
    L.gpu_device_sync()
    t0 = time.perf_counter()
    for _ in range(10):
        assert L.anni_copy_bytes(dst.ptr, src.ptr, nbytes) == 0
    L.gpu_device_sync()
    ms = (time.perf_counter() - t0) * 1e3 / 10
    print(json.dumps({"copy_bytes": nbytes, "launches": 10, "ms_per_launch": round(ms, 4),
                      "GBps_read_plus_write": round(2 * nbytes / ms / 1e6, 1)}))


_LAP = [time.perf_counter()]


def lap(what):
    """Where the run's wall clock goes, on stderr (the result line on stdout stays one JSON object)."""
    now = time.perf_counter()
    print("[bench] %-32s %6.1f s" % (what, now - _LAP[0]), file=sys.stderr, flush=True)
    _LAP[0] = now


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 10 for the headline workload, 8 otherwise)")
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="555m", choices=sorted(WORKLOADS))
    ap.add_argument("--layout", default="auto", choices=["auto", "compact", "split"],
                    help="arena layout (split: two allocations in different 96 GiB sections of device memory)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-core baseline")
    ap.add_argument("--cpu-full", action="store_true",
                    help="time the multithreaded host baseline on the whole parameter set, not a sample")
    ap.add_argument("--no-legs", action="store_true",
                    help="skip the side legs of the headline workload (compact layout, 185m)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="only run the plain copy kernel over BYTES ten times (counter calibration)")
    ap.add_argument("--ckpt", action="store_true",
                    help="only time the optimizer block of a checkpoint written from / read into the arena")
    ap.add_argument("--ceilings", action="store_true",
                    help="only measure write-only, copy and read-only throughput of the box")
    ap.add_argument("--sections", action="store_true",
                    help="only map free device memory as 16 GiB physical blocks and time the update with its "
                         "flats in chosen blocks: shows the three 96 GiB sections the placement is about")
    ap.add_argument("--colsum", type=int, default=0, metavar="ROWS",
                    help="only time the bias / LayerNorm gradient column sums over ROWS token rows")
    ap.add_argument("--placement-cost", action="store_true",
                    help="only measure what the search for the arena's second block costs and leaves behind")
    ap.add_argument("--reference-caller-only", action="store_true",
                    help="only time the unchanged reference caller on this backend (one JSON line)")
    ap.add_argument("--ref-size", default="both", choices=["185m", "555m", "both"],
                    help="with --reference-caller-only: which of the two compiled sizes of the reference to run")
    ap.add_argument("--call-trace", action="store_true",
                    help="with --reference-caller-only: time every backend call of one step through the interposer")
    ap.add_argument("--cpu-budget", type=float, default=20.0, help="seconds for the CPU legs")
    ap.add_argument("--derived", nargs="?", const="both", default=None,
                    choices=["both", "fp8", "pack"],
                    help="the reference's own tensor list (separate Wq, Wk, Wv) with the fused "
                         "producers on: E4M3 twins of every matrix and a packed [Wq|Wk|Wv] per block")
    ap.add_argument("--ref-jsonl", default=None, metavar="FILE",
                    help="also append one row in the reference's bench-log schema (optimizer "
                         "phase only); steps are then timed one call each")
    a = ap.parse_args()
    if a.steps is None:
        a.steps = 10 if a.workload == "555m" else 8
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the step has no multi-GPU path); "
                 "use --gpus 1")
    if a.steps < 1 or a.warmup < 0:
        sys.exit("bench.py: --steps >= 1 and --warmup >= 0")

    from anni_amd import layout, lib
    from anni_amd.lm_adam import LmAdam
    L = lib.require_gpu()
    env = None
    if a.ref_jsonl:
        from anni_amd import bench_row
        env = bench_row.probe_env(L, os.path.dirname(os.path.abspath(__file__)))
    if a.copy_calibration:
        copy_calibration(L, a.copy_calibration)
        return
    if a.ckpt:
        print(json.dumps({"checkpoint_block": ckpt_leg(L)}))
        return
    if a.ceilings:
        print(json.dumps({"ceilings": ceilings(L)}))
        return
    if a.sections:
        print(json.dumps({"sections": sections_leg(L)}))
        return
    if a.colsum:
        print(json.dumps({"colsum_add": colsum_leg(L, a.colsum)}))
        return
    if a.placement_cost:
        print(json.dumps({"placement_cost": placement_cost_leg(L)}))
        return
    if a.reference_caller_only:
        print(json.dumps({"reference_caller_" + sz: reference_caller_leg(L, sz, a.call_trace)
                          for sz in ("185m", "555m") if a.ref_size in (sz, "both")}))
        return

    size, gt, mt, norm_bpp, upd_bpp = WORKLOADS[a.workload]
    tensors = layout.tensors(size, "reference" if a.derived else "baseline")
    packs, pack_elems, fp8_elems = [], 0, 0
    if a.derived:
        if gt != 0 or mt != 0:
            sys.exit("bench.py: --derived is measured on the all-f32 workloads")
        d = layout.SIZES[size][0]
        names = [t[0] for t in tensors]
        if a.derived != "pack":
            tensors = [(nm, cnt, f | (lib.T_FP8TWIN if f & lib.T_TWIN else 0))
                       for nm, cnt, f in tensors]
        fp8_elems = sum(cnt for _nm, cnt, f in tensors if f & lib.T_FP8TWIN)
        for b in range(layout.SIZES[size][3] if a.derived != "fp8" else 0):
            for k, w in enumerate(("wq", "wk", "wv")):
                packs.append((names.index("blk%d.%s" % (b, w)), d, pack_elems + k * d, 3 * d))
            pack_elems += 3 * d * d
    total = a.steps + a.warmup
    # Gradient slots: one per step while they fit 32 GiB of device memory (14 at 555M);
    # beyond that the steps run in batches, the slots being refilled between batches with the
    # clock stopped, so that any --steps keeps the arena, and with it the placement, the same.
    n_params = sum(t[1] for t in tensors)
    slot_bytes = -(-n_params * ELEM[gt] // (2 << 20)) * (2 << 20)
    n_slots = min(total, max(4, (32 << 30) // slot_bytes))
    t_create = time.perf_counter()
    opt = LmAdam(tensors, grad_type=gt, moment_type=mt, twins=True, skip_nonfinite=True,
                 grad_slots=n_slots, layout={"auto": 0, "compact": 1, "split": 2}[a.layout],
                 beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    t_create = (time.perf_counter() - t_create) * 1e3
    n = opt.n
    assert L.anni_fill_normal_f32(opt.o.d_param, n, 20260101, 1, 0.0, 0.02) == 0
    if a.derived:
        opt.enable_derived(packs, pack_elems)
    opt.seed_twins()
    ring, scales = fill_grad_slots(L, opt, tensors, min(n_slots, total), gt, 20260101)

    # per-step inputs: warmup(100)+cosine lr at schedule steps 0.., grad scale straddling the clip
    from anni_amd import lm_adam
    lrs = [lm_adam.step_lr(3e-4, s, 100, 1000, "cosine") for s in range(total)]
    unit = 1.0 / (math.sqrt(n) * 1e-3)
    gss = [unit * (1.7 if s % 2 else 0.6) for s in range(total)]

    per_step_ms, skipped_steps, der_acc = [], [], [0.0]

    def run(first, count, per_kernel):
        ptrs = (C.c_void_p * count)(*[ring[(first + i) % n_slots] for i in range(count)])
        lr = (C.c_double * count)(*lrs[first:first + count])
        gs = (C.c_double * count)(*gss[first:first + count])
        ms, ms_a, ms_b = C.c_float(0), C.c_float(0), C.c_float(0)
        if gt == 2 or (a.ref_jsonl and per_kernel):
            # fp8: each flat carries its own per-tensor scales -> one call per step
            # (also when the per-step distribution is wanted)
            tot = sa = sb = 0.0
            for i in range(count):
                if gt == 2:
                    opt.o.d_gscale = scales[(first + i) % n_slots].ptr
                one = (C.c_void_p * 1)(ptrs[i])
                rc = L.anni_adam_time_steps(opt.h, 1, one, 1, C.byref(C.c_double(lr[i])),
                                            C.byref(C.c_double(gs[i])), C.byref(ms),
                                            C.byref(ms_a) if per_kernel else None,
                                            C.byref(ms_b) if per_kernel else None)
                assert rc == 0, L.gpu_debug_last_error()
                tot, sa, sb = tot + ms.value, sa + ms_a.value, sb + ms_b.value
                if per_kernel:
                    per_step_ms.append(ms.value)
                    der_acc[0] += L.anni_adam_timed_derived_ms(opt.h) if a.derived else 0.0
                    o = opt.sync_stats() if a.ref_jsonl else None
                    if o is not None and (o.last_skipped or not math.isfinite(o.last_grad_norm)):
                        skipped_steps.append(first + i)
            return tot, sa, sb
        rc = L.anni_adam_time_steps(opt.h, count, ptrs, count, lr, gs, C.byref(ms),
                                    C.byref(ms_a) if per_kernel else None,
                                    C.byref(ms_b) if per_kernel else None)
        assert rc == 0, L.gpu_debug_last_error()
        if per_kernel and a.derived:
            der_acc[0] += L.anni_adam_timed_derived_ms(opt.h)
        return ms.value, ms_a.value, ms_b.value

    # steps 0 .. total-1 in batches of n_slots (one batch when they all fit); the clock runs only
    # over the timed steps of each batch, bracketed by device synchronisations
    ev_ms = ms_sumsq = ms_update = wall_ms = 0.0
    for b0 in range(0, total, n_slots):
        b1 = min(b0 + n_slots, total)
        if b0:
            refill = fill_grad_slots(L, opt, tensors, b1 - b0, gt, 20260101, b0)
            for sc_old in scales:
                if sc_old is not None:
                    sc_old.free()
            ring, scales = refill
        w1 = min(max(a.warmup, b0), b1)                 # [b0, w1) untimed, [w1, b1) timed
        if w1 > b0:
            run(b0, w1 - b0, False)
        if b1 > w1:
            L.gpu_device_sync()
            t0 = time.perf_counter()
            e, sa, sb = run(w1, b1 - w1, True)
            L.gpu_device_sync()
            wall_ms += (time.perf_counter() - t0) * 1e3
            ev_ms, ms_sumsq, ms_update = ev_ms + e, ms_sumsq + sa, ms_update + sb

    peak_mb = 0.0
    fr, tt = C.c_size_t(0), C.c_size_t(0)
    if L.gpu_mem_info(C.byref(fr), C.byref(tt)) == 0:
        peak_mb = (tt.value - fr.value) / 1048576.0
    st = opt.sync_stats()
    assert opt.t == total and math.isfinite(st.last_grad_norm)
    bpp = norm_bpp + upd_bpp
    ms_step = wall_ms / a.steps
    # derived outputs: 2 more bytes written per packed element by the update, and the E4M3 pass
    # reads p (4) and writes the code (1) of every flagged element
    extra_bytes = 2 * pack_elems + 5 * fp8_elems
    step_gbps = (n * bpp + extra_bytes) / (ms_step * 1e-3) / 1e9
    upd_ms = ms_update / a.steps
    sumsq_ms = ms_sumsq / a.steps
    upd_bytes = n * upd_bpp + 2 * pack_elems
    upd_gbps = upd_bytes / (upd_ms * 1e-3) / 1e9
    traffic, traffic_digest, traffic_current = profiled_traffic(a.workload)
    out = {
        "metric": "AdamW step HBM GB/s (algorithmic bytes / step time; AdamW + global-norm clip "
                  "+ decay + bf16 twins), %s param set" % a.workload,
        "value": round(step_gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": a.workload, "storage": STORAGE[a.workload], "params": n, "tensors": len(tensors),
                   "bytes_per_param": bpp, "clip": 1.0, "weight_decay": 0.1, "beta2": 0.95,
                   "lr": "3e-4 warmup100+cosine", "twins": "bf16 RNE on matrices",
                   "layout": "split" if opt.split else "compact",
                   "placement_apart_ratio": round(opt.apart_ratio, 3),
                   "placement_probe_GBps": round(opt.probe_gbps, 1),
                   "placement_walked_GiB": round(opt.placement_cost[0], 1),
                   "placement_ms": round(opt.placement_cost[1], 1),
                   "arena_bytes": opt.arena_bytes, "resident_bytes": opt.resident_bytes,
                   "grad_slots": n_slots, "arena_create_ms": round(t_create, 1),
                   "launches_per_step": 2},
        "params_per_s": round(n / (ms_step * 1e-3), 1),
        "pct_of_hbm_peak": round(100.0 * step_gbps / HBM_PEAK_GBPS, 2),
        "event_ms_per_step": round(ev_ms / a.steps, 4),
        "roofline": {"bound": "hbm",
                     "kernel": "adam_update_kernel" if gt == 0 and mt == 0 else "adam_update_pipe_kernel",
                     "achieved": round(upd_gbps, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(upd_gbps / HBM_PEAK_GBPS, 4),
                     "traffic": None if a.derived else traffic,
                     "profile_kernel_sources_sha1": None if a.derived else traffic_digest,
                     "profile_matches_these_sources": None if a.derived else traffic_current,
                     "bytes_per_launch": upd_bytes, "avg_ms": round(upd_ms, 4)},
        "sumsq_kernel": {"avg_ms": round(sumsq_ms, 4), "bytes_per_launch": n * norm_bpp,
                         "achieved": round(n * norm_bpp / (sumsq_ms * 1e-3) / 1e9, 1)
                         if sumsq_ms > 0 else None, "unit": "GB/s"},
        "last_grad_norm": st.last_grad_norm, "last_clipped": int(st.last_clipped),
    }
    if gt == 2 and len(QUANT_MS) > 1:
        # the producer of the fp8 gradient format: float flat -> E4M3 codes + one scale per tensor
        # (reads the source twice, writes one byte per element); wall clock, first call left out
        q_ms = sorted(QUANT_MS[1:])[len(QUANT_MS[1:]) // 2]
        out["grad_quantizer"] = {"what": "anni_adam_quantize_grads: amax per tensor, then E4M3 codes + scales, "
                                         "4 launches for all %d tensors" % len(tensors),
                                 "median_ms": round(q_ms, 4), "bytes": 9 * n,
                                 "GBps": round(9 * n / (q_ms * 1e-3) / 1e9, 1)}
    if a.derived:
        der_ms = der_acc[0] / a.steps
        out["config"]["derived"] = {"both": "E4M3 twins of every matrix + packed [Wq|Wk|Wv] per block",
                                    "fp8": "E4M3 twins of every matrix",
                                    "pack": "packed [Wq|Wk|Wv] per block"}[a.derived]
        out["config"]["launches_per_step"] = 3 if fp8_elems else 2
        out["derived"] = {
            "fp8_twin_kernel": {"avg_ms": round(der_ms, 4), "bytes_per_launch": 5 * fp8_elems,
                                "achieved": round(5 * fp8_elems / (der_ms * 1e-3) / 1e9, 1)
                                if der_ms > 0 else None, "unit": "GB/s"},
            "fp8_twin_elems": fp8_elems, "packed_elems": pack_elems,
            "separate_passes_would_move_bytes": 9 * fp8_elems + 4 * pack_elems,
            "fused_moves_bytes": extra_bytes}
    lap("headline workload on the GPU")
    if not a.no_cpu:
        mt_out, serial_out = cpu_baselines(size, norm_bpp, upd_bpp, a.cpu_budget, a.cpu_full)
        out["cpu_baseline"] = mt_out
        out["cpu_reference_serial"] = serial_out
        out["gpu_over_cpu"] = round(step_gbps / mt_out["value"], 1)
        lap("host baselines")
    opt.free()
    opt = None
    if not a.no_cpu and not a.no_legs:
        # the unchanged reference caller on this backend, right after the headline's arena was freed
        try:
            for size in ("185m", "555m"):
                ref_leg = reference_caller_leg(L, size)
                if ref_leg:
                    out["reference_caller_" + size] = ref_leg
                lap("reference caller " + size)
        except Exception as e:                      # the checker must never sink the bench line
            out["reference_caller_error"] = repr(e)
    if a.workload == "555m" and not a.derived and not a.no_legs:
        # the same workload with every flat in ONE allocation, and the other configurations the
        # metric names, each on an arena of its own after the one before it was freed
        try:
            out["layout_compact"] = short_leg(L, "555m", "compact")
            lap("one-allocation leg")
            out["workloads"] = {}
            for w in ("185m", "555m-bf16", "1p4b-fp8"):
                out["workloads"][w] = short_leg(L, w, "auto")
                lap("workload " + w)
        except Exception as e:                      # a side leg must never sink the bench line
            out["side_legs_error"] = repr(e)
    if a.ref_jsonl:
        row = bench_row.adam_row(env, a.workload, size, gt, mt, n, a.warmup, per_step_ms, 3e-4,
                                 peak_mb, not skipped_steps)
        bench_row.append(a.ref_jsonl, row)
        out["ref_jsonl_row"] = row
        out["vram_used_before_mb"] = env["vram_used_mb"]
    print(json.dumps(out))
    if opt is not None:
        opt.free()


if __name__ == "__main__":
    main()
