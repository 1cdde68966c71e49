#!/usr/bin/env python3
"""Headline benchmark: foreground latency under a saturating background on one MI355X.

Default workload (`--config 2`): a background XQueue streams fp32 AXPY y = 0.5*x + y over
2^28 elements back to back (Level-1, HPF policy, priority 1); a foreground XQueue submits the
same kernel over 2^22 elements every 20 ms (priority 2). One "step" is one foreground command
under contention (submit -> XQueueWaitAll returns); `--warmup` untimed steps, then exactly
`--steps` timed ones give `ms_per_step`.

Prints ONE JSON line. `value` is the foreground p99 latency under contention in microseconds
(percentile rule sorted[floor(p*n)], as XSched's own DataProcessor) over a block of FIXED size
(400 samples, whatever --steps says: the p99 of 20 samples would be their maximum). The line
also carries: the background kernel's achieved rate against the MI355X peak (`roofline`), where
a foreground command's latency goes and the plain-HIP floor beside it (`fg_latency_us`), a
bit-exact check of the buffers the timed phases produced (`bit_exact`), guard overhead and
Level-2 preemption latency, compact blocks for the other four configurations (`others`), and a
CPU baseline of the same workload (`cpu_baseline`).

Each configuration also prints a full line of its own:
    --config 1   CPU only, host adapter: two XQueues, L1, HPF, window 8/4; background streams of
                 1000 fp32 vector additions over 2^20 elements, foreground 2^16 every 10 ms
    --config 3   Level-2 guarded bf16 GEMM 8192^3 back to back, foreground GEMM 1024^3
                 every 5 ms (MFMA roofline, guard on/off, preemption latency)
    --config 4   laxity policy: 4 background XQueues histogramming 2^26 Zipf keys,
                 foreground 2^20 keys every 2 ms with a 1 ms deadline (deadline-miss rate)
    --config 5   16 XQueues, priorities 0-15, cycling AXPY 2^24 / GEMM 2048^3 / histogram
                 2^24, exponential arrivals (mean 5 ms, seed 7), HPF, Level-2

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1|2|3|4|5] [--quick]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
os.environ.setdefault("XLOG_LEVEL", "WARN")

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16 MFMA, vendor figure
# Background in-flight window: one kernel running and one queued behind it keeps the
# device busy (a 2^28 AXPY runs ~0.5 ms, a launch costs ~10 us) and bounds what a
# suspended queue still has on the device to two kernels.
BG_THRESHOLD, BG_BATCH = 2, 1


def axpy_bytes(n):
    return 12.0 * n  # read x, read y, write y


def gemm_flops(n):
    return 2.0 * n * n * n


def hist_bytes(n):
    return 4.0 * n  # one int32 key read


def fg_summary(H, alone, cont):
    p50a, p99a = H.pct(alone, 0.50), H.pct(alone, 0.99)
    p50c, p99c = H.pct(cont, 0.50), H.pct(cont, 0.99)
    return {"alone_p50": p50a, "alone_p99": p99a, "contended_p50": p50c, "contended_p99": p99c,
            "p99_ratio": p99c / p99a if p99a else None}


def bg_ms_per_launch(H, kind, n, level, guard, commands=40, warm=8):
    """Average device time per background launch for one guard variant, no foreground."""
    cfg = H.Config(0, 1, H.spec(kind, n, guard, level, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(kind, 0, 0, 1, 8, 4, 2), 64, 0)
    with H.Bench(cfg) as b:
        b.bg_alone(warm)
        res = b.bg_alone(commands)
        return res.bg_stream_ms / res.bg_stream_cmds


def preempt_latency(H, kind, n, level, samples, guard=1):
    cfg = H.Config(0, 1, H.spec(kind, n, guard, level, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(kind, 0, 0, 1, 8, 4, 2), 64, 0)
    with H.Bench(cfg) as b:
        sus, resume, res = b.preempt(samples)
        return sus, resume, list(res.stats)


def device_drain(H, kind, n, level, samples, guard=1):
    """Device-side preemption latency (HIP events, see bench.h), microseconds."""
    cfg = H.Config(0, 1, H.spec(kind, n, guard, level, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(kind, 0, 0, 1, 8, 4, 2), 64, 0)
    with H.Bench(cfg) as b:
        drain, _ = b.preempt_device_timed(samples)
        return drain


def preempt_block(H, kind, n, quick):
    sus2, res2, st2 = preempt_latency(H, kind, n, 2, 60 if quick else 200)
    sus1, _, _ = preempt_latency(H, kind, n, 1, 30 if quick else 60)
    dev2 = device_drain(H, kind, n, 2, 60 if quick else 200)
    dev1 = device_drain(H, kind, n, 1, 30 if quick else 60)
    return {"level2_device_drain_p50": H.pct(dev2, 0.5), "level2_device_drain_p99": H.pct(dev2, 0.99),
            "level1_device_drain_p50": H.pct(dev1, 0.5), "level1_device_drain_p99": H.pct(dev1, 0.99),
            "level2_suspend_sync_p50": H.pct(sus2, 0.5), "level2_suspend_sync_p99": H.pct(sus2, 0.99),
            "level2_resume_p50": H.pct(res2, 0.5), "level2_resume_p99": H.pct(res2, 0.99),
            "level1_suspend_sync_p50": H.pct(sus1, 0.5), "level1_suspend_sync_p99": H.pct(sus1, 0.99),
            "level2_stats": st2}


LATENCY_BLOCK = 400   # foreground samples per phase of the fixed-size latency block
BREAKDOWN_SAMPLES = 200


def contended_run(H, cfg, steps, warmup, bg_warm=8, bg_cmds=40, block=0, keep=None):
    """fg alone -> bg alone -> contended. With `block` > 0 the latencies come from phases of
    that many samples (after `warmup` untimed ones) and the `steps` timed steps are a phase of
    their own; otherwise (the per-configuration lines) the timed steps are the samples.
    `keep`, when given, is called with the live harness before it is torn down."""
    with H.Bench(cfg) as b:
        n_alone = (block or steps) + warmup
        alone, _ = b.fg_alone(n_alone)
        b.bg_alone(bg_warm)
        alone_res = b.bg_alone(bg_cmds)
        bg_alone_ms = alone_res.bg_stream_ms / alone_res.bg_stream_cmds
        if warmup:
            b.contended(warmup)
        t0 = time.perf_counter()
        timed, timed_res = b.contended(steps)
        wall = time.perf_counter() - t0
        cont, res = (b.contended(block) if block else (timed, timed_res))
        out = {"fg_alone": alone[warmup:], "fg_contended": cont, "fg_timed_steps": timed, "wall_s": wall,
               "bg_alone_ms": bg_alone_ms,
               "bg_alone_cmds": int(alone_res.bg_commands), "bg_alone_elapsed": alone_res.elapsed_s,
               "bg_cont_ms": (res.bg_stream_ms / res.bg_stream_cmds) if res.bg_stream_cmds else None,
               "bg_cont_launches": int(res.bg_stream_cmds),
               "bg_cont_cmds": int(res.bg_commands), "bg_cont_elapsed": res.elapsed_s,
               "deadline_miss": int(res.fg_deadline_miss), "stats": list(res.stats)}
        if keep is not None:
            out["kept"] = keep(b)
        return out


def recorded_traffic(summary, applies=True):
    """HBM bytes per launch of a kernel as recorded by the two rocprofv3 counter runs
    summarised in profiles/<summary> (counters cannot be read from inside this process);
    None when the workload is not the one that summary covers, or the summary is absent."""
    path = os.path.join(ROOT, "profiles", summary)
    if not applies or not os.path.exists(path):
        return None
    for ln in open(path):
        if ln.startswith("traffic_bytes_per_launch_plain:"):
            return int(ln.split(":")[1])
    return None


def cpu_baseline(config=2, compact=False):
    """The same workload on host cores, on XSched's own host loop compiled from the reference
    sources (oracle/_ref, kind "reference"); bounded sample."""
    try:
        from oracle import cpu_baseline as cb
        if config == 1:
            return cb.run_config1_sample(150)
        if config == 3:
            return cb.run_config3_sample(100 if compact else 300)
        if config == 4:
            return cb.run_config4_sample(200 if compact else 600)
        if config == 5:
            return cb.run_config5_sample(2.0 if compact else 4.0)
        return cb.run_config2_sample(15.0, samples=300)
    except Exception as e:  # checker libraries not built
        return {"value": None, "unit": "us", "cores": 0, "kind": "reference", "sample": f"unavailable: {e}"}


def base_line(a, value, wall_s, workload, extra_cfg):
    cfg = {"workload": workload, "percentile_rule": "sorted[floor(p*n)]"}
    cfg.update(extra_cfg)
    return {"metric": "fg_p99_latency_us_under_contention", "value": value, "unit": "us", "n_gpus": 1,
            "steps": a.steps, "warmup": a.warmup, "ms_per_step": wall_s * 1e3 / a.steps,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "data": "synthetic",
            "config": cfg}


# ---- bit-exact checks against the CPU oracle (the checker; nothing timed runs through it) ----

def axpy_slices(n, pieces=8, length=1 << 12):
    """Slices spread over [0, n): the head, the tail and evenly spaced ones in between."""
    length = min(length, n)
    starts = sorted({0, n - length} | {((n - length) * k // (pieces - 1)) // 4 * 4 for k in range(pieces)})
    return [(s0, length) for s0 in starts]


def check_axpy_buffer(b, which, q, lane_id, n, seed=0, full=False):
    """Compares a result buffer of the harness, bit for bit, with `applied` oracle
    applications of y = fma(0.5, x, y) to the seeded inputs: the whole buffer when `full`,
    else slices (an application count in the thousands makes the whole buffer a matter of
    minutes on the host)."""
    import numpy as np
    import oracle
    s_x, s_y = lane_id * 4, lane_id * 4 + 1
    checked = 0
    applied = None
    for first, count in ([(0, n)] if full else axpy_slices(n)):
        got, applied = b.read(which, q, first, count, np.float32)
        want = oracle.axpy(0.5, oracle.fill_uniform(seed, s_x, first, count),
                           oracle.fill_uniform(seed, s_y, first, count), times=applied)
        if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
            return {"ok": False, "applied": applied, "first_bad_slice": first}
        checked += count
    return {"ok": True, "applied": applied, "elements_checked": checked}


def full_buffer_check(H, bg_n, fg_n):
    """Fresh queues at the full sizes. Level 1, plain kernels: two background and three
    foreground commands, then EVERY element of both buffers against the oracle. Level 2,
    guarded kernels: the background streams through three suspend / resume rounds (a hundred
    or more commands, flushed and replayed), then slices of its buffer against as many oracle
    applications as commands were applied."""
    cfg = H.Config(H.HPF, 1, H.spec(H.AXPY, bg_n, 0, 1, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(H.AXPY, fg_n, 0, 1, 8, 4, 2, period_us=2000), 2, 0)
    with H.Bench(cfg) as b:
        b.bg_alone(2)
        b.fg_alone(3)
        out = {"level1_plain_every_element": {"bg": check_axpy_buffer(b, 0, 0, 1, bg_n, full=True),
                                              "fg": check_axpy_buffer(b, 1, 0, 0, fg_n, full=True)}}
    cfg = H.Config(H.HPF, 1, H.spec(H.AXPY, bg_n, 1, 2, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(H.AXPY, fg_n, 1, 2, 8, 4, 2, period_us=2000), 8, 0)
    with H.Bench(cfg) as b:
        _, _, res = b.preempt(3)
        out["level2_guarded_preempted_slices"] = {"bg": dict(check_axpy_buffer(b, 0, 0, 1, bg_n),
                                                             replayed_launches=int(res.stats[1]))}
    return out


def check_hist_bins(b, which, q, lane_id, n, seed=0, bins=65536):
    """All bins of a histogram lane against `applied` times the oracle's counts of the lane's
    seeded Zipf keys (modulo 2^32), bit for bit."""
    import numpy as np
    import oracle
    got, applied = b.read(which, q, 0, bins, np.uint32)
    one = oracle.histogram(oracle.fill_zipf(seed, lane_id * 4, 0, n), bins).astype(np.uint64)
    ok = int(one.sum()) == n and np.array_equal(got.astype(np.uint64), (one * applied) & 0xFFFFFFFF)
    return {"ok": bool(ok), "applied": applied, "bins_checked": bins}


def check_gemm_rows(b, which, q, lane_id, n, rows, seed=0):
    """Rows [r, r + 4) of C, for each r, against the oracle's product of the lane's seeded
    matrices (ascending-k fmaf, one rounding to bf16): the matrix cores sum in another order,
    so the bar is the stated tolerance 2^-8 * |ref| + 2^-16 * sqrt(K); bit-exactness of this
    kernel is the separate comparison of a preempted run's C with an uninterrupted one's."""
    import numpy as np
    import oracle
    bmat = oracle.fill_normal_bf16(seed, lane_id * 4 + 1, 0, n * n)
    worst, applied = 0.0, None
    for r in rows:
        got, applied = b.read(which, q, r * n, 4 * n, np.uint16)
        a = oracle.fill_normal_bf16(seed, lane_id * 4, r * n, 4 * n)
        _, want = oracle.gemm_bf16(a, bmat, 4, n, n, want_f32=True)
        tol = np.abs(want) * 2.0 ** -8 + 2.0 ** -16 * np.sqrt(n)
        worst = max(worst, float(np.max(np.abs(oracle.bf16_bits_to_f32(got).reshape(4, n) - want) / tol)))
    return {"ok": bool(worst <= 1.0), "applied": applied, "rows_checked": 4 * len(rows), "worst_error_over_tolerance": round(worst, 3)}


def breakdown_block(b, H, samples):
    """Where a foreground command's latency goes (see bench.h), alone and contended, through the
    XQueue, through the adapter alone, and for plain HIP launches (the floor)."""
    out = {}
    for name, mode in (("xqueue", 0), ("adapter_only", 1), ("plain_hip_floor", 2)):
        for cont in (False, True):
            r = b.fg_breakdown(samples, mode, cont)
            out[name + ("_contended" if cont else "_alone")] = {
                k: {"p50": H.pct(v[5:], 0.5), "p99": H.pct(v[5:], 0.99)} for k, v in r.items()}
    out["samples"] = samples - 5
    out["note"] = ("submit = host time to hand over (two timing-event records + the kernel), device = between "
                   "the two events, wait = until the host knows, total = submit + wait; the XQueue rows carry "
                   "two extra event-record commands per sample, the fixed-size block above does not")
    return out


# ---- configurations ------------------------------------------------------------------

def config1(a):
    """CPU only: the host adapter (libhalhost.so), no GPU and no torch."""
    import ctypes
    import numpy as np
    import oracle
    import xsched_amd as xs
    h = xs.halhost()
    n_bg, n_fg, samples = 1 << 20, 1 << 16, (100 if a.quick else LATENCY_BLOCK)

    class Cfg(ctypes.Structure):
        _fields_ = [("bg_n", ctypes.c_uint64), ("fg_n", ctypes.c_uint64), ("bg_burst", ctypes.c_int32),
                    ("threshold", ctypes.c_int32), ("batch", ctypes.c_int32), ("samples", ctypes.c_int32),
                    ("period_us", ctypes.c_int64)]

    class Res(ctypes.Structure):
        _fields_ = [("alone_s", ctypes.c_double), ("contended_s", ctypes.c_double),
                    ("bg_commands", ctypes.c_uint64), ("fg_commands", ctypes.c_uint64)]

    def filled(n, stream):
        arr = np.empty(n, np.float32)
        h.HostBenchFillUniform(arr.ctypes.data, 0, n, 0, stream)
        return arr
    bg_a, bg_b, fg_a, fg_b = filled(n_bg, 4), filled(n_bg, 5), filled(n_fg, 0), filled(n_fg, 1)
    bg_c, fg_c = np.zeros(n_bg, np.float32), np.zeros(n_fg, np.float32)
    cfg, res = Cfg(n_bg, n_fg, 1000, 8, 4, samples, 10000), Res()
    alone, cont = (ctypes.c_double * samples)(), (ctypes.c_double * samples)()
    t0 = time.perf_counter()
    xs.check(h.HostBenchRunVecAdd(ctypes.byref(cfg), bg_a.ctypes.data, bg_b.ctypes.data, bg_c.ctypes.data,
                                  fg_a.ctypes.data, fg_b.ctypes.data, fg_c.ctypes.data, alone, cont,
                                  ctypes.byref(res)))
    wall = time.perf_counter() - t0
    alone, cont = list(alone)[5:], list(cont)[5:]
    # the checker: seeded inputs and sums recomputed by the oracle
    exact = (np.array_equal(bg_a, oracle.fill_uniform(0, 4, 0, n_bg)) and np.array_equal(fg_b, oracle.fill_uniform(0, 1, 0, n_fg))
             and np.array_equal(bg_c.view(np.uint32), oracle.vecadd(bg_a, bg_b).view(np.uint32))
             and np.array_equal(fg_c.view(np.uint32), oracle.vecadd(fg_a, fg_b).view(np.uint32)))
    pct = lambda v, p: sorted(v)[min(int(p * len(v)), len(v) - 1)]
    line = {"metric": "fg_p99_latency_us_under_contention", "value": pct(cont, 0.99), "unit": "us", "n_gpus": 0,
            "steps": len(cont), "warmup": 5, "ms_per_step": res.contended_s * 1e3 / samples,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "data": "synthetic", "dtype": "f32",
            "config": {"workload": "cfg1: host adapter, 2 XQueues, L1 HPF, window 8/4, bg streams of 1000 fp32 vector "
                                   "additions 2^20, fg 2^16 every 10 ms", "percentile_rule": "sorted[floor(p*n)]"},
            "fg_latency_us": {"alone_p50": pct(alone, 0.5), "alone_p99": pct(alone, 0.99),
                              "contended_p50": pct(cont, 0.5), "contended_p99": pct(cont, 0.99),
                              "p99_ratio": pct(cont, 0.99) / pct(alone, 0.99), "samples": len(cont)},
            "bg": {"commands_while_contended": int(res.bg_commands),
                   "host_GBs": 12.0 * n_bg * res.bg_commands / res.contended_s / 1e9},
            "bit_exact": bool(exact), "wall_s": wall,
            "roofline": {"bound": "hbm", "achieved": 12.0 * n_bg * res.bg_commands / res.contended_s / 1e9, "peak": None,
                         "unit": "GB/s", "frac": None, "traffic": None,
                         "note": "host DRAM, one executor thread: informational, no device kernel in this configuration"}}
    return line


def config2(H, a):
    bg_n, fg_n = 1 << a.bg_log2, 1 << a.fg_log2
    cfg = H.Config(H.HPF, 1, H.spec(H.AXPY, bg_n, 1, 1, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(H.AXPY, fg_n, 0, 1, 8, 4, 2, period_us=20000), 64, 0)
    block = 100 if a.quick else LATENCY_BLOCK

    def after(b):
        kept = {"breakdown": None if a.quick else breakdown_block(b, H, BREAKDOWN_SAMPLES)}
        kept["bit_exact_slices"] = {"bg": check_axpy_buffer(b, 0, 0, 1, bg_n), "fg": check_axpy_buffer(b, 1, 0, 0, fg_n)}
        return kept
    r = contended_run(H, cfg, a.steps, a.warmup, block=block, keep=after)
    fg = fg_summary(H, r["fg_alone"], r["fg_contended"])
    fg["samples_per_phase"] = block
    fg["timed_steps"] = {"n": a.steps, "p50": H.pct(r["fg_timed_steps"], 0.5), "max": max(r["fg_timed_steps"])}
    per_launch_ms = r["bg_cont_ms"] or r["bg_alone_ms"]
    achieved = axpy_bytes(bg_n) / (per_launch_ms * 1e-3) / 1e9
    line = base_line(a, fg["contended_p99"], r["wall_s"],
                     "cfg2: L1 HPF, bg AXPY 2^%d back-to-back, fg AXPY 2^%d every 20 ms" % (a.bg_log2, a.fg_log2),
                     {"bg_threshold": BG_THRESHOLD, "bg_batch": BG_BATCH, "fg_threshold": 8, "fg_batch": 4,
                      "value_from": "p99 of %d contended foreground samples (fixed-size block, not the --steps region)" % block})
    line["dtype"] = "f32"
    line["fg_latency_us"] = fg
    if r["kept"]["breakdown"]:
        line["fg_latency_us"]["breakdown"] = r["kept"]["breakdown"]
    line["bg"] = {"alone_GBs": axpy_bytes(bg_n) / r["bg_alone_ms"] / 1e6,
                  "contended_GBs": axpy_bytes(bg_n) * r["bg_cont_cmds"] / r["bg_cont_elapsed"] / 1e9,
                  "commands_in_latency_block": r["bg_cont_cmds"]}
    line["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": achieved / HBM_PEAK_GBS, "traffic": recorded_traffic("axpy_2p28_hbm_traffic.md", bg_n == 1 << 28),
                        "kernel": "AxpyPersistentKernel<3, false>" if bg_n >= 1 << 23 else "AxpyVec4Kernel<false, 4>",
                        "algorithmic_bytes_per_launch": axpy_bytes(bg_n),
                        "avg_launch_ms": per_launch_ms, "launches_timed": r["bg_cont_launches"],
                        "timed_with": "HIP events on the background stream around the contended latency block"}
    slices = r["kept"]["bit_exact_slices"]
    line["bit_exact"] = {"after_timed_phases_slices": slices}
    if not a.quick:
        line["bit_exact"]["fresh_run_every_element"] = full_buffer_check(H, bg_n, fg_n)
    line["bit_exact"]["all_ok"] = all(
        v["ok"] for grp in ([slices] + list(line["bit_exact"].get("fresh_run_every_element", {}).values())) for v in grp.values())
    if not a.quick:
        ms_plain = bg_ms_per_launch(H, H.AXPY, bg_n, 1, 0)
        ms_guard = bg_ms_per_launch(H, H.AXPY, bg_n, 1, 2)
        ms_l2 = bg_ms_per_launch(H, H.AXPY, bg_n, 2, 1)
        line["guard"] = {"plain_GBs": axpy_bytes(bg_n) / ms_plain / 1e6,
                         "guarded_GBs": axpy_bytes(bg_n) / ms_guard / 1e6,
                         "level2_GBs": axpy_bytes(bg_n) / ms_l2 / 1e6,
                         "guard_overhead_frac": 1.0 - ms_plain / ms_guard,
                         "level2_overhead_frac": 1.0 - ms_plain / ms_l2}
        line["preempt_us"] = preempt_block(H, H.AXPY, bg_n, False)
    return line


def config3(H, a):
    compact = getattr(a, "compact", False)
    bg_n, fg_n = 8192, 1024
    cfg = H.Config(H.HPF, 1, H.spec(H.GEMM, bg_n, 1, 2, BG_THRESHOLD, BG_BATCH, 1),
                   H.spec(H.GEMM, fg_n, 0, 1, 8, 4, 2, period_us=5000), 64, 0)
    def after(b):
        """C of the background queue after the timed phases (hundreds of commands, flushed and
        replayed whenever the foreground became ready), then after a run of suspensions in
        flight, then after one more command that nothing interrupts: the same bits each time.
        Rows of both queues' C against the oracle."""
        import numpy as np
        contended, n_cont = b.read(0, 0, 0, bg_n * bg_n, np.uint16)
        _, _, pres = b.preempt(20)
        preempted, _ = b.read(0, 0, 0, bg_n * bg_n, np.uint16)
        b.bg_alone(1)
        clean, n_clean = b.read(0, 0, 0, bg_n * bg_n, np.uint16)
        same = bool(np.array_equal(contended, clean) and np.array_equal(preempted, clean))
        return {"bg_preempted_equals_uninterrupted": {"ok": same, "commands_applied": n_clean, "elements_compared": bg_n * bg_n,
                                                      "replayed_launches": int(pres.stats[1]), "deactivations": int(pres.stats[2])},
                "bg_rows_vs_oracle": check_gemm_rows(b, 0, 0, 1, bg_n, [0, bg_n // 2, bg_n - 4]),
                "fg_rows_vs_oracle": check_gemm_rows(b, 1, 0, 0, fg_n, [0, fg_n - 4])}
    r = contended_run(H, cfg, a.steps, a.warmup, bg_warm=40, bg_cmds=24, keep=after)
    fg = fg_summary(H, r["fg_alone"], r["fg_contended"])
    per_launch_ms = r["bg_alone_ms"]
    achieved = gemm_flops(bg_n) / (per_launch_ms * 1e-3) / 1e12
    line = base_line(a, fg["contended_p99"], r["wall_s"],
                     "cfg3: L2 HPF, bg bf16 GEMM 8192^3 guarded back-to-back, fg GEMM 1024^3 every 5 ms",
                     {"bg_threshold": BG_THRESHOLD, "bg_batch": BG_BATCH, "fg_threshold": 8, "fg_batch": 4})
    line["dtype"] = "bf16"
    line["fg_latency_us"] = fg
    line["bit_exact"] = dict(r["kept"], all_ok=all(v["ok"] for v in r["kept"].values()))
    line["bg"] = {"alone_TFLOPs": achieved,
                  "contended_TFLOPs": gemm_flops(bg_n) * r["bg_cont_cmds"] / r["bg_cont_elapsed"] / 1e12,
                  "commands_in_timed_region": r["bg_cont_cmds"], "level2_stats": r["stats"]}
    line["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TF, "unit": "TFLOP/s",
                        "frac": achieved / MFMA_BF16_PEAK_TF, "traffic": recorded_traffic("gemm_8192_hbm_traffic.md"), "kernel": "GemmBf16Kernel",
                        "algorithmic_flops_per_launch": gemm_flops(bg_n), "avg_launch_ms": per_launch_ms}
    if not a.quick:
        # Seven (five in the compact block) alternating rounds of 24 launches per form, after 40
        # untimed ones each: the device runs this kernel against its power limit, and after an
        # idle spell the clock first overshoots, then drops by up to 30 %, and needs some 30
        # launches to settle. The settled clock still moves by a
        # few percent within seconds, more than the guard costs: the overheads are medians of
        # the per-round ratios (forms measured within a second of each other), the rates are
        # medians of each form.
        rounds = [(bg_ms_per_launch(H, H.GEMM, bg_n, 1, 0, 24, 40), bg_ms_per_launch(H, H.GEMM, bg_n, 1, 2, 24, 40),
                   bg_ms_per_launch(H, H.GEMM, bg_n, 2, 1, 24, 40)) for _ in range(5 if compact else 7)]
        mid = len(rounds) // 2
        ms_plain, ms_guard, ms_l2 = (sorted(r[i] for r in rounds)[mid] for i in range(3))
        guard_frac = sorted(1.0 - r[0] / r[1] for r in rounds)
        l2_frac = sorted(1.0 - r[0] / r[2] for r in rounds)

        def tf(ms):
            return gemm_flops(bg_n) / ms / 1e9
        line["guard"] = {"plain_TFLOPs": tf(ms_plain), "guarded_TFLOPs": tf(ms_guard), "level2_TFLOPs": tf(ms_l2),
                         "plain_mfma_util": tf(ms_plain) / MFMA_BF16_PEAK_TF,
                         "guarded_mfma_util": tf(ms_guard) / MFMA_BF16_PEAK_TF,
                         "guard_overhead_frac": guard_frac[mid], "level2_overhead_frac": l2_frac[mid],
                         "guard_overhead_frac_min_max": [guard_frac[0], guard_frac[-1]],
                         "level2_overhead_frac_min_max": [l2_frac[0], l2_frac[-1]],
                         "rounds": len(rounds), "launches_per_round_and_form": 24, "untimed_launches_before_each": 40}
        line["preempt_us"] = preempt_block(H, H.GEMM, bg_n, compact)
        line["vendor_library"] = vendor_gemm(bg_n, tf(ms_plain))
    return line


def vendor_gemm(n, ours_tflops):
    """The vendor library's bf16 GEMM of the same shape on the same box, for scale: hipBLASLt
    through torch.matmul, 40 launches after 40 untimed ones, median of five rounds. None when
    torch has no GPU."""
    try:
        import torch
        if not torch.cuda.is_available():
            return None
        a = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
        b = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
        for _ in range(40):
            c = a @ b
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        rounds = []
        for _ in range(5):
            e0.record()
            for _ in range(40):
                c = a @ b  # noqa: F841
            e1.record()
            torch.cuda.synchronize()
            rounds.append(e0.elapsed_time(e1) / 40)
        ms = sorted(rounds)[2]
        vendor = gemm_flops(n) / ms / 1e9
        return {"what": "hipBLASLt through torch.matmul, bf16 %d^3, same process" % n, "ms_per_launch": ms,
                "TFLOPs": vendor, "this_kernel_over_vendor": ours_tflops / vendor}
    except Exception as e:  # informational only
        return {"what": "unavailable: %s" % e}


def config4(H, a):
    compact = getattr(a, "compact", False)
    bg_n, fg_n, deadline = 1 << 26, 1 << 20, 1000
    laxities = [300] if (a.quick or compact) else [0, 300, 600, 900]
    runs = {}
    for lax in laxities:
        # Background queues run at constant priority 0. The foreground runs beside them at
        # priority 0 until `lax` us after it became ready, then at priority 1, which
        # deactivates the four background queues.
        cfg = H.Config(H.LAX, 4, H.spec(H.HIST, bg_n, 1, 2, BG_THRESHOLD, BG_BATCH, 0),
                       H.spec(H.HIST, fg_n, 0, 1, 8, 4, 1, laxity_us=lax, period_us=2000, lax_priority=0,
                              deadline_us=deadline), 16, 0)
        def after(b):
            """Every bin of the four background queues and of the foreground queue after the
            timed phases (repeated deactivations and replays): `applied` times the oracle's
            counts of that queue's keys."""
            out = {"bg%d" % q: check_hist_bins(b, 0, q, q + 1, bg_n) for q in range(4)}
            out["fg"] = check_hist_bins(b, 1, 0, 0, fg_n)
            return out
        runs[lax] = contended_run(H, cfg, a.steps, a.warmup, bg_warm=16, bg_cmds=60, keep=after if lax == 300 else None)
    head = runs[300]
    fg = fg_summary(H, head["fg_alone"], head["fg_contended"])
    # Roofline of the kernel itself: one queue streaming it back to back, Level 2, guarded.
    # Five alternating rounds of 120 commands, the median of each form: a single round moves
    # by a microsecond with where the buffers of that round happen to lie. 120 untimed
    # commands come first (the first ones allocate the queue's scratch buffers and clear
    # their progress maps: 61-63 us per command over the first 120, 55-57 afterwards).
    rounds = [(bg_ms_per_launch(H, H.HIST, bg_n, 2, 1, 120, 120),
               None if a.quick else bg_ms_per_launch(H, H.HIST, bg_n, 1, 0, 120, 120)) for _ in range(3 if compact else 5)]
    per_launch_ms = sorted(r[0] for r in rounds)[len(rounds) // 2]
    achieved = hist_bytes(bg_n) / (per_launch_ms * 1e-3) / 1e9
    line = base_line(a, fg["contended_p99"], head["wall_s"],
                     "cfg4: L2 LAX, 4 bg XQueues histogram 2^26 Zipf(1.1) keys, fg 2^20 keys every 2 ms, "
                     "deadline 1 ms, laxity hint 300 us",
                     {"bg_threshold": BG_THRESHOLD, "bg_batch": BG_BATCH, "fg_threshold": 8, "fg_batch": 4})
    line["dtype"] = "u32"
    line["fg_latency_us"] = fg
    line["bit_exact"] = dict(head["kept"], all_ok=all(v["ok"] for v in head["kept"].values()))
    line["deadline_miss_rate"] = head["deadline_miss"] / a.steps
    line["by_laxity_us"] = {
        str(lax): {"deadline_miss_rate": r["deadline_miss"] / a.steps,
                   "fg_p50": H.pct(r["fg_contended"], 0.5), "fg_p99": H.pct(r["fg_contended"], 0.99),
                   "bg_GBs": hist_bytes(bg_n) * r["bg_cont_cmds"] / r["bg_cont_elapsed"] / 1e9,
                   "bg_deactivations_q0": r["stats"][2]}
        for lax, r in runs.items()}
    # all four queues by the wall clock (commands finished / elapsed), as for the contended figure
    line["bg"] = {"alone_GBs_4_queues_side_by_side":
                      hist_bytes(bg_n) * head["bg_alone_cmds"] / head["bg_alone_elapsed"] / 1e9,
                  "contended_GBs": hist_bytes(bg_n) * head["bg_cont_cmds"] / head["bg_cont_elapsed"] / 1e9}
    line["bg"]["alone_frac_of_hbm_peak"] = line["bg"]["alone_GBs_4_queues_side_by_side"] / HBM_PEAK_GBS
    line["bg"]["contended_frac_of_hbm_peak"] = line["bg"]["contended_GBs"] / HBM_PEAK_GBS
    line["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": achieved / HBM_PEAK_GBS, "traffic": recorded_traffic("histogram_2p26_hbm_traffic.md"), "kernel": "HistogramKernel + HistogramMergeKernel",
                        "algorithmic_bytes_per_launch": hist_bytes(bg_n), "avg_launch_ms": per_launch_ms,
                        "note": "one queue streaming guarded histogram commands back to back; a command is the "
                                "counting kernel followed by the merge kernel, avg_launch_ms covers both"}
    if not a.quick:
        ms_plain = sorted(r[1] for r in rounds)[len(rounds) // 2]
        line["guard"] = {"plain_GBs": hist_bytes(bg_n) / ms_plain / 1e6, "level2_GBs": achieved,
                         # median of the per-round ratios (the two forms of a round run within a second)
                         "level2_overhead_frac": sorted(1.0 - r[1] / r[0] for r in rounds)[len(rounds) // 2],
                         "level2_overhead_frac_min_max": [min(1.0 - r[1] / r[0] for r in rounds),
                                                          max(1.0 - r[1] / r[0] for r in rounds)],
                         "rounds": len(rounds), "commands_per_round_and_form": 120}
        line["preempt_us"] = preempt_block(H, H.HIST, bg_n, True)
    return line


def config5(H, a):
    axpy_n, gemm_n, hist_n, nq = 1 << 24, 2048, 1 << 24, 16
    # seconds of arrivals, ~200 commands per queue and second
    duration = 2.0 if getattr(a, "compact", False) else max(min(a.steps / 100.0, 4.0), 1.0)
    cfg = H.StressConfig(H.HPF, nq, 2, 1, 4, 2, axpy_n, gemm_n, hist_n, 5000.0, 7)
    alone_s = 0.3 if getattr(a, "compact", False) else 0.5
    with H.Bench(cfg) as b:
        b.stress(0.2)  # warm-up
        # every queue by itself first, the other fifteen idle, with its own arrival process:
        # what its commands take with the device to themselves
        alone = [b.stress(alone_s, only=[i])[0][i] for i in range(nq)]
        t0 = time.perf_counter()
        lat, res = b.stress(duration)
        wall = time.perf_counter() - t0
        stats = list(res.stats)
        # every queue's buffer against the oracle, for as many commands as were applied to it
        exact = {}
        for i in range(nq):
            if i % 3 == 0:
                exact[str(i)] = check_axpy_buffer(b, 0, i, i + 1, axpy_n, seed=7)
            elif i % 3 == 1:
                exact[str(i)] = check_gemm_rows(b, 0, i, i + 1, gemm_n, [0, gemm_n // 2, gemm_n - 4], seed=7)
            else:
                exact[str(i)] = check_hist_bins(b, 0, i, i + 1, hist_n, seed=7)
    counts = [len(x) for x in lat]
    kinds = ["axpy", "gemm", "hist"]
    by_prio = {str(i): {"kernel": kinds[i % 3], "commands": counts[i], "p50": H.pct(lat[i], 0.5),
                        "p99": H.pct(lat[i], 0.99), "alone_commands": len(alone[i]), "alone_p50": H.pct(alone[i], 0.5),
                        "alone_p99": H.pct(alone[i], 0.99),
                        "p99_ratio": (H.pct(lat[i], 0.99) / H.pct(alone[i], 0.99)) if alone[i] else None}
               for i in range(nq)}
    hbm_bytes = sum(counts[i] * (axpy_bytes(axpy_n) if i % 3 == 0 else hist_bytes(hist_n) if i % 3 == 2 else 0)
                    for i in range(nq))
    flops = sum(counts[i] * gemm_flops(gemm_n) for i in range(nq) if i % 3 == 1)
    line = base_line(a, H.pct(lat[nq - 1], 0.99), wall,
                     "cfg5: 16 XQueues prio 0-15, AXPY 2^24 / GEMM 2048^3 / histogram 2^24 by queue index mod 3, "
                     "exponential arrivals mean 5 ms seed 7, HPF, L2; value = p99 of priority 15",
                     {"threshold": 4, "batch": 2, "arrival_seconds": duration})
    line["dtype"] = "mixed f32/bf16/u32"
    line["per_priority_latency_us"] = by_prio
    line["bit_exact"] = dict(exact, all_ok=all(v["ok"] for v in exact.values()),
                             note="axpy: slices of y, hist: all bins, bit for bit; gemm: rows within the stated tolerance of the oracle")
    line["aggregate"] = {"commands": sum(counts), "elapsed_s": res.elapsed_s,
                         "hbm_GBs": hbm_bytes / res.elapsed_s / 1e9,
                         "hbm_frac_of_peak": hbm_bytes / res.elapsed_s / 1e9 / HBM_PEAK_GBS,
                         "mfma_TFLOPs": flops / res.elapsed_s / 1e12,
                         "mfma_frac_of_peak": flops / res.elapsed_s / 1e12 / MFMA_BF16_PEAK_TF,
                         "queue0_stats": stats}
    line["roofline"] = {"bound": "hbm", "achieved": hbm_bytes / res.elapsed_s / 1e9, "peak": HBM_PEAK_GBS,
                        "unit": "GB/s", "frac": hbm_bytes / res.elapsed_s / 1e9 / HBM_PEAK_GBS, "traffic": None,
                        "note": "aggregate of an arrival-limited workload (offered load, not a kernel rate)"}
    return line


def shim_launch_cost():
    """us per launch of a tiny kernel by an unmodified HIP program (tests/shim_app.hip, built into
    xsched_amd/lib), natively and with the interception shim in front of the runtime (every
    launch an XQueue command). Informational; None when the programs have not been built."""
    import re
    import subprocess
    lib = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xsched_amd", "lib")
    out = {}
    for key, binary, extra in (("native", "shim_app_plain", {}),
                               ("through_shim", "shim_app", {"XSCHED_AUTO_XQUEUE": "ON", "XSCHED_SCHEDULER": "LCL",
                                                             "XSCHED_POLICY": "HPF", "XLOG_LEVEL": "WARN"})):
        path = os.path.join(lib, binary)
        if not os.path.exists(path):
            return None
        env = {k: v for k, v in os.environ.items() if not k.startswith("XSCHED_")}
        env.update(extra)
        try:
            proc = subprocess.run([path, "--bench", "20000"], env=env, capture_output=True, text=True, timeout=60)
        except subprocess.TimeoutExpired:
            return None
        m = re.search(r"submit_us_per_launch=([\d.]+) total_us_per_launch=([\d.]+)", proc.stdout)
        if proc.returncode != 0 or not m:
            return None
        out[key] = {"submit_us_per_launch": float(m.group(1)), "total_us_per_launch": float(m.group(2))}
    out["launches"] = 20000
    return out


def framework_loop_under_shim(alternations=3):
    """An unmodified PyTorch-ROCm training loop (tests/shim_torch_workload.py --time: about 26
    kernel launches and fills per step, launch-bound), natively and with the interception shim
    preloaded (every launch an XQueue command, level 1): microseconds per step. A process of
    this loop lands in one of two speed classes some 30 % apart whatever is in front of the
    runtime, so the two forms alternate and every run is reported. Informational; None when
    the shim has not been built or a run fails."""
    import re
    import statistics
    import subprocess
    root = os.path.dirname(os.path.abspath(__file__))
    shim = os.path.join(root, "xsched_amd", "lib", "libshimhip.so")
    script = os.path.join(root, "tests", "shim_torch_workload.py")
    if not os.path.exists(shim):
        return None
    base = {k: v for k, v in os.environ.items() if not k.startswith("XSCHED_")}
    preload = " ".join(x for x in (os.environ.get("LD_PRELOAD", ""), shim) if x)
    forms = (("native", {}),
             ("under_shim_level1", {"LD_PRELOAD": preload, "XSCHED_AUTO_XQUEUE": "ON", "XSCHED_AUTO_XQUEUE_LEVEL": "1",
                                    "XSCHED_SCHEDULER": "LCL", "XSCHED_POLICY": "HPF", "XLOG_LEVEL": "WARN"}))
    runs = {key: [] for key, _ in forms}
    for _ in range(alternations):
        for key, extra in forms:
            try:
                proc = subprocess.run([sys.executable, script, "--time"], env=dict(base, **extra), capture_output=True,
                                      text=True, timeout=120)
            except subprocess.TimeoutExpired:
                return None
            m = re.search(r"us_per_step=([\d.]+)", proc.stdout)
            if proc.returncode != 0 or not m:
                return None
            runs[key].append(float(m.group(1)))
    native, under = statistics.median(runs["native"]), statistics.median(runs["under_shim_level1"])
    return {"workload": "3-layer MLP, batch 1024, SGD with momentum, 200-step rounds on a side stream, median of 5 rounds per run",
            "native_us_per_step": runs["native"], "under_shim_level1_us_per_step": runs["under_shim_level1"],
            "median_native": native, "median_under_shim": under, "shim_over_native": round(under / native, 3)}


def transparent_preemption():
    """Two plain HIP processes (tests/shim_app.hip), one filling the device with 5 ms kernels that
    have the guard compiled in (priority 0), one launching a short kernel every 2 ms (priority 1):
    the short kernel's launch-to-completion latency alone, next to the load under hardware
    scheduling, and with both processes under the interception shim, the scheduler daemon (HPF)
    and level 2. Informational; None when something it needs has not been built or a run fails."""
    import re
    import shutil
    import subprocess
    import tempfile
    lib = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xsched_amd", "lib")
    need = [os.path.join(lib, n) for n in ("shim_app", "shim_app_plain", "xserver")]
    if not all(os.path.exists(n) for n in need):
        return None
    base = {k: v for k, v in os.environ.items() if not k.startswith("XSCHED_")}
    probe_args = ["--probe", "300", "2000"]

    def percentiles(out):
        m = re.search(r"probe n=(\d+) p50_us=([\d.]+) p99_us=([\d.]+)", out)
        return {"p50": float(m.group(2)), "p99": float(m.group(3))} if m else None

    def next_to(binary, load_env, probe_env):
        load = subprocess.Popen([os.path.join(lib, binary), "--load-guarded", "1.6"], env=dict(base, **load_env),
                                stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        try:
            if load.stdout.readline().strip() != "ready":
                return None
            probe = subprocess.run([os.path.join(lib, binary)] + probe_args, env=dict(base, **probe_env),
                                   capture_output=True, text=True, timeout=60)
            load_out, load_err = load.communicate(timeout=60)
        finally:
            if load.poll() is None:
                load.kill()
            load.wait()          # reaped: no zombie is left behind for the rest of the run
        if probe.returncode != 0 or load.returncode != 0:
            return None
        m = re.search(r"ms_per_kernel=([\d.]+) work_groups_not_exactly_once=(\d+)", load_out)
        stats = dict(item.split("=") for item in re.search(r"\[xsched shim\] (.*)", load_err).group(1).split()) \
            if "[xsched shim]" in load_err else {}
        return {"fg": percentiles(probe.stdout), "load_ms_per_kernel": float(m.group(1)) if m else None,
                "load_work_groups_not_exactly_once": int(m.group(2)) if m else None,
                "load_queue_deactivations": int(stats["deactivations"]) if stats else None,
                "load_replayed_launches": int(stats["replays"]) if stats else None}

    try:
        alone = subprocess.run([os.path.join(lib, "shim_app_plain")] + probe_args, env=base, capture_output=True,
                               text=True, timeout=60)
        native = next_to("shim_app_plain", {}, {})
        def under_daemon(extra):
            """Both processes under shim + daemon + level 2; `extra` goes into all three environments."""
            sock_dir = tempfile.mkdtemp(prefix="xsched-bench-")
            server = subprocess.Popen([os.path.join(lib, "xserver"), "HPF"],
                                      env=dict(base, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="WARN", **extra))
            started = time.time()
            try:
                deadline = time.time() + 5
                while not os.path.exists(os.path.join(sock_dir, "xsched-1.sock")) and time.time() < deadline:
                    time.sleep(0.01)
                common = dict({"XSCHED_SOCKET_DIR": sock_dir, "XSCHED_SCHEDULER": "GLB", "XSCHED_AUTO_XQUEUE": "ON",
                               "XSCHED_AUTO_XQUEUE_LEVEL": "2", "XSCHED_SHIM_STATS": "1", "XLOG_LEVEL": "WARN"}, **extra)
                out = next_to("shim_app", dict(common, XSCHED_AUTO_XQUEUE_PRIORITY="0", XSCHED_AUTO_XQUEUE_THRESHOLD="2",
                                               XSCHED_AUTO_XQUEUE_BATCH_SIZE="1"),
                              dict(common, XSCHED_AUTO_XQUEUE_PRIORITY="1"))
                if out is not None:
                    try:   # what the daemon's threads cost while the two clients ran
                        import psutil
                        t = psutil.Process(server.pid).cpu_times()
                        out["daemon_cpu_cores"] = round((t.user + t.system) / (time.time() - started), 3)
                    except Exception:
                        out["daemon_cpu_cores"] = None
                return out
            finally:
                server.terminate()
                try:
                    server.wait(timeout=5)
                except subprocess.TimeoutExpired:
                    server.kill()
                    server.wait()
                shutil.rmtree(sock_dir, ignore_errors=True)

        # Default: receivers poll briefly after each message and are up ahead of a periodic
        # sender's next burst (csrc/sched/spin.h). Beside it: receivers that only block, and
        # receivers that poll for 5 ms after each message, i.e. all the time here.
        under = under_daemon({})
        under_blocking = under_daemon({"XSCHED_WAKE_AHEAD": "OFF"})
        under_polling = under_daemon({"XSCHED_SPIN_US": "5000"})
    except (OSError, subprocess.SubprocessError, AttributeError):
        return None
    if native is None or under is None or alone.returncode != 0:
        return None
    return {"workload": "fg: 256x256-thread kernel every 2 ms, 300 samples; load: 2048x256-thread guarded kernels of "
                        "5 ms back to back; two processes, plain HIP host code, percentile = sorted[floor(p*n)]",
            "fg_alone_us": percentiles(alone.stdout), "hardware_scheduling_only": native,
            "under_xsched_shim_daemon_level2": under,
            "p99_over_alone": (round(under["fg"]["p99"] / percentiles(alone.stdout)["p99"], 3)
                               if under.get("fg") and percentiles(alone.stdout) else None),
            "under_xsched_shim_daemon_level2_XSCHED_WAKE_AHEAD_OFF": under_blocking,
            "under_xsched_shim_daemon_level2_XSCHED_SPIN_US_5000": under_polling}


def compact_of(line):
    """The figures of a configuration's full line that the default line carries."""
    keep = {"workload": line["config"]["workload"], "fg_p99_contended_us": line["value"],
            "fg_latency_us": {k: v for k, v in line.get("fg_latency_us", {}).items()
                              if k in ("alone_p50", "alone_p99", "contended_p50", "contended_p99", "p99_ratio", "samples")},
            "fg_samples": line["steps"]}
    roof = line.get("roofline", {})
    keep["roofline"] = {k: roof.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "avg_launch_ms", "traffic")}
    if "guard" in line:
        keep["guard"] = {k: v for k, v in line["guard"].items() if k.endswith("overhead_frac") or k.endswith("_min_max")}
    if "preempt_us" in line:
        keep["preempt_us"] = {k: v for k, v in line["preempt_us"].items()
                              if k.startswith("level2_device_drain") or k.startswith("level2_resume") or k.startswith("level2_suspend")}
    for k in ("deadline_miss_rate", "bit_exact", "vendor_library"):
        if k in line:
            keep[k] = line[k]
    if isinstance(line.get("bg"), dict) and "contended_frac_of_hbm_peak" in line["bg"]:
        keep["bg_all_queues_frac_of_hbm_peak"] = {"alone": line["bg"]["alone_frac_of_hbm_peak"],
                                                  "contended": line["bg"]["contended_frac_of_hbm_peak"]}
    if isinstance(keep.get("bit_exact"), dict) and "all_ok" in keep["bit_exact"]:
        keep["bit_exact"] = keep["bit_exact"]["all_ok"]
    if "per_priority_latency_us" in line:
        keep["p99_by_priority_us"] = {k: v["p99"] for k, v in line["per_priority_latency_us"].items()}
        keep["p99_ratio_by_priority"] = {k: (round(v["p99_ratio"], 2) if v["p99_ratio"] else None)
                                         for k, v in line["per_priority_latency_us"].items()}
        keep["aggregate"] = {k: line["aggregate"][k] for k in ("commands", "hbm_frac_of_peak", "mfma_frac_of_peak")}
    return keep


def other_configurations(H, a):
    """Compact blocks of configurations 1, 3, 4 and 5 for the default line (about 45 s in all:
    200 foreground samples each, fewer overhead rounds than their own full lines)."""
    sub = argparse.Namespace(steps=200, warmup=10, quick=False, compact=True, bg_log2=28, fg_log2=22)
    out = {}
    for name, run in (("cfg1", lambda: config1(argparse.Namespace(quick=True))), ("cfg3", lambda: config3(H, sub)),
                      ("cfg4", lambda: config4(H, sub)), ("cfg5", lambda: config5(H, sub))):
        t0 = time.perf_counter()
        try:
            out[name] = compact_of(run())
        except Exception as e:  # one configuration failing must not take the headline line with it
            out[name] = {"error": repr(e)}
        out[name]["seconds"] = round(time.perf_counter() - t0, 1)
        if name != "cfg1" and not a.skip_cpu:
            # the same configuration on host cores (reduced sizes, stated in `sample`), on XSched's own host loop
            base = cpu_baseline(int(name[3:]), compact=True)
            out[name]["cpu_baseline"] = {k: base.get(k) for k in ("value", "unit", "cores", "kind", "sample", "bit_exact",
                                                                  "fg_alone_p99_us", "deadline_miss_rate", "p99_by_priority_us")
                                         if base.get(k) is not None}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--bg-log2", type=int, default=28)
    ap.add_argument("--fg-log2", type=int, default=22)
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--quick", action="store_true", help="headline phases only")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: XQueues are per-device and this path has no "
              "cross-GPU exchange; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if a.steps < 1:
        print("--steps must be at least 1", file=sys.stderr)
        sys.exit(2)

    if a.config == 1:
        line = config1(a)
        line["cpu_baseline"] = ({"value": None, "unit": "us", "cores": 0, "kind": "reference", "sample": "skipped"}
                                if a.skip_cpu else cpu_baseline(1))
        print(json.dumps(line))
        return

    # The package first: like the adapter library it asks the HIP runtime for a larger pool of
    # completion signals (ROC_SIGNAL_POOL_SIZE, unless set), which the runtime reads when it
    # starts, i.e. at the first HIP call of the process - torch's device check below.
    import xsched_amd  # noqa: F401
    import torch  # device presence check only; the harness allocates through HIP itself
    if not torch.cuda.is_available():
        print("no GPU visible: bench.py needs an MI355X", file=sys.stderr)
        sys.exit(1)
    from xsched_amd import harness as H

    line = {2: config2, 3: config3, 4: config4, 5: config5}[a.config](H, a)
    if isinstance(line.get("config"), dict):
        line["config"]["runtime_env"] = {"ROC_SIGNAL_POOL_SIZE": os.environ.get("ROC_SIGNAL_POOL_SIZE"),
                                         "XSCHED_HIP_MARKER_ON_KERNEL": os.environ.get("XSCHED_HIP_MARKER_ON_KERNEL", "ON (default)")}
    if a.config == 2 and not a.quick:
        line["others"] = other_configurations(H, a)
        line["shim_launch_cost"] = shim_launch_cost()
        line["framework_loop_under_shim"] = framework_loop_under_shim()
        line["transparent_preemption"] = transparent_preemption()
    if not a.skip_cpu:
        line["cpu_baseline"] = cpu_baseline(a.config)
    else:
        line["cpu_baseline"] = {"value": None, "unit": "us", "cores": 0, "kind": "reference", "sample": "skipped"}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
