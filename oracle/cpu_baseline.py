"""ORACLE - test infrastructure only: runs the headline workload on CPU cores, on a
bounded sample, and reports it in bench.py's `cpu_baseline` format. Preferred: the
reference's own XQueue core, scheduler and policy (oracle/_ref/libxqueue_ref.so, kind
"reference") driving scalar CPU kernels through oracle/host_bench.cpp. Without that build
there is no CPU baseline: the call raises."""
import ctypes
import os
from ctypes import POINTER, byref, c_double, c_int, c_int64, c_uint64

_DIR = os.path.dirname(os.path.abspath(__file__))


def host_cpu():
    """(model name, logical cores of the machine, cores this process may run on)."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 0
    return model, os.cpu_count() or 0, usable


def _pct(samples, p):
    s = sorted(samples)
    return s[min(int(p * len(s)), len(s) - 1)]


def run_config2_sample(seconds_budget=15.0, scale_log2=4, samples=100, which="auto"):
    """Same structure as the GPU run (bg AXPY back to back at priority 1, fg AXPY every
    20 ms at priority 2, level 1, HPF), with both arrays scaled down by 2^scale_log2 so
    that the sample takes on the order of ten seconds of CPU work."""
    ref_path = os.path.join(_DIR, "_ref", "libxqueue_ref.so")
    if which == "auto":
        which = "reference"
    if which == "reference":
        if not os.path.exists(ref_path):
            raise RuntimeError(f"{ref_path} missing: it is built from the reference sources by "
                               "`make -C oracle ref` where that tree is present")
        os.environ.setdefault("XLOG_LEVEL", "ERRO")
        fn = ctypes.CDLL(ref_path, mode=ctypes.RTLD_LOCAL).hostbench_run_fg_bg_axpy
    elif which == "shipped":
        fn = ctypes.CDLL(os.path.join(_DIR, "libhostbench.so"), mode=ctypes.RTLD_LOCAL).hostbench_run_fg_bg_axpy
    else:
        raise ValueError("which must be auto, reference or shipped")
    fn.restype = c_int
    fn.argtypes = [c_uint64, c_uint64, c_int64, c_int, c_int, c_int, POINTER(c_double), POINTER(c_double),
                   POINTER(c_uint64), POINTER(c_double), POINTER(c_uint64)]
    bg_n, fg_n = (1 << 28) >> scale_log2, (1 << 22) >> scale_log2
    alone = (c_double * samples)()
    cont = (c_double * samples)()
    bg_cmds, secs, chk = c_uint64(), c_double(), c_uint64()
    rc = fn(bg_n, fg_n, 20000, samples, 4, 2, alone, cont, byref(bg_cmds), byref(secs), byref(chk))
    if rc != 0:
        raise RuntimeError(f"CPU baseline run failed with XResult {rc}")
    alone, cont = list(alone)[5:], list(cont)[5:]
    bg_gbs = 12.0 * bg_n * bg_cmds.value / secs.value / 1e9 if secs.value else 0.0
    return {
        "value": _pct(cont, 0.99),
        "unit": "us",
        "cores": 7,
        "host_cpu_model": host_cpu()[0], "host_logical_cores": host_cpu()[1], "host_usable_cores": host_cpu()[2],
        "kind": "reference" if which == "reference" else "shipped-host",
        "sample": ("%s (2 XQueues, level 1, HPF, bg window 4/2, fg 8/4), scalar single-threaded fmaf AXPY per "
                   "queue; bg 2^%d and fg 2^%d elements (1/%d of the GPU sizes), fg every 20 ms, %d fg samples; "
                   "threads: 2 executors + 2 launch workers + 1 scheduler + 2 submitters"
                   % ({"reference": "oracle/_ref/libxqueue_ref.so: XSched's own XQueue core, local scheduler and "
                                    "HPF policy compiled from the reference sources, driving this repository's "
                                    "host adapter through oracle/host_bench.cpp",
                       "shipped-host": "shipped libpreempt.so + libhalhost.so through oracle/host_bench.cpp"}
                      ["reference" if which == "reference" else "shipped-host"],
                      28 - scale_log2, 22 - scale_log2, 1 << scale_log2, len(cont))),
        "fg_alone_p50_us": _pct(alone, 0.5), "fg_alone_p99_us": _pct(alone, 0.99),
        "fg_contended_p50_us": _pct(cont, 0.5), "fg_contended_p99_us": _pct(cont, 0.99),
        "bg_GBs": bg_gbs,
    }


def run_config1_sample(samples=150, which="reference"):
    """The CPU-only configuration at its full size on the reference's own host loop: background
    streams of 1000 fp32 vector additions over 2^20 elements, a 2^16-element addition every
    10 ms in the foreground, window 8 / 4, level 1, HPF."""
    ref_path = os.path.join(_DIR, "_ref", "libxqueue_ref.so")
    path = ref_path if which == "reference" else os.path.join(_DIR, "libhostbench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} missing")
    os.environ.setdefault("XLOG_LEVEL", "ERRO")
    fn = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL).hostbench_run_fg_bg_vecadd
    fn.restype = c_int
    fn.argtypes = [c_uint64, c_uint64, c_int64, c_int, c_int, c_int, c_int, POINTER(c_double), POINTER(c_double),
                   POINTER(c_uint64), POINTER(c_double), POINTER(c_uint64)]
    alone, cont = (c_double * samples)(), (c_double * samples)()
    bg_cmds, secs, chk = c_uint64(), c_double(), c_uint64()
    rc = fn(1 << 20, 1 << 16, 10000, samples, 8, 4, 1000, alone, cont, byref(bg_cmds), byref(secs), byref(chk))
    if rc != 0:
        raise RuntimeError(f"CPU baseline run failed with XResult {rc}")
    alone, cont = list(alone)[5:], list(cont)[5:]
    model, logical, usable = host_cpu()
    return {
        "value": _pct(cont, 0.99), "unit": "us", "cores": 7,
        "host_cpu_model": model, "host_logical_cores": logical, "host_usable_cores": usable,
        "kind": "reference" if which == "reference" else "shipped-host",
        "sample": ("XSched's own XQueue core, local scheduler and HPF policy (oracle/_ref/libxqueue_ref.so) over this "
                   "repository's host adapter: bg fp32 vector additions 2^20 in streams of 1000, fg 2^16 every 10 ms, "
                   "window 8/4, %d fg samples; scalar single-threaded kernels; threads: 2 executors + 2 launch workers "
                   "+ 1 scheduler + 2 submitters" % len(cont)),
        "fg_alone_p50_us": _pct(alone, 0.5), "fg_alone_p99_us": _pct(alone, 0.99),
        "fg_contended_p50_us": _pct(cont, 0.5), "fg_contended_p99_us": _pct(cont, 0.99),
        "bg_GBs": 12.0 * (1 << 20) * bg_cmds.value / secs.value / 1e9 if secs.value else 0.0,
        "fg_checksum": chk.value,
    }


def _host_lib(which):
    ref_path = os.path.join(_DIR, "_ref", "libxqueue_ref.so")
    path = ref_path if which == "reference" else os.path.join(_DIR, "libhostbench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} missing (reference build: `make -C oracle ref` where that tree is present)")
    os.environ.setdefault("XLOG_LEVEL", "ERRO")
    return ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)


_CORE = {"reference": "XSched's own XQueue core, local scheduler and policies compiled from the reference sources "
                      "(oracle/_ref/libxqueue_ref.so)",
         "shipped": "the shipped libpreempt.so"}


def _fg_bg_kernel(which, kind, bg_n, fg_n, n_bg, level, policy, laxity_us, period_us, deadline_us, samples):
    fn = _host_lib(which).hostbench_run_fg_bg_kernel
    fn.restype = c_int
    fn.argtypes = [c_int, c_uint64, c_uint64, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_int,
                   POINTER(c_double), POINTER(c_double), POINTER(c_uint64), POINTER(c_double), POINTER(c_uint64),
                   POINTER(c_int)]
    alone, cont = (c_double * samples)(), (c_double * samples)()
    cmds, secs, misses, exact = c_uint64(), c_double(), c_uint64(), c_int()
    rc = fn(kind, bg_n, fg_n, n_bg, level, policy, laxity_us, period_us, deadline_us, samples, alone, cont,
            byref(cmds), byref(secs), byref(misses), byref(exact))
    if rc != 0:
        raise RuntimeError(f"CPU baseline run failed with XResult {rc}")
    model, logical, usable = host_cpu()
    alone, cont = list(alone)[5:], list(cont)[5:]
    return {"value": _pct(cont, 0.99), "unit": "us", "cores": 2 * (n_bg + 1) + 1 + n_bg + 1,
            "host_cpu_model": model, "host_logical_cores": logical, "host_usable_cores": usable,
            "kind": "reference" if which == "reference" else "shipped-host",
            "fg_alone_p50_us": _pct(alone, 0.5), "fg_alone_p99_us": _pct(alone, 0.99),
            "fg_contended_p50_us": _pct(cont, 0.5), "fg_contended_p99_us": _pct(cont, 0.99),
            "bit_exact": bool(exact.value), "bg_commands": cmds.value, "contended_seconds": secs.value,
            "deadline_misses": misses.value, "fg_samples": samples}


def run_config3_sample(samples=150, which="reference", bg_edge=256, fg_edge=32):
    """Level 2, HPF: a background queue of guarded bf16 GEMMs (fp32 accumulation, one fmaf per
    product in ascending k: the oracle's arithmetic) back to back, a foreground GEMM every
    5 ms, both edges 1/32 of the GPU's (8192 -> 256, 1024 -> 32: a scalar core does about one
    GFLOP/s on this dependent chain)."""
    r = _fg_bg_kernel(which, 1, bg_edge, fg_edge, 1, 2, 1, -1, 5000, 0, samples)
    r["bg_GFLOPs"] = 2.0 * bg_edge ** 3 * r["bg_commands"] / r["contended_seconds"] / 1e9 if r["contended_seconds"] else 0.0
    r["sample"] = ("%s over this repository's host adapter at level 2 (flush and replay between work-groups of 8 rows), "
                   "HPF: bg bf16 GEMM %d^3 back to back (window 2/1), fg GEMM %d^3 every 5 ms (window 8/4), %d fg "
                   "samples; scalar single-threaded kernels; threads: 2 executors + 2 launch workers + 1 scheduler + 2 "
                   "submitters" % (_CORE["reference" if which == "reference" else "shipped"], bg_edge, fg_edge, samples - 5))
    return r


def run_config4_sample(samples=300, which="reference", scale_log2=4, laxity_us=300):
    """Level 2, LAX: four background queues of guarded histograms (2^16 bins, Zipf(1.1) keys)
    back to back, a foreground histogram every 2 ms with a laxity hint and a 1 ms deadline; key
    counts scaled down by 2^scale_log2."""
    bg_n, fg_n = (1 << 26) >> scale_log2, (1 << 20) >> scale_log2
    r = _fg_bg_kernel(which, 2, bg_n, fg_n, 4, 2, 8, laxity_us, 2000, 1000, samples)
    r["deadline_miss_rate"] = r["deadline_misses"] / samples
    r["bg_GBs"] = 4.0 * bg_n * r["bg_commands"] / r["contended_seconds"] / 1e9 if r["contended_seconds"] else 0.0
    r["sample"] = ("%s over this repository's host adapter at level 2, LAX (laxity hint %d us, deadline 1 ms): 4 bg "
                   "queues histogram 2^%d keys each back to back, fg 2^%d keys every 2 ms (1/%d of the GPU sizes), %d "
                   "fg samples; one atomic add per key, single-threaded per queue; threads: 5 executors + 5 launch "
                   "workers + 1 scheduler + 5 submitters"
                   % (_CORE["reference" if which == "reference" else "shipped"], laxity_us, 26 - scale_log2,
                      20 - scale_log2, 1 << scale_log2, samples - 5))
    return r


def run_config5_sample(duration_s=2.0, which="reference", axpy_log2=16, gemm_edge=32, hist_log2=15, nq=16):
    """Level 2, HPF, 16 queues with priorities 0-15 and exponential arrivals (mean 5 ms, seed
    7), kernels by queue index mod 3 at sizes a scalar core finishes in a fraction of the
    arrival interval."""
    fn = _host_lib(which).hostbench_run_stress
    fn.restype = c_int
    cap = 4096
    fn.argtypes = [c_int, c_int, c_uint64, c_uint64, c_uint64, c_double, c_uint64, c_double, POINTER(c_double),
                   c_uint64, POINTER(c_uint64), POINTER(c_double), POINTER(c_int)]
    lat, counts, secs, exact = (c_double * (nq * cap))(), (c_uint64 * nq)(), c_double(), c_int()
    rc = fn(nq, 2, 1 << axpy_log2, gemm_edge, 1 << hist_log2, 5000.0, 7, duration_s, lat, cap, counts, byref(secs),
            byref(exact))
    if rc != 0:
        raise RuntimeError(f"CPU baseline run failed with XResult {rc}")
    rows = [list(lat[i * cap:i * cap + counts[i]]) for i in range(nq)]
    model, logical, usable = host_cpu()
    return {"value": _pct(rows[nq - 1], 0.99), "unit": "us", "cores": 3 * nq + 1,
            "host_cpu_model": model, "host_logical_cores": logical, "host_usable_cores": usable,
            "kind": "reference" if which == "reference" else "shipped-host", "bit_exact": bool(exact.value),
            "p99_by_priority_us": {str(i): _pct(rows[i], 0.99) for i in range(nq) if rows[i]},
            "p50_by_priority_us": {str(i): _pct(rows[i], 0.5) for i in range(nq) if rows[i]},
            "commands": int(sum(counts)), "elapsed_s": secs.value,
            "sample": ("%s over this repository's host adapter at level 2, HPF: 16 queues prio 0-15, AXPY 2^%d / bf16 "
                       "GEMM %d^3 / histogram 2^%d by queue index mod 3, exponential arrivals mean 5 ms seed 7 for %.1f "
                       "s; scalar single-threaded kernels; threads: 16 executors + 16 launch workers + 1 scheduler + "
                       "16 submitters; value = p99 of priority 15"
                       % (_CORE["reference" if which == "reference" else "shipped"], axpy_log2, gemm_edge, hist_log2,
                          duration_s))}


if __name__ == "__main__":
    import json
    import sys
    print(json.dumps(run_config2_sample(which=sys.argv[1] if len(sys.argv) > 1 else "auto")))
