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


if __name__ == "__main__":
    import json
    import sys
    print(json.dumps(run_config2_sample(which=sys.argv[1] if len(sys.argv) > 1 else "auto")))
