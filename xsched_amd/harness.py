"""ctypes mirror of the contention-benchmark harness in libhalhip.so
(include/xsched/hip/bench.h). Nothing is computed here: every phase runs inside the native
library so that no Python call sits on a timed path."""
import ctypes
from ctypes import POINTER, Structure, byref, c_double, c_int, c_int32, c_int64, c_uint64, c_void_p

import xsched_amd

AXPY, GEMM, HIST = 0, 1, 2
HPF, LAX = xsched_amd.kPolicyHighestPriorityFirst, xsched_amd.kPolicyLaxity


class QueueSpec(Structure):
    _fields_ = [("kind", c_int32), ("guard", c_int32), ("n", c_uint64), ("level", c_int32),
                ("threshold", c_int32), ("batch", c_int32), ("priority", c_int32),
                ("laxity_us", c_int64), ("period_us", c_int64), ("lax_priority", c_int32),
                ("reserved", c_int32), ("deadline_us", c_int64)]


class Config(Structure):
    _fields_ = [("policy", c_int32), ("n_bg", c_int32), ("bg", QueueSpec), ("fg", QueueSpec),
                ("bg_burst", c_int32), ("seed", c_uint64)]


class PhaseResult(Structure):
    _fields_ = [("elapsed_s", c_double), ("bg_commands", c_uint64), ("bg_stream_ms", c_double),
                ("bg_stream_cmds", c_uint64), ("fg_samples", c_uint64), ("fg_deadline_miss", c_uint64),
                ("stats", c_uint64 * 8)]


class StressConfig(Structure):
    _fields_ = [("policy", c_int32), ("n_queues", c_int32), ("level", c_int32), ("guard", c_int32),
                ("threshold", c_int32), ("batch", c_int32), ("axpy_n", c_uint64), ("gemm_n", c_uint64),
                ("hist_n", c_uint64), ("mean_interarrival_us", c_double), ("seed", c_uint64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        h = xsched_amd.halhip()
        h.XBenchCreate.restype = c_void_p
        h.XBenchCreate.argtypes = [POINTER(Config)]
        h.XBenchCreateStress.restype = c_void_p
        h.XBenchCreateStress.argtypes = [POINTER(StressConfig)]
        h.XBenchDestroy.argtypes = [c_void_p]
        h.XBenchRunForegroundAlone.argtypes = [c_void_p, c_int, POINTER(c_double), POINTER(PhaseResult)]
        h.XBenchRunBackgroundAlone.argtypes = [c_void_p, c_int, POINTER(PhaseResult)]
        h.XBenchRunContended.argtypes = [c_void_p, c_int, POINTER(c_double), POINTER(PhaseResult)]
        h.XBenchRunForegroundBreakdown.argtypes = [c_void_p, c_int, c_int, c_int, POINTER(c_double),
                                                   POINTER(PhaseResult)]
        h.XBenchRunPreempt.argtypes = [c_void_p, c_int, POINTER(c_double), POINTER(c_double),
                                       POINTER(PhaseResult)]
        h.XBenchRunPreemptDeviceTimed.argtypes = [c_void_p, c_int, POINTER(c_double), POINTER(PhaseResult)]
        h.XBenchRunStress.argtypes = [c_void_p, c_double, POINTER(c_double), c_uint64, POINTER(c_uint64),
                                      POINTER(PhaseResult)]
        h.XBenchRunStressQueues.argtypes = [c_void_p, c_double, c_uint64, POINTER(c_double), c_uint64,
                                            POINTER(c_uint64), POINTER(PhaseResult)]
        h.XBenchReadOutput.argtypes = [c_void_p, c_int, c_int, c_uint64, c_uint64, c_void_p,
                                       POINTER(c_uint64)]
        _lib = h
    return _lib


def spec(kind, n, guard, level, threshold, batch, priority, laxity_us=-1, period_us=0,
         lax_priority=xsched_amd.PRIORITY_MIN, deadline_us=0):
    return QueueSpec(kind, guard, n, level, threshold, batch, priority, laxity_us, period_us,
                     lax_priority, 0, deadline_us)


def pct(samples, p):
    """XSched's percentile rule: sorted[floor(p*n)] (reference utils/data.h:57-65)."""
    s = sorted(samples)
    return s[min(int(p * len(s)), len(s) - 1)] if s else 0.0


class Bench:
    """One harness instance (context manager)."""

    def __init__(self, cfg):
        self.cfg = cfg
        create = lib().XBenchCreateStress if isinstance(cfg, StressConfig) else lib().XBenchCreate
        self.h = create(byref(cfg))
        if not self.h:
            raise RuntimeError("harness refused the configuration")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        lib().XBenchDestroy(self.h)
        self.h = None

    def fg_alone(self, samples):
        lat, res = (c_double * samples)(), PhaseResult()
        xsched_amd.check(lib().XBenchRunForegroundAlone(self.h, samples, lat, byref(res)))
        return list(lat), res

    def bg_alone(self, commands):
        res = PhaseResult()
        xsched_amd.check(lib().XBenchRunBackgroundAlone(self.h, commands, byref(res)))
        return res

    def contended(self, samples):
        lat, res = (c_double * samples)(), PhaseResult()
        xsched_amd.check(lib().XBenchRunContended(self.h, samples, lat, byref(res)))
        return list(lat), res

    def fg_breakdown(self, samples, mode, contended):
        """Columns submit / device / wait / total (lists, microseconds); see bench.h."""
        out, res = (c_double * (samples * 4))(), PhaseResult()
        xsched_amd.check(lib().XBenchRunForegroundBreakdown(self.h, samples, mode, 1 if contended else 0, out, byref(res)))
        return {name: [out[i * 4 + k] for i in range(samples)]
                for k, name in enumerate(("submit", "device", "wait", "total"))}

    def preempt(self, samples):
        sus, resume, res = (c_double * samples)(), (c_double * samples)(), PhaseResult()
        xsched_amd.check(lib().XBenchRunPreempt(self.h, samples, sus, resume, byref(res)))
        return list(sus), list(resume), res

    def preempt_device_timed(self, samples):
        drain, res = (c_double * samples)(), PhaseResult()
        xsched_amd.check(lib().XBenchRunPreemptDeviceTimed(self.h, samples, drain, byref(res)))
        return list(drain), res

    def stress(self, duration_s, cap=4096, only=None):
        """Per-queue latency lists of a stress run; `only` = the queues that take arrivals
        (all of them when None)."""
        nq = self.cfg.n_queues
        mask = (1 << nq) - 1 if only is None else sum(1 << i for i in only)
        lat, counts, res = (c_double * (nq * cap))(), (c_uint64 * nq)(), PhaseResult()
        xsched_amd.check(lib().XBenchRunStressQueues(self.h, duration_s, mask, lat, cap, counts, byref(res)))
        return [list(lat[i * cap:i * cap + counts[i]]) for i in range(nq)], res

    def read(self, which, q, first, count, np_dtype):
        """(array, commands applied so far) of one output buffer slice."""
        import numpy as np
        out = np.empty(count, np_dtype)
        applied = c_uint64()
        xsched_amd.check(lib().XBenchReadOutput(self.h, which, q, first, count,
                                                out.ctypes.data_as(c_void_p), byref(applied)))
        return out, applied.value
