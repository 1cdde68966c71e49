"""The reference's Python interface over this repository's libraries: the same names, the
same argument order and the same return convention as `python/xsched/__init__.py` of XSched
(`XSched.XQueueCreate(hwq, level, flags) -> (XResult, handle)`, reference lines 232-348; enum
classes lines 14-112), so a script written against `from xsched import XSched, XPreemptLevel`
runs with `from xsched_amd.xsched_api import XSched, XPreemptLevel`.

Additions for this backend: `XSched.HipQueueCreate(stream)` and the guarded-command
constructors, which the reference leaves to each platform's own module."""
import ctypes
from enum import IntEnum
from typing import Tuple

import xsched_amd as _xs


def _enum(name, pairs):
    return IntEnum(name, pairs)


XResult = _enum("XResult", [("kXSchedSuccess", 0), ("kXSchedErrorHardware", 1), ("kXSchedErrorInvalidValue", 2),
                            ("kXSchedErrorNotFound", 3), ("kXSchedErrorNotAllowed", 4),
                            ("kXSchedErrorNotSupported", 5), ("kXSchedErrorBadResponse", 6),
                            ("kXSchedErrorUnknown", 999)])
XPlatform = _enum("XPlatform", [("kPlatformUnknown", 0), ("kPlatformVPI", 1), ("kPlatformCUDA", 2),
                                ("kPlatformCUDLA", 3), ("kPlatformHIP", 4), ("kPlatformAscend", 5),
                                ("kPlatformOpenCL", 6), ("kPlatformLevelZero", 7)])
XDeviceType = _enum("XDeviceType", [("kDeviceTypeUnknown", 0), ("kDeviceTypeCPU", 1), ("kDeviceTypeGPU", 2),
                                    ("kDeviceTypeNPU", 3), ("kDeviceTypeFPGA", 4), ("kDeviceTypeASIC", 5),
                                    ("kDeviceTypeMCA", 6)])
XPreemptLevel = _enum("XPreemptLevel", [("kPreemptLevelUnknown", 0), ("kPreemptLevelBlock", 1),
                                        ("kPreemptLevelDeactivate", 2), ("kPreemptLevelInterrupt", 3),
                                        ("kPreemptLevelMax", 4)])
XQueueState = _enum("XQueueState", [("kQueueStateUnknown", 0), ("kQueueStateIdle", 1), ("kQueueStateReady", 2)])
XQueueFeature = _enum("XQueueFeature", [("kQueueFeatureNone", 0), ("kQueueFeatureAsyncSubmit", 1),
                                        ("kQueueFeatureDynamicLevel", 2), ("kQueueFeatureDynamicThreshold", 4),
                                        ("kQueueFeatureDynamicBatchSize", 8), ("kQueueFeatureSyncSuspend", 16),
                                        ("kQueueFeatureResumeDropCommands", 32), ("kQueueFeatureMaskAll", -1)])
XQueueCreateFlag = _enum("XQueueCreateFlag", [("kQueueCreateFlagNone", 0), ("kQueueCreateFlagBlockingSubmit", 1),
                                              ("kQueueCreateFlagMaskAll", -1)])
XQueueSuspendFlag = _enum("XQueueSuspendFlag", [("kQueueSuspendFlagNone", 0), ("kQueueSuspendFlagSyncHwQueue", 1),
                                                ("kQueueSuspendFlagWaitAll", 2), ("kQueueSuspendFlagWaitIdle", 4),
                                                ("kQueueSuspendFlagMaskAll", -1)])
XQueueResumeFlag = _enum("XQueueResumeFlag", [("kQueueResumeFlagNone", 0), ("kQueueResumeFlagDropCommands", 1),
                                              ("kQueueResumeFlagMaskAll", -1)])
XSchedulerType = _enum("XSchedulerType", [("kSchedulerUnknown", 0), ("kSchedulerAppManaged", 1),
                                          ("kSchedulerLocal", 2), ("kSchedulerGlobal", 3), ("kSchedulerMax", 4)])
XPolicyType = _enum("XPolicyType", [("kPolicyUnknown", 0), ("kPolicyHighestPriorityFirst", 1),
                                    ("kPolicyHeterogeneousHighestPriorityFirst", 2),
                                    ("kPolicyCPUHighestPriorityFirst", 3), ("kPolicyUtilizationPartition", 4),
                                    ("kPolicyProcessUtilizationPartition", 5),
                                    ("kPolicyStrictProcessUtilizationPartition", 6),
                                    ("kPolicyKEarliestDeadlineFirst", 7), ("kPolicyLaxity", 8),
                                    ("kPolicyActiveWindowFirst", 9), ("kPolicyCompletelyFairScheduler", 10),
                                    ("kPolicyMultiLevelFeedbackQueue", 11), ("kPolicyMax", 12)])

XQueueHandle = int
HwQueueHandle = int
HwCommandHandle = int

Priority = int
PRIORITY_NO_EXECUTE, PRIORITY_MIN, PRIORITY_DEFAULT, PRIORITY_MAX = -256, -255, 0, 255
Utilization = int
UTILIZATION_MIN, UTILIZATION_DEFAULT, UTILIZATION_MAX = 0, 100, 100
Timeslice = int
TIMESLICE_MIN, TIMESLICE_DEFAULT, TIMESLICE_MAX, TIMESLICE_UNLIMITED = 100, 5000, 10000000, 0xFFFFFFFFFFFFFFFF
Laxity = int
NO_LAXITY = -1
Deadline = int
NO_DEADLINE = -1


def _res(code) -> XResult:
    try:
        return XResult(code)
    except ValueError:
        return XResult.kXSchedErrorUnknown


class XSched:
    """Static methods only, as in the reference. The libraries are loaded at the first call
    (xsched_amd raises NativeLibraryMissing when they have not been built)."""

    # ---- XQueue ----
    @staticmethod
    def XQueueCreate(hwq: HwQueueHandle, level: XPreemptLevel, flags: int) -> Tuple[XResult, XQueueHandle]:
        xq = ctypes.c_uint64(0)
        res = _xs.preempt().XQueueCreate(ctypes.byref(xq), hwq, int(level), int(flags))
        return _res(res), xq.value

    @staticmethod
    def XQueueDestroy(xq: XQueueHandle) -> XResult:
        return _res(_xs.preempt().XQueueDestroy(xq))

    @staticmethod
    def XQueueGet(hwq: HwQueueHandle) -> Tuple[XResult, XQueueHandle]:
        xq = ctypes.c_uint64(0)
        res = _xs.preempt().XQueueGet(ctypes.byref(xq), hwq)
        return _res(res), xq.value

    @staticmethod
    def XQueueSetPreemptLevel(xq: XQueueHandle, level: XPreemptLevel) -> XResult:
        return _res(_xs.preempt().XQueueSetPreemptLevel(xq, int(level)))

    @staticmethod
    def XQueueSetLaunchConfig(xq: XQueueHandle, threshold: int, batch_size: int) -> XResult:
        return _res(_xs.preempt().XQueueSetLaunchConfig(xq, threshold, batch_size))

    @staticmethod
    def XQueueSubmit(xq: XQueueHandle, hw_cmd: HwCommandHandle) -> XResult:
        return _res(_xs.preempt().XQueueSubmit(xq, hw_cmd))

    @staticmethod
    def XQueueWait(xq: XQueueHandle, hw_cmd: HwCommandHandle) -> XResult:
        return _res(_xs.preempt().XQueueWait(xq, hw_cmd))

    @staticmethod
    def XQueueWaitAll(xq: XQueueHandle) -> XResult:
        return _res(_xs.preempt().XQueueWaitAll(xq))

    @staticmethod
    def XQueueQuery(xq: XQueueHandle) -> Tuple[XResult, XQueueState]:
        state = ctypes.c_int(0)
        res = _xs.preempt().XQueueQuery(xq, ctypes.byref(state))
        try:
            return _res(res), XQueueState(state.value)
        except ValueError:
            return _res(res), XQueueState.kQueueStateUnknown

    @staticmethod
    def XQueueSuspend(xq: XQueueHandle, flags: int) -> XResult:
        return _res(_xs.preempt().XQueueSuspend(xq, int(flags)))

    @staticmethod
    def XQueueResume(xq: XQueueHandle, flags: int) -> XResult:
        return _res(_xs.preempt().XQueueResume(xq, int(flags)))

    @staticmethod
    def XQueueProfileHwCommandCount(xq: XQueueHandle) -> Tuple[XResult, int]:
        count = ctypes.c_int64(0)
        res = _xs.preempt().XQueueProfileHwCommandCount(xq, ctypes.byref(count))
        return _res(res), count.value

    # ---- HwQueue / HwCommand ----
    @staticmethod
    def HwQueueDestroy(hwq: HwQueueHandle) -> XResult:
        return _res(_xs.preempt().HwQueueDestroy(hwq))

    @staticmethod
    def HwQueueLaunch(hwq: HwQueueHandle, hw_cmd: HwCommandHandle) -> XResult:
        return _res(_xs.preempt().HwQueueLaunch(hwq, hw_cmd))

    @staticmethod
    def HwQueueSynchronize(hwq: HwQueueHandle) -> XResult:
        return _res(_xs.preempt().HwQueueSynchronize(hwq))

    @staticmethod
    def HwCommandDestroy(hw_cmd: HwCommandHandle) -> XResult:
        return _res(_xs.preempt().HwCommandDestroy(hw_cmd))

    # ---- hints ----
    @staticmethod
    def XHintSetScheduler(scheduler: XSchedulerType, policy: XPolicyType) -> XResult:
        return _res(_xs.preempt().XHintSetScheduler(int(scheduler), int(policy)))

    @staticmethod
    def XHintPriority(xq: XQueueHandle, prio: Priority) -> XResult:
        return _res(_xs.preempt().XHintPriority(xq, prio))

    @staticmethod
    def XHintUtilization(xq: XQueueHandle, util: Utilization) -> XResult:
        return _res(_xs.preempt().XHintUtilization(xq, util))

    @staticmethod
    def XHintTimeslice(ts_us: Timeslice) -> XResult:
        return _res(_xs.preempt().XHintTimeslice(ts_us))

    @staticmethod
    def XHintLaxity(xq: XQueueHandle, lax_us: Laxity, lax_prio: Priority, crit_prio: Priority) -> XResult:
        return _res(_xs.preempt().XHintLaxity(xq, lax_us, lax_prio, crit_prio))

    @staticmethod
    def XHintDeadline(xq: XQueueHandle, ddl_us: Deadline) -> XResult:
        return _res(_xs.preempt().XHintDeadline(xq, ddl_us))

    @staticmethod
    def XHintKDeadline(k: int) -> XResult:
        return _res(_xs.preempt().XHintKDeadline(k))

    # ---- this backend's adapter (no counterpart in the reference's module) ----
    @staticmethod
    def HipQueueCreate(stream: int) -> Tuple[XResult, HwQueueHandle]:
        """`stream` is the hipStream_t as an integer, e.g. torch.cuda.Stream().cuda_stream."""
        hwq = ctypes.c_uint64(0)
        res = _xs.halhip().HipQueueCreate(ctypes.byref(hwq), ctypes.c_void_p(stream))
        return _res(res), hwq.value

    @staticmethod
    def HipAxpyCommandCreate(alpha: float, x: int, y: int, n: int, guard: int) -> Tuple[XResult, HwCommandHandle]:
        cmd = ctypes.c_uint64(0)
        res = _xs.halhip().HipAxpyCommandCreate(ctypes.byref(cmd), alpha, x, y, n, guard)
        return _res(res), cmd.value

    @staticmethod
    def HipGemmBf16CommandCreate(a: int, b: int, c: int, m: int, n: int, k: int,
                                 guard: int) -> Tuple[XResult, HwCommandHandle]:
        cmd = ctypes.c_uint64(0)
        res = _xs.halhip().HipGemmBf16CommandCreate(ctypes.byref(cmd), a, b, c, m, n, k, guard)
        return _res(res), cmd.value

    @staticmethod
    def HipHistogramCommandCreate(keys: int, n: int, bins: int, n_bins: int,
                                  guard: int) -> Tuple[XResult, HwCommandHandle]:
        cmd = ctypes.c_uint64(0)
        res = _xs.halhip().HipHistogramCommandCreate(ctypes.byref(cmd), keys, n, bins, n_bins, guard)
        return _res(res), cmd.value

    @staticmethod
    def HipGuardedKernelCommandCreate(host_func: int, n_workgroups: int, block: Tuple[int, int, int],
                                      args: list, shared_mem_bytes: int = 0) -> Tuple[XResult, HwCommandHandle]:
        """A kernel of the caller's own that has the guard of xsched/hip/guard.h compiled in and an
        XGuardArgs as its last parameter. `host_func` is the kernel's host-side address, `args` the
        parameters in front of the XGuardArgs as ctypes values (c_void_p, c_float, c_size_t, ...);
        they are copied before this returns."""
        n = len(args)
        ptrs = (ctypes.c_void_p * max(n, 1))(*[ctypes.addressof(a) for a in args])
        sizes = (ctypes.c_size_t * max(n, 1))(*[ctypes.sizeof(a) for a in args])
        cmd = ctypes.c_uint64(0)
        res = _xs.halhip().HipGuardedKernelCommandCreate(ctypes.byref(cmd), ctypes.c_void_p(host_func), n_workgroups,
                                                         block[0], block[1], block[2], ptrs, sizes, n, shared_mem_bytes)
        return _res(res), cmd.value

    @staticmethod
    def HostQueueCreate() -> Tuple[XResult, HwQueueHandle]:
        hwq = ctypes.c_uint64(0)
        res = _xs.halhost().HostQueueCreate(ctypes.byref(hwq))
        return _res(res), hwq.value

    @staticmethod
    def HostVecAddCommandCreate(a: int, b: int, c: int, n: int, guard: int) -> Tuple[XResult, HwCommandHandle]:
        cmd = ctypes.c_uint64(0)
        res = _xs.halhost().HostVecAddCommandCreate(ctypes.byref(cmd), a, b, c, n, guard)
        return _res(res), cmd.value
