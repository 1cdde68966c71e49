"""ctypes binding of the XQueue / XHint C API and of the two hardware adapters.

The binding mirrors XSched's own Python package (reference
python/xsched/__init__.py:14-348 and platforms/hip/python/xsched/hip/__init__.py):
same enumerator values, same function names, errors reported as XResult codes.
Nothing is computed in Python; every call goes to the native libraries built by
``python -m xsched_amd.build`` into ``xsched_amd/lib``.
"""
import ctypes
import os
from ctypes import (CFUNCTYPE, POINTER, byref, c_char_p, c_double, c_float, c_int, c_int32, c_int64,
                    c_size_t, c_uint32, c_uint64, c_void_p)

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")


def _ask_for_larger_signal_pool():
    """What libhalhip.so does when it is loaded, done here as well because a Python program has
    usually imported torch (and with it the HIP runtime's library) before it loads the adapter:
    the runtime reads ROC_SIGNAL_POOL_SIZE at the first HIP call of the process. A value the
    user has set stays; XSCHED_HIP_SIGNAL_POOL=0 leaves the variable alone, any other number
    is the size asked for (default 512)."""
    try:
        size = int(os.environ.get("XSCHED_HIP_SIGNAL_POOL", "512"))
    except ValueError:
        size = 512
    if size > 0:
        os.environ.setdefault("ROC_SIGNAL_POOL_SIZE", str(size))


_ask_for_larger_signal_pool()

# ---- enumerators (include/xsched/types.h) ------------------------------------
kXSchedSuccess, kXSchedErrorHardware, kXSchedErrorInvalidValue = 0, 1, 2
kXSchedErrorNotFound, kXSchedErrorNotAllowed, kXSchedErrorNotSupported = 3, 4, 5
kXSchedErrorBadResponse, kXSchedErrorUnknown = 6, 999

kPreemptLevelUnknown, kPreemptLevelBlock, kPreemptLevelDeactivate, kPreemptLevelInterrupt = 0, 1, 2, 3
kQueueStateUnknown, kQueueStateIdle, kQueueStateReady = 0, 1, 2
kQueueCreateFlagNone, kQueueCreateFlagBlockingSubmit = 0, 1
kQueueSuspendFlagNone, kQueueSuspendFlagSyncHwQueue = 0, 1
kQueueSuspendFlagWaitAll, kQueueSuspendFlagWaitIdle = 2, 4
kQueueResumeFlagNone, kQueueResumeFlagDropCommands = 0, 1
kSchedulerUnknown, kSchedulerAppManaged, kSchedulerLocal, kSchedulerGlobal = 0, 1, 2, 3
kPolicyUnknown, kPolicyHighestPriorityFirst, kPolicyLaxity = 0, 1, 8
kPolicyHeterogeneousHighestPriorityFirst, kPolicyCPUHighestPriorityFirst = 2, 3
kPolicyUtilizationPartition, kPolicyProcessUtilizationPartition = 4, 5
kPolicyKEarliestDeadlineFirst, kPolicyActiveWindowFirst = 7, 9
kPolicyCompletelyFairScheduler, kPolicyMultiLevelFeedbackQueue = 10, 11
PRIORITY_NO_EXECUTE, PRIORITY_MIN, PRIORITY_DEFAULT, PRIORITY_MAX = -256, -255, 0, 255

XResult = c_int
XQueueHandle = c_uint64
HwQueueHandle = c_uint64
HwCommandHandle = c_uint64
LaunchCallback = CFUNCTYPE(c_int, c_uint64, c_void_p)
HostKernelFn = CFUNCTYPE(None, c_void_p, c_uint32, c_uint32)


class NativeLibraryMissing(RuntimeError):
    """Raised when a native library has not been built; there is no fallback."""


def _load(name, mode=ctypes.RTLD_LOCAL):
    path = os.path.join(_LIB_DIR, name)
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} not found: run `python -m xsched_amd.build` (no Python fallback exists)")
    return ctypes.CDLL(path, mode=mode)


_preempt = None
_halhost = None
_halhip = None

# name -> (restype, argtypes) ; one table per library, used both to set up ctypes
# prototypes and by the tests that check every declared symbol is exported.
PREEMPT_API = {
    "XQueueCreate": (XResult, [POINTER(c_uint64), c_uint64, c_int64, c_int64]),
    "XQueueDestroy": (XResult, [c_uint64]),
    "XQueueGet": (XResult, [POINTER(c_uint64), c_uint64]),
    "XQueueSetPreemptLevel": (XResult, [c_uint64, c_int]),
    "XQueueSetLaunchConfig": (XResult, [c_uint64, c_int64, c_int64]),
    "XQueueSubmit": (XResult, [c_uint64, c_uint64]),
    "XQueueWait": (XResult, [c_uint64, c_uint64]),
    "XQueueWaitAll": (XResult, [c_uint64]),
    "XQueueQuery": (XResult, [c_uint64, POINTER(c_int)]),
    "XQueueSuspend": (XResult, [c_uint64, c_int64]),
    "XQueueResume": (XResult, [c_uint64, c_int64]),
    "XQueueProfileHwCommandCount": (XResult, [c_uint64, POINTER(c_int64)]),
    "XQueueProfileDirectLaunchCount": (XResult, [c_uint64, POINTER(c_int64)]),
    "HwQueueDestroy": (XResult, [c_uint64]),
    "HwQueueLaunch": (XResult, [c_uint64, c_uint64]),
    "HwQueueSynchronize": (XResult, [c_uint64]),
    "HwCommandCreateCallback": (XResult, [POINTER(c_uint64), LaunchCallback, c_void_p]),
    "HwCommandDestroy": (XResult, [c_uint64]),
    "XHintSetScheduler": (XResult, [c_int, c_int]),
    "XHintPriority": (XResult, [c_uint64, c_int32]),
    "XHintUtilization": (XResult, [c_uint64, c_int32]),
    "XHintTimeslice": (XResult, [c_int64]),
    "XHintLaxity": (XResult, [c_uint64, c_int64, c_int32, c_int32]),
    "XHintDeadline": (XResult, [c_uint64, c_int64]),
    "XHintKDeadline": (XResult, [c_size_t]),
}

HALHOST_API = {
    "HostQueueCreate": (XResult, [POINTER(c_uint64)]),
    "HostKernelCommandCreate": (XResult, [POINTER(c_uint64), HostKernelFn, c_void_p, c_uint32, c_int]),
    "HostVecAddCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_void_p, c_void_p, c_size_t, c_int]),
    "HostAxpyCommandCreate": (XResult, [POINTER(c_uint64), c_float, c_void_p, c_void_p, c_size_t, c_int]),
    "HostBenchFillUniform": (None, [c_void_p, c_uint64, c_uint64, c_uint64, c_uint64]),
    "HostBenchRunVecAdd": (XResult, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     POINTER(c_double), POINTER(c_double), c_void_p]),
    "HostQueueGetStats": (XResult, [c_uint64, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64)]),
}

HALHIP_API = {
    "HipQueueCreate": (XResult, [POINTER(c_uint64), c_void_p]),
    "HipQueueGetStats": (XResult, [c_uint64, POINTER(c_uint64)]),
    "HipQueueGetPoolStats": (XResult, [c_uint64, POINTER(c_uint64)]),
    "HipQueueSetMarkerOnKernel": (XResult, [c_uint64, c_int]),
    "HipQueueMarkEpochFlushed": (XResult, [c_uint64]),
    "HipAxpyCommandCreate": (XResult, [POINTER(c_uint64), c_float, c_void_p, c_void_p, c_size_t, c_int]),
    "HipGemmBf16CommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_void_p, c_void_p,
                                           c_int, c_int, c_int, c_int]),
    "HipHistogramCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_size_t, c_void_p,
                                            c_uint32, c_int]),
    "HipHistogramLaunchNoAlloc": (XResult, [c_void_p, c_void_p, c_size_t, c_void_p, c_uint32]),
    "HipMemcpyCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_void_p, c_size_t, c_int]),
    "HipMemsetCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_int, c_size_t]),
    "HipMemsetWideCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_uint32, c_size_t, c_uint32]),
    "HipEventRecordCommandCreate": (XResult, [POINTER(c_uint64), c_void_p]),
    "HipEventWaitCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_uint32]),
    "HipRecordedEventWaitCommandCreate": (XResult, [POINTER(c_uint64), c_uint64]),
    "HipKernelCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_uint32, c_uint32, c_uint32,
                                         c_uint32, c_uint32, c_uint32, POINTER(c_void_p),
                                         POINTER(c_size_t), c_size_t, c_uint32]),
    "HipGuardedKernelCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_uint32, c_uint32, c_uint32, c_uint32,
                                                POINTER(c_void_p), POINTER(c_size_t), c_size_t, c_uint32]),
    "HipModuleKernelCommandCreate": (XResult, [POINTER(c_uint64), c_void_p, c_uint32, c_uint32, c_uint32,
                                               c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_size_t]),
}

SHIMHIP_API = {
    "HipShimKernelArgLayout": (XResult, [c_void_p, c_size_t, c_char_p, POINTER(c_uint32), POINTER(c_uint32),
                                         c_size_t, POINTER(c_size_t)]),
    "HipShimGetStats": (XResult, [POINTER(c_uint64)]),
}


def _bind(lib, table):
    for name, (res, args) in table.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


def preempt():
    """libpreempt.so: XQueue core + scheduler + C API."""
    global _preempt
    if _preempt is None:
        _preempt = _load("libpreempt.so")
        _bind(_preempt, PREEMPT_API)
    return _preempt


def halhost():
    """libhalhost.so: CPU hardware-queue adapter."""
    global _halhost
    if _halhost is None:
        preempt()
        _halhost = _load("libhalhost.so")
        _bind(_halhost, HALHOST_API)
    return _halhost


def halhip():
    """libhalhip.so: MI355X HIP adapter (fails loudly when it has not been built)."""
    global _halhip
    if _halhip is None:
        preempt()
        _halhip = _load("libhalhip.so")
        _bind(_halhip, HALHIP_API)
    return _halhip


_shimhip = None


def shimhip():
    """libshimhip.so: the HIP interception shim. Loaded here only for its two test entry points;
    a library loaded this way interposes nothing."""
    global _shimhip
    if _shimhip is None:
        halhip()
        _shimhip = _load("libshimhip.so")
        _bind(_shimhip, SHIMHIP_API)
    return _shimhip


def check(res, what=""):
    if res != kXSchedSuccess:
        raise RuntimeError(f"XSched call failed with XResult {res} {what}")
    return res


# ---- thin conveniences used by tests and bench ---------------------------------

def xqueue_create(hwq, level=kPreemptLevelBlock, flags=kQueueCreateFlagNone):
    xq = c_uint64(0)
    check(preempt().XQueueCreate(byref(xq), hwq, level, flags), "XQueueCreate")
    return xq.value


def host_queue_create():
    hwq = c_uint64(0)
    check(halhost().HostQueueCreate(byref(hwq)), "HostQueueCreate")
    return hwq.value


def hip_queue_create(stream):
    hwq = c_uint64(0)
    check(halhip().HipQueueCreate(byref(hwq), c_void_p(stream)), "HipQueueCreate")
    return hwq.value


__all__ = [n for n in dir() if not n.startswith("_")]
