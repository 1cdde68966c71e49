"""The reference-shaped Python interface (xsched_amd/xsched_api.py): same names, values
and return conventions as XSched's python/xsched/__init__.py, exercised on the host adapter."""
import numpy as np

from xsched_amd.xsched_api import (XPolicyType, XPreemptLevel, XQueueCreateFlag, XQueueResumeFlag, XQueueState,
                                   XQueueSuspendFlag, XResult, XSched, XSchedulerType, PRIORITY_MAX,
                                   TIMESLICE_DEFAULT)


def test_enum_values_are_the_wire_values():
    assert XResult.kXSchedErrorUnknown == 999 and XResult.kXSchedErrorNotSupported == 5
    assert XPreemptLevel.kPreemptLevelDeactivate == 2
    assert XPolicyType.kPolicyLaxity == 8 and XPolicyType.kPolicyMultiLevelFeedbackQueue == 11
    assert XSchedulerType.kSchedulerGlobal == 3
    assert XQueueSuspendFlag.kQueueSuspendFlagWaitIdle == 4
    assert PRIORITY_MAX == 255 and TIMESLICE_DEFAULT == 5000


def test_queue_life_cycle_through_the_reference_shaped_interface():
    res, hwq = XSched.HostQueueCreate()
    assert res == XResult.kXSchedSuccess and hwq != 0
    res, xq = XSched.XQueueCreate(hwq, XPreemptLevel.kPreemptLevelBlock, XQueueCreateFlag.kQueueCreateFlagNone)
    assert res == XResult.kXSchedSuccess and xq != 0
    assert XSched.XQueueGet(hwq) == (XResult.kXSchedSuccess, xq)
    assert XSched.XQueueSetLaunchConfig(xq, 4, 2) == XResult.kXSchedSuccess
    assert XSched.XQueueSetPreemptLevel(xq, XPreemptLevel.kPreemptLevelDeactivate) == XResult.kXSchedSuccess
    # above what the adapter offers: a warning and no change, but success, as in the reference
    # (preempt/src/xqueue/async_xqueue.cpp:161-165)
    assert XSched.XQueueSetPreemptLevel(xq, XPreemptLevel.kPreemptLevelInterrupt) == XResult.kXSchedSuccess
    assert XSched.XQueueSetPreemptLevel(xq, XPreemptLevel.kPreemptLevelMax) == XResult.kXSchedErrorInvalidValue

    n = 1 << 12
    a = np.arange(n, dtype=np.float32)
    b = np.full(n, 0.5, np.float32)
    c = np.zeros(n, np.float32)
    for _ in range(3):
        res, cmd = XSched.HostVecAddCommandCreate(a.ctypes.data, b.ctypes.data, c.ctypes.data, n, 1)
        assert res == XResult.kXSchedSuccess
        assert XSched.XQueueSubmit(xq, cmd) == XResult.kXSchedSuccess
    assert XSched.XQueueWaitAll(xq) == XResult.kXSchedSuccess
    assert np.array_equal(c, a + b)
    # idle a moment after WaitAll has returned: when the launch thread comes back and finds nothing
    import time
    deadline = time.time() + 2.0
    while XSched.XQueueQuery(xq)[1] != XQueueState.kQueueStateIdle and time.time() < deadline:
        time.sleep(0.0005)
    assert XSched.XQueueQuery(xq) == (XResult.kXSchedSuccess, XQueueState.kQueueStateIdle)
    res, count = XSched.XQueueProfileHwCommandCount(xq)
    assert res == XResult.kXSchedSuccess and count == 3

    assert XSched.XQueueSuspend(xq, XQueueSuspendFlag.kQueueSuspendFlagNone) == XResult.kXSchedSuccess
    assert XSched.XQueueResume(xq, XQueueResumeFlag.kQueueResumeFlagNone) == XResult.kXSchedSuccess
    assert XSched.HwQueueDestroy(hwq) == XResult.kXSchedErrorNotAllowed      # an XQueue is still attached
    assert XSched.XQueueDestroy(xq) == XResult.kXSchedSuccess
    assert XSched.XQueueDestroy(xq) == XResult.kXSchedErrorNotFound
    assert XSched.HwQueueDestroy(hwq) == XResult.kXSchedSuccess


def test_hints_through_the_reference_shaped_interface():
    assert XSched.XHintSetScheduler(XSchedulerType.kSchedulerLocal,
                                    XPolicyType.kPolicyKEarliestDeadlineFirst) == XResult.kXSchedSuccess
    res, hwq = XSched.HostQueueCreate()
    res, xq = XSched.XQueueCreate(hwq, XPreemptLevel.kPreemptLevelBlock, 0)
    assert XSched.XHintDeadline(xq, 5000) == XResult.kXSchedSuccess
    assert XSched.XHintKDeadline(2) == XResult.kXSchedSuccess
    assert XSched.XHintPriority(xq, 3) == XResult.kXSchedSuccess
    assert XSched.XHintUtilization(xq, 50) == XResult.kXSchedSuccess
    assert XSched.XHintTimeslice(2000) == XResult.kXSchedSuccess
    assert XSched.XHintLaxity(xq, 1000, 1, 2) == XResult.kXSchedSuccess
    assert XSched.XHintSetScheduler(XSchedulerType.kSchedulerLocal,
                                    XPolicyType.kPolicyStrictProcessUtilizationPartition) == XResult.kXSchedErrorInvalidValue
    assert XSched.XQueueDestroy(xq) == XResult.kXSchedSuccess
    assert XSched.HwQueueDestroy(hwq) == XResult.kXSchedSuccess
    assert XSched.XHintSetScheduler(XSchedulerType.kSchedulerAppManaged, XPolicyType.kPolicyUnknown) == XResult.kXSchedSuccess
