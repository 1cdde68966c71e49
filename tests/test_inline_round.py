"""In-process scheduling rounds on the submitter's thread. A queue that becomes ready tells the
local scheduler from inside XQueueSubmit, and the scheduler (when no other round is under way)
runs the round right there: it suspends and deactivates OTHER queues on the submitter's
thread. That must happen with none of the submitting queue's own locks held, or the queue's
launcher, its other submitters and every XQueueQuery / XQueueWaitAll caller stall for the whole
round. The recording hardware queue of oracle/xqueue_probe.cpp calls back from its
Deactivate(), i.e. from inside the round."""
import threading
import time
from ctypes import CFUNCTYPE, byref, c_int, c_int32, c_uint64, c_void_p

from xqueue_trace_driver import DEACTIVATABLE, NONE, Core, ok

LOCAL, APP_MANAGED, HPF = 2, 1, 1
READY = 2


def wait_for(cond, limit=3.0):
    deadline = time.time() + limit
    while not cond() and time.time() < deadline:
        time.sleep(0.001)
    return cond()


def trace(rec, hwq):
    import ctypes
    buf = ctypes.create_string_buffer(1 << 14)
    rec.RecQueueTrace(hwq, buf, 1 << 14)
    return buf.value.decode().split()


def test_a_round_on_the_submitters_thread_holds_none_of_its_queues_locks():
    core = Core.product()
    api, rec = core.api, core.rec
    api.XHintPriority.argtypes = [c_uint64, c_int32]
    rec.RecQueueOnDeactivate.argtypes = [c_uint64, c_void_p, c_void_p]
    ok(api.XHintSetScheduler(LOCAL, HPF))
    hw_lo, hw_hi, xq_lo, xq_hi = c_uint64(), c_uint64(), c_uint64(), c_uint64()
    ok(rec.RecQueueCreate(byref(hw_lo), 2)); ok(rec.RecQueueCreate(byref(hw_hi), 2))
    ok(api.XQueueCreate(byref(xq_lo), hw_lo.value, 2, 0)); ok(api.XQueueCreate(byref(xq_hi), hw_hi.value, 1, 0))
    ok(api.XHintPriority(xq_lo.value, 1)); ok(api.XHintPriority(xq_hi.value, 5))
    time.sleep(0.05)   # the hints are folded in by the scheduler's own thread

    try:
        # the low queue gets a flushable command that stays in flight (the test never completes it yet)
        cmd = c_uint64()
        rec.RecCommandCreate(byref(cmd), DEACTIVATABLE, 0)
        ok(api.XQueueSubmit(xq_lo.value, cmd.value))
        assert wait_for(lambda: any(t.startswith("L1") for t in trace(rec, hw_lo.value)))
        time.sleep(0.02)   # its own round is over

        seen = {}

        @CFUNCTYPE(None, c_void_p)
        def inside_the_round(_):
            seen["thread"] = threading.get_ident()
            answered = threading.Event()

            def ask():   # needs the submitting queue's ring lock
                st = c_int()
                ok(api.XQueueQuery(xq_hi.value, byref(st)))
                seen["state"] = st.value
                answered.set()

            helper = threading.Thread(target=ask)
            helper.start()
            seen["query_answered_during_the_round"] = answered.wait(2.0)
            seen["helper"] = helper

        ok(rec.RecQueueOnDeactivate(hw_lo.value, inside_the_round, None))
        submitter = threading.get_ident()
        rec.RecCommandCreate(byref(cmd), NONE, 0)
        ok(api.XQueueSubmit(xq_hi.value, cmd.value))      # Ready -> round -> Suspend(low) -> Deactivate(low) -> callback

        assert wait_for(lambda: "thread" in seen), "the high queue's Ready did not deactivate the low queue"
        seen["helper"].join(5)
        assert seen["thread"] == submitter, "the round did not run on the submitting thread"
        assert seen["query_answered_during_the_round"], "XQueueQuery on the submitting queue blocked until the round was over"
        assert seen["state"] == READY
        assert "D" in trace(rec, hw_lo.value)
        # the submission itself is not lost or reordered by the round: the launcher launches it
        assert wait_for(lambda: any(t.startswith("L1") for t in trace(rec, hw_hi.value)))
    finally:
        rec.RecQueueOnDeactivate(hw_lo.value, None, None)
        rec.RecQueueComplete(hw_hi.value, 1000); rec.RecQueueComplete(hw_lo.value, 1000)
        ok(api.XQueueDestroy(xq_hi.value)); ok(api.XQueueDestroy(xq_lo.value))
        ok(api.HwQueueDestroy(hw_hi.value)); ok(api.HwQueueDestroy(hw_lo.value))
        ok(api.XHintSetScheduler(APP_MANAGED, 0))


def test_ready_and_idle_reach_the_scheduler_in_order_when_ready_is_sent_after_the_launch():
    """Many short busy periods on a queue whose commands complete at once: after each, the
    queue must end up Idle for the scheduler as well (a Ready that overtook its Idle would leave
    the lower queue suspended for good: its command would never be launched)."""
    core = Core.product()
    api, rec = core.api, core.rec
    api.XHintPriority.argtypes = [c_uint64, c_int32]
    api.XQueueWaitAll.argtypes = [c_uint64]
    ok(api.XHintSetScheduler(LOCAL, HPF))
    hw_lo, hw_hi, xq_lo, xq_hi = c_uint64(), c_uint64(), c_uint64(), c_uint64()
    ok(rec.RecQueueCreate(byref(hw_lo), 2)); ok(rec.RecQueueCreate(byref(hw_hi), 2))
    ok(api.XQueueCreate(byref(xq_lo), hw_lo.value, 1, 0)); ok(api.XQueueCreate(byref(xq_hi), hw_hi.value, 1, 0))
    ok(api.XHintPriority(xq_lo.value, 1)); ok(api.XHintPriority(xq_hi.value, 5))
    rec.RecQueueComplete(hw_hi.value, 1 << 40); rec.RecQueueComplete(hw_lo.value, 1 << 40)   # everything completes at once
    time.sleep(0.05)
    try:
        cmd = c_uint64()
        for i in range(200):
            rec.RecCommandCreate(byref(cmd), NONE, 0)
            ok(api.XQueueSubmit(xq_hi.value, cmd.value))
            if i % 3 == 0:
                ok(api.XQueueWaitAll(xq_hi.value))
        ok(api.XQueueWaitAll(xq_hi.value))
        # the high queue is idle now; the low queue's command has to get through
        rec.RecCommandCreate(byref(cmd), NONE, 0)
        ok(api.XQueueSubmit(xq_lo.value, cmd.value))
        assert wait_for(lambda: any(t.startswith("L1") for t in trace(rec, hw_lo.value)), 3.0), \
            "the low queue stayed suspended: the scheduler still believes the high queue is ready"
    finally:
        ok(api.XQueueDestroy(xq_hi.value)); ok(api.XQueueDestroy(xq_lo.value))
        ok(api.HwQueueDestroy(hw_hi.value)); ok(api.HwQueueDestroy(hw_lo.value))
        ok(api.XHintSetScheduler(APP_MANAGED, 0))
