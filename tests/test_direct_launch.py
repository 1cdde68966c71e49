"""Direct launch: with an adapter that allows it, a command that arrives while the launch
thread sleeps on an empty buffer is launched on the submitting thread, and XQueueWaitAll
drains on the calling thread. Neither may change what the queue computes, the order it
launches in, or what a scheduler is told; XSCHED_DIRECT_LAUNCH=OFF switches both off."""
import os
import subprocess
import sys
import threading
import time
from ctypes import byref, c_int, c_int64, c_uint64

import numpy as np

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def direct_count(xs, xq):
    n = c_int64()
    xs.check(xs.preempt().XQueueProfileDirectLaunchCount(xq, byref(n)))
    return n.value


def wait_idle(xs, xq):
    st = c_int()
    for _ in range(2000):
        xs.check(xs.preempt().XQueueQuery(xq, byref(st)))
        if st.value == xs.kQueueStateIdle:
            return
        time.sleep(0.0005)
    raise AssertionError("queue never became idle")


def test_sparse_submissions_launch_on_the_submitting_thread(xs):
    """One command at a time, the queue idle in between: each is launched directly, the
    chained additions still give k, and the queue still goes Ready -> Idle every time."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 8, 4))
    n, k = 4096, 40
    ones = np.ones(n, np.float32); acc = np.zeros(n, np.float32)
    for i in range(k):
        wait_idle(xs, xq)
        cmd = c_uint64()
        xs.check(h.HostVecAddCommandCreate(byref(cmd), acc.ctypes.data, ones.ctypes.data, acc.ctypes.data, n, 0))
        xs.check(p.XQueueSubmit(xq, cmd.value))
        xs.check(p.XQueueWaitAll(xq))
        assert np.all(acc == i + 1), "XQueueWaitAll returned before the command had run"
    assert direct_count(xs, xq) == k
    wait_idle(xs, xq)
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_bursts_keep_submission_order(xs):
    """Bursts from two threads into one queue, each burst starting on an idle queue: the
    first command of a burst may go directly, the rest queue up behind it. In-place AXPY
    is order-sensitive per element only through the count, so the check is the count of
    applications plus the launch thread's own accounting."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 4, 2))
    n, bursts, per = 1 << 14, 30, 7
    x = oracle.fill_uniform(2, 1, 0, n); y0 = oracle.fill_uniform(2, 2, 0, n); y = y0.copy()

    def submitter():
        for _ in range(bursts):
            for _ in range(per):
                cmd = c_uint64()
                xs.check(h.HostAxpyCommandCreate(byref(cmd), 0.5, x.ctypes.data, y.ctypes.data, n, 0))
                xs.check(p.XQueueSubmit(xq, cmd.value))
            xs.check(p.XQueueWaitAll(xq))
            time.sleep(0.001)

    threads = [threading.Thread(target=submitter) for _ in range(2)]
    for t in threads: t.start()
    for t in threads: t.join()
    xs.check(p.XQueueWaitAll(xq))
    total = c_int64()
    xs.check(p.XQueueProfileHwCommandCount(xq, byref(total)))
    assert total.value == 2 * bursts * per
    want = oracle.axpy(0.5, x, y0, 2 * bursts * per)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert 0 < direct_count(xs, xq) <= 2 * bursts * per
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_suspended_queue_never_launches_directly(xs):
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq, xs.kPreemptLevelDeactivate)
    n = 1 << 14
    x = np.ones(n, np.float32); y = np.zeros(n, np.float32)
    wait_idle(xs, xq)
    xs.check(p.XQueueSuspend(xq, 0))
    cmd = c_uint64()
    xs.check(h.HostAxpyCommandCreate(byref(cmd), 1.0, x.ctypes.data, y.ctypes.data, n, 1))
    xs.check(p.XQueueSubmit(xq, cmd.value))
    time.sleep(0.05)
    assert direct_count(xs, xq) == 0 and np.all(y == 0), "a suspended queue launched a command"
    xs.check(p.XQueueResume(xq, 0))
    xs.check(p.XQueueWaitAll(xq))
    assert np.all(y == 1)
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_level2_churn_with_sparse_direct_launches(xs):
    """Suspend / resume churn at Level 2 while commands arrive one by one on a mostly idle
    queue (so that many go directly): flushed and replayed or not, every application
    happens exactly once."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq, xs.kPreemptLevelDeactivate)
    xs.check(p.XQueueSetLaunchConfig(xq, 4, 2))
    n, times = 1 << 18, 120
    x = oracle.fill_uniform(3, 1, 0, n); y0 = oracle.fill_uniform(3, 2, 0, n); y = y0.copy()
    stop = threading.Event()

    def churn():
        while not stop.is_set():
            time.sleep(0.0003)
            p.XQueueSuspend(xq, 0)
            time.sleep(0.0001)
            p.XQueueResume(xq, 0)

    t = threading.Thread(target=churn); t.start()
    for i in range(times):
        cmd = c_uint64()
        xs.check(h.HostAxpyCommandCreate(byref(cmd), 0.25, x.ctypes.data, y.ctypes.data, n, 1))
        xs.check(p.XQueueSubmit(xq, cmd.value))
        if i % 3 == 2:
            xs.check(p.XQueueWaitAll(xq))
            time.sleep(0.0004)
    stop.set(); t.join()
    xs.check(p.XQueueWaitAll(xq))
    want = oracle.axpy(0.25, x, y0, times)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert direct_count(xs, xq) > 0
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


SWITCH_OFF = """
import sys, time
sys.path.insert(0, %r)
from ctypes import byref, c_int64, c_uint64
import numpy as np
import xsched_amd as xs
p, h = xs.preempt(), xs.halhost()
hwq = xs.host_queue_create(); xq = xs.xqueue_create(hwq)
a = np.zeros(64, np.float32); one = np.ones(64, np.float32)
for _ in range(5):
    time.sleep(0.01)
    cmd = c_uint64()
    xs.check(h.HostVecAddCommandCreate(byref(cmd), a.ctypes.data, one.ctypes.data, a.ctypes.data, 64, 0))
    xs.check(p.XQueueSubmit(xq, cmd.value)); xs.check(p.XQueueWaitAll(xq))
n = c_int64(); xs.check(p.XQueueProfileDirectLaunchCount(xq, byref(n)))
print(int(a[0]), n.value)
"""


def test_environment_switch():
    for value, want_direct in (("OFF", False), ("ON", True)):
        env = dict(os.environ, XSCHED_DIRECT_LAUNCH=value, XLOG_LEVEL="ERRO")
        out = subprocess.run([sys.executable, "-c", SWITCH_OFF % ROOT], env=env, capture_output=True,
                             text=True, timeout=60, check=True).stdout.split()
        assert out[0] == "5"
        assert (int(out[1]) > 0) == want_direct


def test_a_wait_on_a_queue_paused_after_a_direct_launch_ends_with_the_resume(xs):
    """The submitter launches, the queue is paused before the submitter starts to wait, and it
    is resumed a moment later: the wait returns with the resume. (The launcher stands by for
    callers that launch themselves; a waiter that left the device to it whenever the queue
    was paused got its answer only when the stand-by of 500 us had passed.) The smallest of
    several trials is what is checked: it cannot be lowered by a busy machine."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 8, 4))
    n = 1024
    ones = np.ones(n, np.float32); acc = np.zeros(n, np.float32)
    waits = []
    for trial in range(12):
        wait_idle(xs, xq)
        cmd = c_uint64()
        xs.check(h.HostVecAddCommandCreate(byref(cmd), acc.ctypes.data, ones.ctypes.data, acc.ctypes.data, n, 0))
        before = direct_count(xs, xq)
        xs.check(p.XQueueSubmit(xq, cmd.value))
        assert direct_count(xs, xq) == before + 1, "the command was not launched by the submitter"
        xs.check(p.XQueueSuspend(xq, 0))
        resumer = threading.Thread(target=lambda: (time.sleep(0.00005), xs.check(p.XQueueResume(xq, 0))))
        t0 = time.perf_counter()
        resumer.start()
        xs.check(p.XQueueWaitAll(xq))
        waits.append(time.perf_counter() - t0)
        resumer.join()
        assert np.all(acc == trial + 1)
    print("waits (us):", [round(w * 1e6) for w in waits])
    # the stand-by lasts 500 us from the launch; the resume comes 50 us (plus the start of a
    # Python thread) after the wait began
    assert min(waits) < 460e-6, "every wait took as long as the launcher's stand-by"
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_a_command_launched_by_the_launcher_is_waited_for_by_the_launcher_at_once(xs):
    """Submitted while the queue is paused, a command is launched by the launcher once the
    queue runs again, and the submitter sleeps on the completion number: the launcher has to
    wait for the device right away, not stand by as it does after a submitter's own launch."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 8, 4))
    n = 1024
    ones = np.ones(n, np.float32); acc = np.zeros(n, np.float32)
    waits = []
    for trial in range(12):
        wait_idle(xs, xq)
        cmd = c_uint64()
        xs.check(h.HostVecAddCommandCreate(byref(cmd), acc.ctypes.data, ones.ctypes.data, acc.ctypes.data, n, 0))
        xs.check(p.XQueueSuspend(xq, 0))
        before = direct_count(xs, xq)
        xs.check(p.XQueueSubmit(xq, cmd.value))
        assert direct_count(xs, xq) == before, "a paused queue launched on the submitter's thread"
        resumer = threading.Thread(target=lambda: (time.sleep(0.00005), xs.check(p.XQueueResume(xq, 0))))
        t0 = time.perf_counter()
        resumer.start()
        xs.check(p.XQueueWaitAll(xq))
        waits.append(time.perf_counter() - t0)
        resumer.join()
        assert np.all(acc == trial + 1)
    print("waits (us):", [round(w * 1e6) for w in waits])
    assert min(waits) < 2e-3, "the launcher did not wait for the device when it had launched"
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_a_submitter_that_never_waits_hands_its_launches_to_the_launcher(xs):
    """Direct launch is for submitters that wait for what they submit. After eight
    submissions in a row with no wait in between, the rest of the stream goes through the
    ring (the launcher makes the launches on another core while the submitter goes on);
    a wait re-arms it. The computed values are the same either way."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 16, 8))
    n, k = 2048, 40
    ones = np.ones(n, np.float32); acc = np.zeros(n, np.float32)

    def stream_of(count, gap):
        for _ in range(count):
            cmd = c_uint64()
            xs.check(h.HostVecAddCommandCreate(byref(cmd), acc.ctypes.data, ones.ctypes.data, acc.ctypes.data, n, 0))
            xs.check(p.XQueueSubmit(xq, cmd.value))
            time.sleep(gap)     # long enough for the launcher to go back to sleep in between

    wait_idle(xs, xq)
    stream_of(k, 0.004)
    streamed = direct_count(xs, xq)
    xs.check(p.XQueueWaitAll(xq))
    assert np.all(acc == k)
    assert 1 <= streamed <= 8, f"{streamed} of {k} unwaited submissions were launched by the submitter"
    wait_idle(xs, xq)
    stream_of(3, 0.004)
    assert direct_count(xs, xq) == streamed + 3, "a wait did not re-arm the direct launch"
    xs.check(p.XQueueWaitAll(xq))
    assert np.all(acc == k + 3)
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))
