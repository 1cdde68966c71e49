"""CPU-only checks of the C ABI: every declared symbol is exported, argument errors
come back as the reference's XResult codes, ownership rules hold, and the whole stack
(XQueue core + local scheduler + host adapter) runs the CPU configuration end to end
with results equal to the oracle's."""
import ctypes
import os
import re
import threading
import time
from ctypes import byref, c_int, c_int64, c_uint64, c_void_p

import numpy as np
import pytest

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include", "xsched")


def declared(header):
    text = open(os.path.join(INC, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:XResult|XBench \*|void)\s+\*?([A-Za-z]\w+)\s*\(", text, flags=re.M)


def exported(lib):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(ROOT, "xsched_amd", "lib", lib)],
                         capture_output=True, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line}


def test_every_declared_symbol_is_exported(xs):
    pre = exported("libpreempt.so")
    for h in ("xqueue.h", "hint.h"):
        names = declared(h)
        assert len(names) >= 7
        for n in names:
            assert n in pre, f"{n} declared in {h} but not exported by libpreempt.so"
    host = exported("libhalhost.so")
    for h in ("host/hal.h", "host/bench.h"):
        for n in declared(h):
            assert n in host, f"{n} declared in {h} but not exported by libhalhost.so"
    hip_path = os.path.join(ROOT, "xsched_amd", "lib", "libhalhip.so")
    assert os.path.exists(hip_path), "libhalhip.so has not been built"
    hip = exported("libhalhip.so")
    for h in ("hip/hal.h", "hip/bench.h"):
        for n in declared(h):
            assert n in hip, f"{n} declared in {h} but not exported by libhalhip.so"
    # the ctypes tables and the headers agree
    assert set(xs.PREEMPT_API) == set(declared("xqueue.h")) | set(declared("hint.h"))
    assert set(xs.HALHOST_API) == set(declared("host/hal.h")) | set(declared("host/bench.h"))
    assert set(xs.HALHIP_API) == set(declared("hip/hal.h"))


def test_hip_library_loads_without_a_gpu(xs):
    lib = xs.halhip()   # load + bind only; no HIP call is made
    assert lib.HipQueueCreate is not None


def test_gemm_command_takes_any_shape_and_refuses_what_no_kernel_can_address(xs):
    """Creating a command launches nothing, so the argument checks run without a GPU. The fast
    kernels take M and N in multiples of 128, K of 64 (K and N at most 2^22) and operands
    aligned to 16 bytes; everything else with positive sizes and element-aligned operands goes
    to the any-shape kernel. Refused: sizes below 1, odd addresses, null pointers, guard modes
    outside 0..3, more tiles than a progress map has bytes."""
    from ctypes import byref, c_uint64
    lib, cmd = xs.halhip(), c_uint64()
    a, b, c = 1 << 20, 2 << 20, 3 << 20           # never dereferenced here
    ok = lambda *args: lib.HipGemmBf16CommandCreate(byref(cmd), *args)  # noqa: E731
    for good in [(a, b, c, 256, 384, 64, 0), (a, b, c, 128, 128, 1 << 22, 1),
                 (a, b, c, 200, 256, 64, 0), (a, b, c, 256, 200, 64, 0), (a, b, c, 256, 256, 96, 0),
                 (a, b, c, 256, 256, (1 << 22) + 64, 0), (a + 2, b, c, 256, 256, 64, 0),
                 (a, b, c + 8, 256, 256, 64, 0), (a, b, c, 1, 1, 1, 3)]:
        assert ok(*good) == xs.kXSchedSuccess, good
    for bad in [(a, b, c, 256, 256, 64, 4), (a, b, c, 256, 256, 64, -1), (a, b, c, 0, 256, 64, 0),
                (a, b, c, 256, 0, 64, 0), (a, b, c, 256, 256, 0, 0), (a, b, c, -128, 256, 64, 0),
                (0, b, c, 256, 256, 64, 0), (a, 0, c, 256, 256, 64, 0), (a, b, 0, 256, 256, 64, 0),
                (a + 1, b, c, 256, 256, 64, 0), (a, b, c + 1, 8, 8, 8, 0),
                (a, b, c, 64 * 1024, 64 * 1024 + 1, 1, 1)]:
        assert ok(*bad) == xs.kXSchedErrorInvalidValue, bad


def test_enum_values_are_the_wire_values():
    text = open(os.path.join(INC, "types.h")).read()
    want = {"kXSchedSuccess": 0, "kXSchedErrorNotFound": 3, "kXSchedErrorNotSupported": 5,
            "kXSchedErrorUnknown": 999, "kPreemptLevelBlock": 1, "kPreemptLevelDeactivate": 2,
            "kPreemptLevelInterrupt": 3, "kQueueStateIdle": 1, "kQueueStateReady": 2,
            "kQueueSuspendFlagSyncHwQueue": 0x0001, "kQueueSuspendFlagWaitAll": 0x0002,
            "kQueueSuspendFlagWaitIdle": 0x0004, "kQueueResumeFlagDropCommands": 0x0001,
            "kSchedulerLocal": 2, "kSchedulerGlobal": 3, "kPolicyHighestPriorityFirst": 1,
            "kPolicyLaxity": 8, "kPolicyMultiLevelFeedbackQueue": 11, "kPlatformHIP": 4,
            "kDeviceTypeGPU": 2}
    for name, val in want.items():
        m = re.search(name + r"\s*=\s*(0x[0-9a-fA-F]+|\d+)", text)
        assert m and int(m.group(1), 0) == val, name
    assert "#define PRIORITY_NO_EXECUTE -256" in text and "#define PRIORITY_MAX         255" in text


def test_argument_errors(xs):
    p, h = xs.preempt(), xs.halhost()
    xq = c_uint64()
    assert p.XQueueCreate(None, 1, 1, 0) == xs.kXSchedErrorInvalidValue
    assert p.XQueueCreate(byref(xq), 0xDEAD, 1, 0) == xs.kXSchedErrorNotFound
    hwq = xs.host_queue_create()
    assert p.XQueueCreate(byref(xq), hwq, 0, 0) == xs.kXSchedErrorInvalidValue
    assert p.XQueueCreate(byref(xq), hwq, 4, 0) == xs.kXSchedErrorInvalidValue
    assert p.XQueueCreate(byref(xq), hwq, 1, xs.kQueueCreateFlagBlockingSubmit) == xs.kXSchedErrorNotSupported
    assert p.XQueueCreate(byref(xq), hwq, 1, 0) == xs.kXSchedSuccess
    again = c_uint64()
    assert p.XQueueCreate(byref(again), hwq, 1, 0) == xs.kXSchedSuccess and again.value == xq.value
    got = c_uint64()
    assert p.XQueueGet(byref(got), hwq) == xs.kXSchedSuccess and got.value == xq.value
    assert p.XQueueGet(byref(got), 0xBEEF) == xs.kXSchedErrorNotFound
    assert p.HwQueueDestroy(hwq) == xs.kXSchedErrorNotAllowed          # XQueue still attached
    for fn, args in [(p.XQueueWaitAll, ()), (p.XQueueSuspend, (0,)), (p.XQueueResume, (0,)),
                     (p.XQueueSetLaunchConfig, (8, 4)), (p.XQueueSubmit, (1,))]:
        assert fn(0x1234, *args) == xs.kXSchedErrorNotFound
    assert p.XQueueQuery(xq.value, None) == xs.kXSchedErrorInvalidValue
    assert p.XQueueProfileHwCommandCount(xq.value, None) == xs.kXSchedErrorInvalidValue
    assert p.XQueueSetPreemptLevel(xq.value, 0) == xs.kXSchedErrorInvalidValue
    assert p.XQueueSubmit(xq.value, 0x999) == xs.kXSchedErrorNotFound
    assert p.XHintPriority(0x1234, 1) == xs.kXSchedErrorNotFound
    assert p.XHintLaxity(0x1234, 10, 0, 1) == xs.kXSchedErrorNotFound
    assert p.XHintSetScheduler(0, 1) == xs.kXSchedErrorInvalidValue
    assert p.HwCommandDestroy(0x777) == xs.kXSchedErrorNotFound
    assert p.XQueueDestroy(xq.value) == xs.kXSchedSuccess
    assert p.XQueueDestroy(xq.value) == xs.kXSchedErrorNotFound
    assert p.HwQueueDestroy(hwq) == xs.kXSchedSuccess
    assert p.HwQueueDestroy(hwq) == xs.kXSchedErrorNotFound


def test_submit_moves_ownership_and_counts(xs):
    p, h = xs.preempt(), xs.halhost()
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    a = np.ones(1000, np.float32); b = np.full(1000, 2, np.float32); c = np.zeros(1000, np.float32)
    cmd = c_uint64()
    xs.check(h.HostVecAddCommandCreate(byref(cmd), a.ctypes.data, b.ctypes.data, c.ctypes.data, 1000, 0))
    xs.check(p.XQueueSubmit(xq, cmd.value))
    assert p.XQueueSubmit(xq, cmd.value) == xs.kXSchedErrorNotFound   # handle is gone after submit
    assert p.XQueueWait(xq, cmd.value) == xs.kXSchedErrorNotFound     # (reference xqueue.cpp:338-342)
    xs.check(p.XQueueWaitAll(xq))
    assert np.all(c == 3)
    n = c_int64()
    xs.check(p.XQueueProfileHwCommandCount(xq, byref(n)))
    assert n.value == 1
    # The queue turns idle when its launch thread comes back for the next command and finds
    # none, which is a moment after the wait-all command has completed and WaitAll has returned
    # (as in the reference: command_buffer.cpp:39-60).
    import time
    st = c_int()
    deadline = time.time() + 2.0
    while True:
        xs.check(p.XQueueQuery(xq, byref(st)))
        if st.value == xs.kQueueStateIdle or time.time() > deadline:
            break
        time.sleep(0.0005)
    assert st.value == xs.kQueueStateIdle
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_callback_command_runs_on_launch(xs):
    p = xs.preempt()
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    seen = []

    @xs.LaunchCallback
    def cb(q, data):
        seen.append(q)
        return 0

    cmd = c_uint64()
    xs.check(p.HwCommandCreateCallback(byref(cmd), cb, None))
    xs.check(p.XQueueSubmit(xq, cmd.value))
    xs.check(p.XQueueWaitAll(xq))
    assert seen == [hwq]
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_known_answer_chained_adds(xs):
    """The reference's own device test: k chained additions of ones yield k everywhere
    (platforms/example/test/src/vecadd.cpp:91-102), 1024 commands of 4096 elements."""
    p, h = xs.preempt(), xs.halhost()
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XQueueSetLaunchConfig(xq, 8, 4))
    n, k = 4096, 1024
    ones = np.ones(n, np.float32); acc = np.zeros(n, np.float32)
    for _ in range(k):
        cmd = c_uint64()
        xs.check(h.HostVecAddCommandCreate(byref(cmd), acc.ctypes.data, ones.ctypes.data, acc.ctypes.data, n, 0))
        xs.check(p.XQueueSubmit(xq, cmd.value))
    xs.check(p.XQueueWaitAll(xq))
    assert np.all(acc == k)
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def host_stats(xs, hwq):
    e, s, r = c_uint64(), c_uint64(), c_uint64()
    xs.check(xs.halhost().HostQueueGetStats(hwq, byref(e), byref(s), byref(r)))
    return e.value, s.value, r.value


def test_host_level2_exactly_once_under_churn(xs):
    """Level 2 on the host adapter: in-place AXPY commands flushed and replayed many times
    must equal the oracle bit for bit, and every work-group must have run exactly once."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq, xs.kPreemptLevelDeactivate)
    xs.check(p.XQueueSetLaunchConfig(xq, 4, 2))
    n, times = 1 << 20, 40
    x = oracle.fill_uniform(1, 1, 0, n); y0 = oracle.fill_uniform(1, 2, 0, n); y = y0.copy()
    stop = threading.Event()

    def churn():
        while not stop.is_set():
            time.sleep(0.0005)
            p.XQueueSuspend(xq, 0)
            time.sleep(0.0002)
            p.XQueueResume(xq, 0)

    t = threading.Thread(target=churn); t.start()
    for _ in range(times):
        cmd = c_uint64()
        xs.check(h.HostAxpyCommandCreate(byref(cmd), 0.3337, x.ctypes.data, y.ctypes.data, n, 1))
        xs.check(p.XQueueSubmit(xq, cmd.value))
    time.sleep(0.02)
    stop.set(); t.join()
    xs.check(p.XQueueWaitAll(xq))
    executed, skipped, replays = host_stats(xs, hwq)
    want = oracle.axpy(np.float32(0.3337), x, y0, times)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert executed == times * (n // 16384)
    assert replays > 0 and skipped > 0, "the churn never flushed a kernel: test too gentle"
    xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hwq))


def test_cpu_configuration_two_queues_hpf(xs):
    """The CPU plumbing configuration on the host adapter: two XQueues, level 1, HPF, threshold 8
    and batch 4. Background: 1000 fp32 vector additions of 2^20 elements (uniform [-1,1),
    seed 0); foreground: one 2^16-element addition every 10 ms, higher priority. Outputs
    must be bit-exact; the foreground latency is printed."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, xs.kPolicyHighestPriorityFirst))
    hw_bg, hw_fg = xs.host_queue_create(), xs.host_queue_create()
    xq_bg, xq_fg = xs.xqueue_create(hw_bg), xs.xqueue_create(hw_fg)
    for xq, prio in ((xq_bg, 1), (xq_fg, 2)):
        xs.check(p.XQueueSetLaunchConfig(xq, 8, 4))
        xs.check(p.XHintPriority(xq, prio))
    n_bg, n_fg = 1 << 20, 1 << 16
    a = oracle.fill_uniform(0, 1, 0, n_bg); b = oracle.fill_uniform(0, 2, 0, n_bg)
    c = np.zeros(n_bg, np.float32); fc = np.zeros(n_fg, np.float32)

    def bg():
        for _ in range(1000):
            cmd = c_uint64()
            xs.check(h.HostVecAddCommandCreate(byref(cmd), a.ctypes.data, b.ctypes.data, c.ctypes.data, n_bg, 0))
            xs.check(p.XQueueSubmit(xq_bg, cmd.value))
        xs.check(p.XQueueWaitAll(xq_bg))

    t = threading.Thread(target=bg); t.start()
    lat = []
    while t.is_alive() and len(lat) < 200:
        t0 = time.perf_counter()
        cmd = c_uint64()
        xs.check(h.HostVecAddCommandCreate(byref(cmd), a.ctypes.data, b.ctypes.data, fc.ctypes.data, n_fg, 0))
        xs.check(p.XQueueSubmit(xq_fg, cmd.value))
        xs.check(p.XQueueWaitAll(xq_fg))
        lat.append((time.perf_counter() - t0) * 1e6)
        time.sleep(0.01)
    t.join()
    assert np.array_equal(c.view(np.uint32), oracle.vecadd(a, b).view(np.uint32))
    assert np.array_equal(fc.view(np.uint32), oracle.vecadd(a[:n_fg], b[:n_fg]).view(np.uint32))
    print("fg latency us: p50 %.0f p99 %.0f over %d samples" %
          (oracle.percentile(lat, 0.5), oracle.percentile(lat, 0.99), len(lat)))
    for xq, hw in ((xq_bg, hw_bg), (xq_fg, hw_fg)):
        xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hw))
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))


def test_hpf_suspends_the_lower_priority_queue(xs):
    """While the high-priority queue has work, the local scheduler keeps the low-priority
    queue from launching: its backlog only moves once the high one is idle."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, xs.kPolicyHighestPriorityFirst))
    hw_lo, hw_hi = xs.host_queue_create(), xs.host_queue_create()
    xq_lo, xq_hi = xs.xqueue_create(hw_lo), xs.xqueue_create(hw_hi)
    xs.check(p.XHintPriority(xq_lo, 1)); xs.check(p.XHintPriority(xq_hi, 5))
    for xq in (xq_lo, xq_hi):
        xs.check(p.XQueueSetLaunchConfig(xq, 2, 1))
    gate = threading.Event()

    @xs.HostKernelFn
    def slow(arg, wg, n_wg):
        gate.wait(5)

    @xs.HostKernelFn
    def quick(arg, wg, n_wg):
        pass

    cmd = c_uint64()
    xs.check(h.HostKernelCommandCreate(byref(cmd), slow, None, 1, 0))
    xs.check(p.XQueueSubmit(xq_hi, cmd.value))          # high queue is now busy
    time.sleep(0.05)                                     # let the scheduler react
    for _ in range(10):
        xs.check(h.HostKernelCommandCreate(byref(cmd), quick, None, 1, 0))
        xs.check(p.XQueueSubmit(xq_lo, cmd.value))
    time.sleep(0.1)
    executed_while_blocked, _, _ = host_stats(xs, hw_lo)
    gate.set()
    xs.check(p.XQueueWaitAll(xq_hi)); xs.check(p.XQueueWaitAll(xq_lo))
    executed_after, _, _ = host_stats(xs, hw_lo)
    assert executed_while_blocked == 0, "low-priority queue ran while the high-priority one had work"
    assert executed_after == 10
    for xq, hw in ((xq_lo, hw_lo), (xq_hi, hw_hi)):
        xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hw))
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))


def test_laxity_policy_promotes_after_the_laxity(xs):
    """LAX: a queue hinted (laxity 150 ms, lax priority -5, critical priority 9) next to a
    busy default-priority queue is held back at first and released once its laxity is used
    up - by the policy's own timer, without any further event."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, xs.kPolicyLaxity))
    hw_a, hw_b = xs.host_queue_create(), xs.host_queue_create()
    xq_a, xq_b = xs.xqueue_create(hw_a), xs.xqueue_create(hw_b)
    xs.check(p.XHintLaxity(xq_b, 150000, -5, 9))
    gate = threading.Event()

    @xs.HostKernelFn
    def slow(arg, wg, n_wg):
        gate.wait(5)

    @xs.HostKernelFn
    def quick(arg, wg, n_wg):
        pass

    cmd = c_uint64()
    xs.check(h.HostKernelCommandCreate(byref(cmd), slow, None, 1, 0))
    xs.check(p.XQueueSubmit(xq_a, cmd.value))            # queue A (priority 0) busy
    time.sleep(0.03)
    xs.check(h.HostKernelCommandCreate(byref(cmd), quick, None, 1, 0))
    xs.check(p.XQueueSubmit(xq_b, cmd.value))            # B ready at lax priority -5 < 0
    time.sleep(0.05)
    early, _, _ = host_stats(xs, hw_b)
    time.sleep(0.25)                                     # laxity expires -> priority 9 > 0
    late, _, _ = host_stats(xs, hw_b)
    gate.set()
    xs.check(p.XQueueWaitAll(xq_a)); xs.check(p.XQueueWaitAll(xq_b))
    assert early == 0 and late == 1
    for xq, hw in ((xq_a, hw_a), (xq_b, hw_b)):
        xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hw))
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))


def test_every_policy_with_a_class_can_be_selected(xs):
    """The reference names eleven policies and implements ten (the strict process
    partition has an enum value and a name only); so does this build."""
    p = xs.preempt()
    for policy in (1, 2, 3, 4, 5, 7, 8, 9, 10, 11):
        assert p.XHintSetScheduler(xs.kSchedulerLocal, policy) == xs.kXSchedSuccess, policy
    for policy in (0, 6, 12, -1):
        assert p.XHintSetScheduler(xs.kSchedulerLocal, policy) == xs.kXSchedErrorInvalidValue, policy
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))


def test_kedf_runs_the_earliest_deadline_first(xs):
    """KEDF with k = 1 through the C API: of two queues with work, the one whose deadline
    (ready time + XHintDeadline) comes first runs; the other's backlog moves only when the
    first is idle. With XHintKDeadline(2) both run."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, 7))
    hw_a, hw_b = xs.host_queue_create(), xs.host_queue_create()
    xq_a, xq_b = xs.xqueue_create(hw_a), xs.xqueue_create(hw_b)
    xs.check(p.XHintDeadline(xq_a, 1_000))            # 1 ms after it becomes ready
    xs.check(p.XHintDeadline(xq_b, 10_000_000))       # 10 s
    gate = threading.Event()

    @xs.HostKernelFn
    def slow(arg, wg, n_wg):
        gate.wait(5)

    @xs.HostKernelFn
    def quick(arg, wg, n_wg):
        pass

    cmd = c_uint64()
    xs.check(h.HostKernelCommandCreate(byref(cmd), slow, None, 1, 0))
    xs.check(p.XQueueSubmit(xq_a, cmd.value))
    time.sleep(0.05)
    for _ in range(4):
        xs.check(h.HostKernelCommandCreate(byref(cmd), quick, None, 1, 0))
        xs.check(p.XQueueSubmit(xq_b, cmd.value))
    time.sleep(0.1)
    held, _, _ = host_stats(xs, hw_b)
    xs.check(p.XHintKDeadline(2))
    time.sleep(0.1)
    released, _, _ = host_stats(xs, hw_b)
    gate.set()
    xs.check(p.XQueueWaitAll(xq_a)); xs.check(p.XQueueWaitAll(xq_b))
    assert held == 0, "the later deadline ran while the earlier one had work"
    assert released == 4
    for xq, hw in ((xq_a, hw_a), (xq_b, hw_b)):
        xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hw))
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))


def test_utilization_partition_takes_turns(xs):
    """UP through the C API: two queues with equal shares of a 40 ms timeslice, both with a
    long backlog of 2 ms commands. At any time only one of them runs; over 400 ms both make
    progress and neither gets more than about three quarters of the work done."""
    p, h = xs.preempt(), xs.halhost()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, 4))
    hw_a, hw_b = xs.host_queue_create(), xs.host_queue_create()
    xq_a, xq_b = xs.xqueue_create(hw_a), xs.xqueue_create(hw_b)
    for xq in (xq_a, xq_b):
        xs.check(p.XQueueSetLaunchConfig(xq, 2, 1))
        xs.check(p.XHintUtilization(xq, 50))
    xs.check(p.XHintTimeslice(40_000))

    @xs.HostKernelFn
    def work(arg, wg, n_wg):
        time.sleep(0.002)

    cmd = c_uint64()
    for _ in range(400):
        for xq in (xq_a, xq_b):
            xs.check(h.HostKernelCommandCreate(byref(cmd), work, None, 1, 0))
            xs.check(p.XQueueSubmit(xq, cmd.value))
    time.sleep(0.4)
    done_a, _, _ = host_stats(xs, hw_a)
    done_b, _, _ = host_stats(xs, hw_b)
    # drop what is left instead of waiting another second for it
    for xq in (xq_a, xq_b):
        xs.check(p.XQueueSuspend(xq, 0)); xs.check(p.XQueueResume(xq, 1))
        xs.check(p.XQueueWaitAll(xq))
    total = done_a + done_b
    print("UP: a %d b %d" % (done_a, done_b))
    assert total > 60
    assert 0.25 < done_a / total < 0.75
    for xq, hw in ((xq_a, hw_a), (xq_b, hw_b)):
        xs.check(p.XQueueDestroy(xq)); xs.check(p.HwQueueDestroy(hw))
    xs.check(p.XHintSetScheduler(xs.kSchedulerAppManaged, 0))
