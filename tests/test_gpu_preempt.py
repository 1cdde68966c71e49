"""GPU: Level-2 deactivate / reactivate. Results of runs that are suspended and
resumed many times must be bit-identical to uninterrupted runs (and, for the integer
and fp32 kernels, to the CPU oracle)."""
import random
import threading
import time
from ctypes import byref, c_int, c_uint64

import numpy as np
import pytest

import oracle
from test_gpu_kernels import Queue, axpy_cmd, gemm_cmd, hist_cmd

pytestmark = pytest.mark.gpu


def hip_stats(xs, hwq):
    out = (c_uint64 * 8)()
    xs.check(xs.halhip().HipQueueGetStats(hwq, out))
    return list(out)


def churn(xs, q, stop, seed, flags=0):
    """Suspend / resume the queue at random moments until told to stop."""
    rnd = random.Random(seed)
    p = xs.preempt()
    cycles = 0
    while not stop.is_set():
        # the first suspension comes early: a queue is only deactivated on the device when it
        # has work in flight, and the tests want to see that happen
        time.sleep(rnd.uniform(0.0002, 0.002) if cycles else 0.0002)
        xs.check(p.XQueueSuspend(q.xq, flags))
        time.sleep(rnd.uniform(0.0001, 0.001))
        xs.check(p.XQueueResume(q.xq, 0))
        cycles += 1
    return cycles


# The grid of a guarded AXPY (long-lived waves with several steps of loads in flight, or one
# wave per chunk with the guard at entry) and the steps of 1024 elements in a chunk: with
# more than one step a chunk that has begun must be finished, or the replay would apply
# its first steps twice.
@pytest.mark.parametrize("grid,steps", [("waves", 1), ("waves", 2), ("waves", 7), ("chunk", 1), ("chunk", 4)])
@pytest.mark.parametrize("suspend_flags", [0, 1])  # 1 = kQueueSuspendFlagSyncHwQueue
def test_axpy_preempt_resume_bit_exact(xs, gpu, monkeypatch, suspend_flags, grid, steps):
    torch = gpu
    guard = 1
    monkeypatch.setenv("XSCHED_HIP_AXPY_GRID", grid)
    monkeypatch.setenv("XSCHED_HIP_AXPY_STEPS", str(steps))
    n, times = (1 << 24) + 5, 60
    print(f"case axpy-preempt n={n} times={times} flags={suspend_flags} grid={grid} steps={steps}", flush=True)
    x_h = oracle.fill_uniform(5, 1, 0, n)
    y_h = oracle.fill_uniform(5, 2, 0, n)
    x = torch.from_numpy(x_h).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, level=2, threshold=4, batch=2)
    stop = threading.Event()
    result = {}
    t = threading.Thread(target=lambda: result.setdefault("cycles", churn(xs, q, stop, 1, suspend_flags)))
    t.start()
    for _ in range(times):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, guard))
    # Keep churning while the queue drains, then stop and let it finish.
    time.sleep(0.05)
    stop.set()
    t.join()
    q.wait()
    st = hip_stats(xs, q.hwq)
    got = y.cpu().numpy()
    q.close()
    want = oracle.axpy(0.5, x_h, y_h, times)
    print("stats", st, "cycles", result.get("cycles"), flush=True)
    assert st[2] > 0 and st[3] > 0, "no deactivation happened: the test did not exercise level 2"
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("layout", ["sweep", "merge"])
def test_histogram_preempt_resume_bit_exact(xs, gpu, monkeypatch, layout):
    """Both ways the histogram merges its per-group counts (see hist_layout in
    test_gpu_kernels.py); in the second one a flushed launch leaves partial histograms in
    the queue's scratch buffer for the replay."""
    torch = gpu
    monkeypatch.setenv("XSCHED_HIP_HIST_MERGE_MIN_KEYS", "1" if layout == "merge" else str(1 << 40))
    n, n_bins, times = 1 << 24, 65536, 40
    print(f"case hist-preempt {layout} n={n} times={times}", flush=True)
    table = oracle.zipf_table(n_bins)
    keys_h = oracle.fill_zipf(9, 1, 0, n, table, n_bins)
    keys = torch.from_numpy(keys_h).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, level=2, threshold=4, batch=2)
    stop = threading.Event()
    t = threading.Thread(target=churn, args=(xs, q, stop, 2))
    t.start()
    # A command takes some 15 us: rounds of `times` commands until the suspensions have caught
    # the queue with work in flight a few times (one that finds nothing in flight deactivates
    # nothing), at most a hundred rounds.
    rounds = 0
    while rounds < 100:
        for _ in range(times):
            q.submit(hist_cmd(xs, keys, n, bins, n_bins, 1))
        rounds += 1
        if hip_stats(xs, q.hwq)[2] >= 3:
            break
    times *= rounds
    time.sleep(0.05)
    stop.set()
    t.join()
    q.wait()
    st = hip_stats(xs, q.hwq)
    got = bins.cpu().numpy().view(np.uint32)
    q.close()
    one = oracle.histogram(keys_h, n_bins).astype(np.uint64)
    print("stats", st, "rounds", rounds, flush=True)
    assert st[2] > 0
    # The bins are 32-bit and add with wrap-around: after enough rounds the hottest bin of a
    # Zipf key set passes 2^32, in the device's counters as in the oracle's.
    assert np.array_equal(got.astype(np.uint64), (one * times) & 0xFFFFFFFF)
    assert int(got.sum()) % (1 << 32) == (times * n) % (1 << 32)


@pytest.mark.parametrize("on_kernel", [1, 0])
def test_marker_on_the_kernel_or_recorded_behind_it(xs, gpu, on_kernel):
    """A queue's kernel commands carry their markers as the stop event of their own launch
    (the default) or as events recorded behind them (HipQueueSetMarkerOnKernel(hwq, 0)). Either
    way every command is waited for and the results are the oracle's, also across suspensions
    that flush and replay; with recorded markers the runtime sees the stream idle the moment
    the XQueue is."""
    torch = gpu
    n, times = (1 << 22) + 3, 60
    print(f"case marker-mode on_kernel={on_kernel} n={n} times={times}", flush=True)
    x_h = oracle.fill_uniform(6, 1, 0, n)
    y_h = oracle.fill_uniform(6, 2, 0, n)
    x = torch.from_numpy(x_h).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    n_bins, nk = 4096, 1 << 20
    keys_h = oracle.fill_zipf(6, 3, 0, nk, oracle.zipf_table(n_bins), n_bins)
    keys = torch.from_numpy(keys_h).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, level=2, threshold=2, batch=1)   # every command carries a marker
    xs.check(xs.halhip().HipQueueSetMarkerOnKernel(q.hwq, on_kernel))
    idle_at_once = 0
    for i in range(times):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
        q.submit(hist_cmd(xs, keys, nk, bins, n_bins, 1))
        if i % 10 == 9:
            q.wait()
            idle_at_once += 1 if q.stream.query() else 0
    stop = threading.Event()
    t = threading.Thread(target=churn, args=(xs, q, stop, 3))
    t.start()
    for i in range(times):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
        q.submit(hist_cmd(xs, keys, nk, bins, n_bins, 1))
    time.sleep(0.02)
    stop.set()
    t.join()
    q.wait()
    st = hip_stats(xs, q.hwq)
    got_y = y.cpu().numpy()
    got_bins = bins.cpu().numpy().view(np.uint32)
    q.close()
    print("stats", st, "stream idle at once", idle_at_once, "of", times // 10, flush=True)
    want = oracle.axpy(0.5, x_h, y_h, 2 * times)
    assert np.array_equal(got_y.view(np.uint32), want.view(np.uint32))
    one = oracle.histogram(keys_h, n_bins).astype(np.uint64)
    assert np.array_equal(got_bins.astype(np.uint64), (one * 2 * times) & 0xFFFFFFFF)
    if not on_kernel:
        # (one miss allowed: the answer is the runtime's, asked once without waiting)
        assert idle_at_once >= times // 10 - 1


def test_commands_waiting_in_the_xqueue_hold_no_device_memory(xs, gpu):
    """A burst of guarded histogram commands far deeper than the in-flight window: the
    queue's pools (partial-histogram buffers, progress maps) grow with what is launched and
    not yet destroyed, not with what waits in the XQueue."""
    torch = gpu
    n, n_bins, burst = 1 << 24, 65536, 96
    print(f"case pool-growth n={n} burst={burst}", flush=True)
    keys_h = oracle.fill_zipf(13, 1, 0, n, oracle.zipf_table(n_bins), n_bins)
    keys = torch.from_numpy(keys_h).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, level=2, threshold=2, batch=1)
    for _ in range(burst):
        q.submit(hist_cmd(xs, keys, n, bins, n_bins, 1))
    q.wait()
    pools = (c_uint64 * 4)()
    xs.check(xs.halhip().HipQueueGetPoolStats(q.hwq, pools))
    got = bins.cpu().numpy().view(np.uint32)
    q.close()
    print("pools", list(pools), flush=True)
    # threshold 2 in flight, plus the commands whose completion the queue has not yet seen,
    # plus the one kept free ahead of the next launch
    assert 1 <= pools[0] <= 8, "scratch buffers grew with the submission burst"
    assert pools[2] <= 16, "progress maps grew with the submission burst"
    assert pools[3] == 0
    one = oracle.histogram(keys_h, n_bins).astype(np.uint64)
    assert np.array_equal(got.astype(np.uint64), (one * burst) & 0xFFFFFFFF)


@pytest.mark.parametrize("tile,shape", [(128, (2048, 2048, 2048)), (256, (2048, 2048, 2048)), (64, (1000, 1999, 1030)),
                                        (128, (1960, 2048, 1024))])
def test_gemm_preempt_resume_matches_uninterrupted(xs, gpu, monkeypatch, tile, shape):
    """Both tile sizes of the fast kernel, the any-shape kernel on a shape only it takes, and a
    command whose rows are split between the two."""
    torch = gpu
    monkeypatch.setenv("XSCHED_HIP_GEMM_TILE", str(tile))
    M, N, K = shape
    times = 12
    print(f"case gemm-preempt {M}x{N}x{K} tile={tile} times={times} x 10", flush=True)
    a_bits = oracle.fill_normal_bf16(13, 1, 0, M * K)
    b_bits = oracle.fill_normal_bf16(13, 2, 0, K * N)
    a = torch.from_numpy(a_bits.view(np.int16).reshape(M, K)).cuda()
    b = torch.from_numpy(b_bits.view(np.int16).reshape(K, N)).cuda()
    c_ref = torch.zeros(M, N, dtype=torch.int16, device="cuda")
    q1 = Queue(xs, torch, level=1)
    q1.submit(gemm_cmd(xs, a, b, c_ref, M, N, K, 0))
    q1.wait()
    q1.close()

    outs = [torch.zeros(M, N, dtype=torch.int16, device="cuda") for _ in range(times)]
    q = Queue(xs, torch, level=2, threshold=4, batch=2)
    stop = threading.Event()
    t = threading.Thread(target=churn, args=(xs, q, stop, 3))
    t.start()
    for _ in range(10):      # ~2 ms of work in all: long enough for suspensions to land in it
        for c in outs:
            q.submit(gemm_cmd(xs, a, b, c, M, N, K, 1))
    time.sleep(0.02)
    stop.set()
    t.join()
    q.wait()
    st = hip_stats(xs, q.hwq)
    print("stats", st, flush=True)
    q.close()
    assert st[2] > 0
    for c in outs:
        assert torch.equal(c, c_ref)


def test_resume_with_drop_commands(xs, gpu):
    """After a suspend, resuming with DropCommands completes everything submitted so
    far without executing what had not started (reference async_xqueue.cpp:137-149)."""
    torch = gpu
    n = 1 << 22
    x = torch.ones(n, device="cuda")
    y = torch.zeros(n, device="cuda")
    q = Queue(xs, torch, level=2, threshold=2, batch=1)
    p = xs.preempt()
    xs.check(p.XQueueSuspend(q.xq, 0))
    for _ in range(20):
        q.submit(axpy_cmd(xs, 1.0, x, y, n, 1))
    xs.check(p.XQueueResume(q.xq, 1))  # kQueueResumeFlagDropCommands
    q.wait()
    state = c_int()
    deadline = time.time() + 2.0   # idle a moment after the wait has returned
    while True:
        xs.check(p.XQueueQuery(q.xq, byref(state)))
        if state.value == xs.kQueueStateIdle or time.time() > deadline:
            break
        time.sleep(0.0005)
    assert state.value == xs.kQueueStateIdle
    got = y.cpu().numpy()
    assert np.all(got == 0.0)
    # The queue is usable afterwards.
    q.submit(axpy_cmd(xs, 1.0, x, y, n, 1))
    q.wait()
    assert np.all(y.cpu().numpy() == 1.0)
    q.close()


def test_dynamic_level_switch(xs, gpu):
    """The reference HIP adapter refuses level changes (hip_queue.h:25); this one
    moves between 1 and 2 and refuses 3."""
    torch = gpu
    q = Queue(xs, torch, level=1)
    p = xs.preempt()
    assert p.XQueueSetPreemptLevel(q.xq, xs.kPreemptLevelDeactivate) == xs.kXSchedSuccess
    assert p.XQueueSetPreemptLevel(q.xq, xs.kPreemptLevelBlock) == xs.kXSchedSuccess
    assert p.XQueueSetPreemptLevel(q.xq, 0) == xs.kXSchedErrorInvalidValue
    # Level 3 is above the adapter's maximum: accepted call, level unchanged (warning).
    assert p.XQueueSetPreemptLevel(q.xq, xs.kPreemptLevelInterrupt) == xs.kXSchedSuccess
    n = 4096
    x = torch.ones(n, device="cuda"); y = torch.zeros(n, device="cuda")
    q.submit(axpy_cmd(xs, 2.0, x, y, n, 1))
    q.wait()
    assert np.all(y.cpu().numpy() == 2.0)
    q.close()


def test_null_stream_and_bad_arguments(xs, gpu):
    h = xs.halhip()
    hwq = c_uint64()
    assert h.HipQueueCreate(byref(hwq), None) == xs.kXSchedErrorNotSupported
    assert h.HipQueueCreate(None, 1) == xs.kXSchedErrorInvalidValue
    cmd = c_uint64()
    assert h.HipGemmBf16CommandCreate(byref(cmd), 16, 16, 16, 100, 0, 64, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipGemmBf16CommandCreate(byref(cmd), 17, 16, 16, 100, 256, 64, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipHistogramCommandCreate(byref(cmd), 16, 4, 16, 70000, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipAxpyCommandCreate(byref(cmd), 1.0, None, None, 4, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipAxpyCommandCreate(byref(cmd), 1.0, 16, 16, 4, 4) == xs.kXSchedErrorInvalidValue
    out = (c_uint64 * 8)()
    assert h.HipQueueGetStats(0x1234, out) == xs.kXSchedErrorNotFound
    assert h.HipQueueGetPoolStats(0x1234, out) == xs.kXSchedErrorNotFound
    assert h.HipQueueSetMarkerOnKernel(0x1234, 1) == xs.kXSchedErrorNotFound


def test_cross_queue_wait_on_recorded_event_follows_replays(xs, gpu):
    """Queue B waits for an event-record command of queue A, which runs at level 2 and is
    suspended and resumed all the time: B's kernel, which reads A's output, must see it
    complete, i.e. the wait must follow A's flushes and replays rather than the raw event."""
    import ctypes
    torch = gpu
    hip = ctypes.CDLL("libamdhip64.so")
    event = ctypes.c_void_p()
    assert hip.hipEventCreateWithFlags(byref(event), 2) == 0  # hipEventDisableTiming
    n, times = 1 << 24, 40
    print(f"case cross-queue-wait n={n} times={times}", flush=True)
    xa_h = oracle.fill_uniform(21, 1, 0, n); ya_h = oracle.fill_uniform(21, 2, 0, n)
    yb_h = oracle.fill_uniform(21, 3, 0, n)
    xa = torch.from_numpy(xa_h).cuda(); ya = torch.from_numpy(ya_h.copy()).cuda()
    yb = torch.from_numpy(yb_h.copy()).cuda()
    qa = Queue(xs, torch, level=2, threshold=4, batch=2)
    qb = Queue(xs, torch, level=1)
    h = xs.halhip()

    record, wait = c_uint64(), c_uint64()
    xs.check(h.HipEventRecordCommandCreate(byref(record), event))
    xs.check(h.HipRecordedEventWaitCommandCreate(byref(wait), record.value))
    assert h.HipRecordedEventWaitCommandCreate(byref(c_uint64()), 0x1234) == xs.kXSchedErrorNotFound

    # B first: its launch thread has to wait for a command that is not even submitted yet.
    qb.submit(wait.value)
    qb.submit(axpy_cmd(xs, 1.0, ya, yb, n, 0))          # yb += ya, once A is done
    time.sleep(0.01)
    stop = threading.Event()
    t = threading.Thread(target=churn, args=(xs, qa, stop, 9))
    t.start()
    for _ in range(times):
        qa.submit(axpy_cmd(xs, 0.5, xa, ya, n, 1))
    qa.submit(record.value)
    qb.wait()                                            # returns only after A's work
    stop.set()
    t.join()
    qa.wait()
    st = hip_stats(xs, qa.hwq)
    got_a, got_b = ya.cpu().numpy(), yb.cpu().numpy()
    qa.close(); qb.close()
    assert hip.hipEventDestroy(event) == 0
    want_a = oracle.axpy(0.5, xa_h, ya_h, times)
    want_b = oracle.axpy(1.0, want_a, yb_h, 1)
    print("stats", st, flush=True)
    assert st[2] > 0, "queue A was never deactivated: the test did not exercise level 2"
    assert np.array_equal(got_a.view(np.uint32), want_a.view(np.uint32))
    assert np.array_equal(got_b.view(np.uint32), want_b.view(np.uint32)), "B ran before A had finished"


@pytest.mark.parametrize("kind", ["axpy", "axpy few waves", "histogram", "gemm"])
def test_launches_of_a_flushed_epoch_do_not_run(xs, gpu, kind):
    """The copies of the preempt word are rewritten one after the other, so a work-group of
    a later launch may still read an old copy when an earlier launch has already been
    flushed. What keeps it from running ahead is the queue's "flushed" word: a flushed
    work-group leaves the epoch of its launch there, and no work-group runs under an epoch
    it finds there. The race itself cannot be staged; the test writes the word the way a
    flushed work-group does and checks both halves of the rule: commands of that epoch
    leave memory untouched, a command replayed after a deactivation / reactivation (a new
    epoch) runs."""
    torch = gpu
    print(f"case flushed-epoch {kind}", flush=True)
    q = Queue(xs, torch, level=2, threshold=4, batch=2)
    p = xs.preempt()
    if kind.startswith("axpy"):
        n = (1 << 20) + 3
        x_h = oracle.fill_uniform(3, 0, 0, n)
        y_h = oracle.fill_uniform(3, 1, 0, n)
        x, y = torch.from_numpy(x_h).cuda(), torch.from_numpy(y_h).cuda()
        make = lambda: axpy_cmd(xs, 0.5, x, y, n, 3 if "few" in kind else 1)
        read = lambda: y.cpu().numpy().view(np.uint32)
        before = y_h.view(np.uint32)
        after = oracle.axpy(0.5, x_h, y_h, 1).view(np.uint32)
    elif kind == "histogram":
        n, n_bins = (1 << 20) + 5, 65536
        keys_h = oracle.fill_zipf(4, 1, 0, n, oracle.zipf_table(n_bins), n_bins)
        keys = torch.from_numpy(keys_h).cuda()
        bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
        make = lambda: hist_cmd(xs, keys, n, bins, n_bins, 1)
        read = lambda: bins.cpu().numpy().view(np.uint32)
        before = np.zeros(n_bins, np.uint32)
        after = oracle.histogram(keys_h, n_bins)
    else:
        M = N = K = 512
        a_h = oracle.fill_normal_bf16(5, 0, 0, M * K)
        b_h = oracle.fill_normal_bf16(5, 1, 0, K * N)
        a = torch.from_numpy(a_h.view(np.int16).reshape(M, K)).cuda()
        b = torch.from_numpy(b_h.view(np.int16).reshape(K, N)).cuda()
        c = torch.zeros(M, N, dtype=torch.int16, device="cuda")
        make = lambda: gemm_cmd(xs, a, b, c, M, N, K, 1)
        read = lambda: c.cpu().numpy().view(np.uint16).ravel()
        before = np.zeros(M * N, np.uint16)
        # what an undisturbed queue computes (bit-identical run to run: fixed summation order)
        c2 = torch.zeros(M, N, dtype=torch.int16, device="cuda")
        q2 = Queue(xs, torch, level=2)
        q2.submit(gemm_cmd(xs, a, b, c2, M, N, K, 1))
        q2.wait()
        q2.close()
        after = c2.cpu().numpy().view(np.uint16).ravel()
        assert after.any()

    xs.check(xs.halhip().HipQueueMarkEpochFlushed(q.hwq))
    q.submit(make())
    q.submit(make())
    q.wait()
    untouched = read().copy()
    # A third command of the flushed epoch, suspended while it is still in the queue's window
    # (a queue with nothing in flight is not deactivated on the device at all): the
    # deactivation opens a new epoch, and the reactivation replays the command under it.
    q.submit(make())
    xs.check(p.XQueueSuspend(q.xq, 0))
    xs.check(p.XQueueResume(q.xq, 0))
    q.wait()
    ran = read().copy()
    q.close()
    assert np.array_equal(untouched, before), "a launch of a flushed epoch wrote something"
    assert np.array_equal(ran, after), "a launch of the next epoch did not run exactly once"


def test_first_commands_of_fresh_queues_on_non_blocking_streams_are_applied_once(xs, gpu):
    """A queue's first guarded command gets a progress map in memory that was allocated a
    moment ago. Whatever prepares that memory must be ordered before the command's kernel on
    the queue's own stream: a stream created with hipStreamNonBlocking does not wait for work
    on the null stream (hipMemset on device memory returns before its fill has run, and the
    fills of several queues wait for each other there). Cleared late, a map loses the bytes of
    the first work-groups, and a replay applies those work-groups a second time. Eight fresh
    queues on fresh non-blocking streams start their first commands together, each is
    suspended and resumed while its kernel runs: every element holds exactly one application."""
    import ctypes
    torch = gpu
    hip = ctypes.CDLL("libamdhip64.so")
    n, n_queues, trials = 1 << 24, 8, 4
    print(f"case fresh-queues-first-command n={n} queues={n_queues} trials={trials}", flush=True)
    x_h = oracle.fill_uniform(31, 1, 0, n)
    y_h = oracle.fill_uniform(31, 2, 0, n)
    want = oracle.axpy(0.5, x_h, y_h, 1).view(np.uint32)
    x = torch.from_numpy(x_h).cuda()
    p = xs.preempt()
    replays = 0
    for trial in range(trials):
        ys = [torch.from_numpy(y_h.copy()).cuda() for _ in range(n_queues)]
        torch.cuda.synchronize()
        streams, hwqs, xqs = [], [], []
        for _ in range(n_queues):
            stream = ctypes.c_void_p()
            assert hip.hipStreamCreateWithFlags(byref(stream), 1) == 0   # hipStreamNonBlocking
            streams.append(stream)
            hwqs.append(xs.hip_queue_create(stream.value))
            xqs.append(xs.xqueue_create(hwqs[-1], 2))
        cmds = [axpy_cmd(xs, 0.5, x, y, n, 1) for y in ys]
        for xq, cmd in zip(xqs, cmds):
            xs.check(p.XQueueSubmit(xq, cmd))
        for _ in range(1 + trial % 2):
            for xq in xqs:
                xs.check(p.XQueueSuspend(xq, 0))
            for xq in xqs:
                xs.check(p.XQueueResume(xq, 0))
        for xq in xqs:
            xs.check(p.XQueueWaitAll(xq))
        replays += sum(hip_stats(xs, hwq)[1] for hwq in hwqs)
        got = [y.cpu().numpy().view(np.uint32) for y in ys]
        for xq, hwq, stream in zip(xqs, hwqs, streams):
            xs.check(p.XQueueDestroy(xq))
            xs.check(p.HwQueueDestroy(hwq))
            assert hip.hipStreamDestroy(stream) == 0
        for i, g in enumerate(got):
            assert np.array_equal(g, want), f"trial {trial}, queue {i}: {int((g != want).sum())} elements differ from one application"
    print("replays", replays, flush=True)
    assert replays > 0, "no command was replayed: the test did not exercise level 2"


def test_user_written_guarded_kernel_is_flushed_and_replayed_exactly_once(xs, gpu):
    """A kernel outside the library (tests/user_guarded_kernel.hip: in place, not idempotent)
    with the guard compiled in, submitted through HipGuardedKernelCommandCreate: suspended and
    resumed at random while 120 launches go through a level-2 queue, every work-group of every
    launch must have taken effect exactly once; the same commands at level 1 give the same bits."""
    import ctypes
    import os
    torch = gpu
    lib = ctypes.CDLL(os.path.join(os.path.dirname(xs.__file__), "lib", "libuserguarded.so"))
    lib.UserAffineKernel.restype = ctypes.c_void_p
    func, chunk = lib.UserAffineKernel(), lib.UserAffineChunk()
    n, times = (1 << 24) + 1234, 120
    n_wg = (n + chunk - 1) // chunk
    print(f"case user-guarded n={n} times={times} work-groups={n_wg}", flush=True)
    y_h = oracle.fill_uniform(21, 2, 0, n)

    from xsched_amd.xsched_api import XSched, XResult

    def command(y, b):
        if int(b) % 2:   # through the Python interface ...
            res, cmd = XSched.HipGuardedKernelCommandCreate(
                func, n_wg, (256, 1, 1), [ctypes.c_void_p(y.data_ptr()), ctypes.c_float(b), ctypes.c_size_t(n)])
            assert res == XResult.kXSchedSuccess
            return cmd
        # ... and through the C entry point itself
        y_ptr, b_val, n_val = ctypes.c_void_p(y.data_ptr()), ctypes.c_float(b), ctypes.c_size_t(n)
        args = (ctypes.c_void_p * 3)(ctypes.addressof(y_ptr), ctypes.addressof(b_val), ctypes.addressof(n_val))
        sizes = (ctypes.c_size_t * 3)(8, 4, 8)
        cmd = c_uint64()
        xs.check(xs.halhip().HipGuardedKernelCommandCreate(byref(cmd), func, n_wg, 256, 1, 1, args, sizes, 3, 0))
        return cmd.value

    def run(level, with_churn):
        y = torch.from_numpy(y_h.copy()).cuda()
        q = Queue(xs, torch, level=level, threshold=4, batch=2)
        stop, result = threading.Event(), {}
        t = threading.Thread(target=lambda: result.setdefault("cycles", churn(xs, q, stop, 3)))
        if with_churn:
            t.start()
        for i in range(times):
            q.submit(command(y, 1.0 + (i % 3)))
        if with_churn:
            time.sleep(0.05)
            stop.set()
            t.join()
        q.wait()
        st = hip_stats(xs, q.hwq)
        got = y.cpu().numpy()
        q.close()
        return got, st

    want = y_h.copy()
    for i in range(times):
        want = np.float32(0.5) * want + np.float32(1.0 + (i % 3))   # 0.5 * y is exact: one rounding, as the fma
    plain, _ = run(1, False)
    assert np.array_equal(plain.view(np.uint32), want.view(np.uint32))
    got, st = run(2, True)
    print("stats", st, flush=True)
    assert st[2] > 0 and st[1] > 0, "no launch was flushed and replayed: the test did not exercise level 2"
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # argument checks
    cmd = c_uint64()
    h = xs.halhip()
    assert h.HipGuardedKernelCommandCreate(byref(cmd), func, 0, 256, 1, 1, None, None, 0, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipGuardedKernelCommandCreate(byref(cmd), func, (1 << 18) + 1, 256, 1, 1, None, None, 0, 0) == xs.kXSchedErrorInvalidValue
    assert h.HipGuardedKernelCommandCreate(byref(cmd), None, 4, 256, 1, 1, None, None, 0, 0) == xs.kXSchedErrorInvalidValue


def test_an_event_destroyed_after_its_record_command_completed_is_not_asked_again(xs, gpu):
    """The adapter waits for a queue through the marker of the newest command, and for an
    event-record command that marker is the application's own event. Once the XQueue has seen
    the command complete the application may destroy the event: a later wait for the (empty)
    hardware queue, here the one inside XQueueSuspend(SyncHwQueue), must not touch it."""
    import ctypes
    torch = gpu
    hip = ctypes.CDLL("libamdhip64.so")
    event = ctypes.c_void_p()
    assert hip.hipEventCreateWithFlags(byref(event), 2) == 0  # hipEventDisableTiming
    n = 1 << 20
    print("case destroyed-event", flush=True)
    x = torch.ones(n, device="cuda"); y = torch.zeros(n, device="cuda")
    q = Queue(xs, torch, level=2, threshold=4, batch=2)
    record = c_uint64()
    xs.check(xs.halhip().HipEventRecordCommandCreate(byref(record), event))
    q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
    q.submit(record.value)                   # the newest command on the stream
    q.wait()
    assert hip.hipEventDestroy(event) == 0
    p = xs.preempt()
    for _ in range(3):
        xs.check(p.XQueueSuspend(q.xq, xs.kQueueSuspendFlagSyncHwQueue))
        xs.check(p.XQueueResume(q.xq, 0))
    q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
    q.wait()
    got = y.cpu().numpy()
    q.close()
    assert np.all(got == 1.0)
