"""The other policies on the HIP adapter at level 2 (reference sched/src/policy/{hhpf,chpf,up,
pup,kedf,awf,cfs,mlfq}.cpp): their decisions are pinned against the compiled reference on the
CPU (tests/test_local_sched_parity.py); here they drive real XQueues whose guarded kernels get
deactivated and replayed, and what the kernels compute must still equal the oracle's bits."""
import threading
import time
from ctypes import byref, c_uint64

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

N_BINS = 65536
POLICY_NAMES = {1: "HPF", 2: "HHPF", 3: "CHPF", 4: "UP", 5: "PUP", 7: "KEDF", 8: "LAX", 9: "AWF", 10: "CFS", 11: "MLFQ"}


class Lane:
    """One stream + HwQueue + level-2 XQueue with a guarded AXPY or histogram workload."""

    def __init__(self, xs, torch, kind, n, seed):
        self.xs, self.torch, self.kind, self.n = xs, torch, kind, n
        self.stream = torch.cuda.Stream()
        self.hwq = xs.hip_queue_create(self.stream.cuda_stream)
        self.xq = xs.xqueue_create(self.hwq, xs.kPreemptLevelDeactivate)
        xs.check(xs.preempt().XQueueSetLaunchConfig(self.xq, 2, 1))
        if kind == "axpy":
            self.x_h = oracle.fill_uniform(seed, 1, 0, n)
            self.y_h = oracle.fill_uniform(seed, 2, 0, n)
            self.x = torch.from_numpy(self.x_h).cuda()
            self.y = torch.from_numpy(self.y_h.copy()).cuda()
        else:
            self.keys_h = oracle.fill_zipf(seed, 3, 0, n)
            self.keys = torch.from_numpy(self.keys_h).cuda()
            self.bins = torch.zeros(N_BINS, dtype=torch.int32, device="cuda")
        self.submitted = 0

    def submit(self, count=1):
        h, p = self.xs.halhip(), self.xs.preempt()
        for _ in range(count):
            cmd = c_uint64()
            if self.kind == "axpy":
                self.xs.check(h.HipAxpyCommandCreate(byref(cmd), 0.5, self.x.data_ptr(), self.y.data_ptr(), self.n, 1))
            else:
                self.xs.check(h.HipHistogramCommandCreate(byref(cmd), self.keys.data_ptr(), self.n,
                                                          self.bins.data_ptr(), N_BINS, 1))
            self.xs.check(p.XQueueSubmit(self.xq, cmd.value))
            self.submitted += 1

    def wait(self):
        self.xs.check(self.xs.preempt().XQueueWaitAll(self.xq))

    def stats(self):
        out = (c_uint64 * 8)()
        self.xs.check(self.xs.halhip().HipQueueGetStats(self.hwq, out))
        return list(out)   # launches, replays, deactivations, reactivations, ...

    def check(self, slices=None):
        """Bit-exact against `submitted` oracle applications (AXPY: on slices when given)."""
        if self.kind == "axpy":
            got = self.y.cpu().numpy()
            for first, count in (slices or [(0, self.n)]):
                want = oracle.axpy(0.5, self.x_h[first:first + count], self.y_h[first:first + count], self.submitted)
                assert np.array_equal(got[first:first + count].view(np.uint32), want.view(np.uint32)), (first, count)
        else:
            want = oracle.histogram(self.keys_h, N_BINS).astype(np.uint64) * self.submitted
            got = self.bins.cpu().numpy().view(np.uint32).astype(np.uint64)
            assert np.array_equal(got, want & 0xFFFFFFFF)

    def close(self):
        p = self.xs.preempt()
        self.xs.check(p.XQueueDestroy(self.xq))
        self.xs.check(p.HwQueueDestroy(self.hwq))


@pytest.fixture()
def app_managed_after(xs):
    yield
    xs.check(xs.preempt().XHintSetScheduler(xs.kSchedulerAppManaged, 0))


@pytest.mark.parametrize("policy", sorted(POLICY_NAMES))
def test_every_policy_schedules_level2_queues_to_the_oracles_bits(xs, gpu, app_managed_after, policy):
    """Two level-2 queues with every hint a policy might read, both streaming guarded commands
    at the same time from two threads: whatever the policy decides (and some of them deactivate
    and reactivate the queues many times), both streams finish and their results are exact."""
    torch, p = gpu, xs.preempt()
    print(f"case policy {POLICY_NAMES[policy]}", flush=True)
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, policy))
    a, b = Lane(xs, torch, "axpy", (1 << 22) + 3, 31), Lane(xs, torch, "hist", (1 << 22) + 5, 32)
    try:
        for lane, prio, util, ddl in ((a, 1, 30, 2_000), (b, 2, 70, 500)):
            xs.check(p.XHintPriority(lane.xq, prio))
            xs.check(p.XHintUtilization(lane.xq, util))
            xs.check(p.XHintDeadline(lane.xq, ddl))
            xs.check(p.XHintLaxity(lane.xq, 300, 0, prio))
        xs.check(p.XHintTimeslice(2_000))
        xs.check(p.XHintKDeadline(1))

        def stream(lane):
            for _ in range(10):
                lane.submit(30)
                lane.wait()
        threads = [threading.Thread(target=stream, args=(lane,)) for lane in (a, b)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
            assert not t.is_alive(), "a queue never finished under policy %s" % POLICY_NAMES[policy]
        n_a = a.n
        a.check(slices=[(0, 1 << 16), (n_a - (1 << 16) - 3, (1 << 16) + 3)])
        b.check()
        print("  deactivations a/b: %d / %d, replayed launches %d / %d" %
              (a.stats()[2], b.stats()[2], a.stats()[1], b.stats()[1]), flush=True)
    finally:
        a.close(); b.close()


def test_kedf_lets_the_earliest_deadline_run_first(xs, gpu, app_managed_after):
    """KEDF with k = 1 on the device: while the queue with the 1 ms deadline streams, the queue
    with the 10 s deadline is deactivated; its four short commands, which alone take well under
    a millisecond, complete only once the first queue has gone idle."""
    torch, p = gpu, xs.preempt()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, 7))
    urgent, patient = Lane(xs, torch, "axpy", 1 << 24, 41), Lane(xs, torch, "hist", 1 << 20, 42)
    try:
        xs.check(p.XHintDeadline(urgent.xq, 1_000))
        xs.check(p.XHintDeadline(patient.xq, 10_000_000))
        xs.check(p.XHintKDeadline(1))
        done = {}

        def run(name, lane, count):
            lane.submit(count)
            lane.wait()
            done[name] = time.perf_counter()
        t_urgent = threading.Thread(target=run, args=("urgent", urgent, 2500))   # ~100 ms of AXPY 2^24
        t_urgent.start()
        time.sleep(0.02)
        t0 = time.perf_counter()
        t_patient = threading.Thread(target=run, args=("patient", patient, 4))
        t_patient.start()
        t_urgent.join(timeout=100); t_patient.join(timeout=100)
        assert not t_urgent.is_alive() and not t_patient.is_alive()
        print("  urgent done after %.1f ms, patient after %.1f ms; patient deactivations %d" %
              ((done["urgent"] - t0) * 1e3, (done["patient"] - t0) * 1e3, patient.stats()[2]), flush=True)
        assert done["patient"] >= done["urgent"] - 2e-3, "the later deadline finished while the earlier one had work"
        # (the patient queue was suspended while it had nothing in flight: its commands waited
        # in its ring, and a queue like that is not deactivated on the device at all)
        urgent.check(slices=[(0, 4096), ((1 << 23) + 8, 4096), ((1 << 24) - 4096, 4096)])
        patient.check()
    finally:
        urgent.close(); patient.close()


def test_utilization_partition_shares_the_device_in_slices(xs, gpu, app_managed_after):
    """UP with equal shares of a 10 ms timeslice: two queues with long backlogs of guarded AXPY
    commands take turns (each is deactivated and reactivated many times), both advance, and
    neither gets much more than its share."""
    torch, p = gpu, xs.preempt()
    xs.check(p.XHintSetScheduler(xs.kSchedulerLocal, 4))
    a, b = Lane(xs, torch, "axpy", 1 << 25, 51), Lane(xs, torch, "axpy", 1 << 25, 52)
    try:
        for lane in (a, b):
            xs.check(p.XHintUtilization(lane.xq, 50))
        xs.check(p.XHintTimeslice(10_000))
        count = 1500                       # ~70 us each alone: ~100 ms per queue, ~200 ms together
        threads = [threading.Thread(target=lambda lane=lane: (lane.submit(count), lane.wait())) for lane in (a, b)]
        for t in threads:
            t.start()
        time.sleep(0.1)
        mid_a, mid_b = a.stats()[0] - a.stats()[1], b.stats()[0] - b.stats()[1]   # first launches so far
        for t in threads:
            t.join(timeout=100)
            assert not t.is_alive()
        print("  after 100 ms: a launched %d, b launched %d; deactivations %d / %d" %
              (mid_a, mid_b, a.stats()[2], b.stats()[2]), flush=True)
        assert mid_a > 50 and mid_b > 50, "one queue was starved"
        assert 0.2 < mid_a / (mid_a + mid_b) < 0.8
        assert a.stats()[2] >= 3 and b.stats()[2] >= 3
        slices = [(0, 4096), ((1 << 24) + 12, 4096), ((1 << 25) - 4096, 4096)]
        a.check(slices); b.check(slices)
    finally:
        a.close(); b.close()
