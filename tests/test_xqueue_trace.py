"""The shipped XQueue core (libpreempt.so), driven through the public C API over a
recording hardware queue, must ask of its adapter exactly what the launch-loop model
(oracle/xqueue_model.py, a restatement of the reference's launch_worker / command_buffer /
async_xqueue) predicts: same launches, same marker placement, same synchronisation
targets, same deactivate / reactivate calls, in the same order."""
import ctypes
import os
import random
import time
from ctypes import byref, c_char_p, c_int, c_int64, c_size_t, c_uint64

import pytest

from oracle.xqueue_model import DEACTIVATABLE, IDEMPOTENT, NONE, XQueueModel

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def rec(xs):
    path = os.path.join(ROOT, "oracle", "libxqueue_probe.so")
    if not os.path.exists(path):
        pytest.fail("oracle/libxqueue_probe.so missing: run __graft_entry__.build()")
    lib = ctypes.CDLL(path)
    lib.RecQueueCreate.argtypes = [ctypes.POINTER(c_uint64), c_int]
    lib.RecCommandCreate.argtypes = [ctypes.POINTER(c_uint64), c_int64, c_int]
    lib.RecQueueComplete.argtypes = [c_uint64, c_int64]
    lib.RecQueueSetGate.argtypes = [c_uint64, c_int]
    lib.RecQueueTrace.argtypes = [c_uint64, ctypes.c_char_p, c_size_t]
    lib.RecQueueTrace.restype = c_size_t
    xs.check(xs.preempt().XHintSetScheduler(xs.kSchedulerAppManaged, xs.kPolicyUnknown))
    return lib


class Product:
    """Same verbs as XQueueModel, executed on the real core."""

    def __init__(self, xs, rec, threshold, batch, level):
        self.xs, self.rec, self.p = xs, rec, xs.preempt()
        hwq = c_uint64()
        xs.check(rec.RecQueueCreate(byref(hwq), 2))
        self.hwq = hwq.value
        self.xq = xs.xqueue_create(self.hwq, level)
        xs.check(self.p.XQueueSetLaunchConfig(self.xq, threshold, batch))

    def burst(self, n, props=NONE):
        # The first command of a burst holds the launch thread in BeforeLaunch() until the
        # whole burst is buffered.
        self.rec.RecQueueSetGate(self.hwq, 0)
        for i in range(n):
            cmd = c_uint64()
            self.rec.RecCommandCreate(byref(cmd), props, 1 if i == 0 else 0)
            self.xs.check(self.p.XQueueSubmit(self.xq, cmd.value))
        self.rec.RecQueueSetGate(self.hwq, 1)

    def complete(self, upto):
        self.rec.RecQueueComplete(self.hwq, upto)

    def suspend(self):
        self.xs.check(self.p.XQueueSuspend(self.xq, 0))

    def resume(self, drop=False):
        self.xs.check(self.p.XQueueResume(self.xq, 1 if drop else 0))

    def trace(self):
        buf = ctypes.create_string_buffer(1 << 16)
        self.rec.RecQueueTrace(self.hwq, buf, 1 << 16)
        return buf.value.decode().split()

    def state(self):
        st = c_int()
        self.xs.check(self.p.XQueueQuery(self.xq, byref(st)))
        return {1: 'idle', 2: 'ready'}[st.value]

    def close(self, last_idx):
        self.complete(last_idx + 1000)
        self.xs.check(self.p.XQueueDestroy(self.xq))
        self.xs.check(self.p.HwQueueDestroy(self.hwq))


def expect(prod, model, what=""):
    """Wait until the product's trace equals the model's, then make sure it stays so."""
    want = model.trace
    deadline = time.time() + 3.0
    got = prod.trace()
    while got != want and time.time() < deadline:
        time.sleep(0.001)
        got = prod.trace()
    assert got == want, f"{what}: trace differs\n got  {got}\n want {want}"
    time.sleep(0.02)
    assert prod.trace() == want, f"{what}: product kept going beyond the model"


def both(xs, rec, thr, batch, level):
    return Product(xs, rec, thr, batch, level), XQueueModel(thr, batch, level)


@pytest.mark.parametrize("thr,batch", [(8, 4), (16, 8), (4, 2), (1, 1), (5, 5)])
def test_window_and_markers_stalled_device(xs, rec, thr, batch):
    prod, model = both(xs, rec, thr, batch, 1)
    n = 3 * thr + 2
    prod.burst(n); model.burst(n)
    expect(prod, model, "burst")
    for upto in range(1, n + 1):
        prod.complete(upto); model.complete(upto)
        expect(prod, model, f"complete({upto})")
    assert prod.state() == model.state == 'idle'
    prod.close(n)


def test_level2_suspend_resume_replay_log(xs, rec):
    prod, model = both(xs, rec, 4, 2, 2)
    prod.burst(7, DEACTIVATABLE); model.burst(7, DEACTIVATABLE)
    expect(prod, model, "burst")
    prod.suspend(); model.suspend()
    expect(prod, model, "suspend")
    prod.resume(); model.resume()
    expect(prod, model, "resume")
    for upto in (1, 3, 5, 7):
        prod.complete(upto); model.complete(upto)
        expect(prod, model, f"complete({upto})")
    prod.close(7)


def test_level2_mixed_properties_drain_points(xs, rec):
    prod, model = both(xs, rec, 8, 4, 2)
    for props, n in [(DEACTIVATABLE, 3), (NONE, 1), (IDEMPOTENT, 2), (DEACTIVATABLE, 2), (NONE, 2)]:
        prod.burst(n, props); model.burst(n, props)
        expect(prod, model, f"burst({n},{props})")
    for upto in range(1, 11):
        prod.complete(upto); model.complete(upto)
        expect(prod, model, f"complete({upto})")
    prod.close(10)


def test_resume_with_drop_commands(xs, rec):
    prod, model = both(xs, rec, 2, 1, 2)
    prod.burst(6, DEACTIVATABLE); model.burst(6, DEACTIVATABLE)
    expect(prod, model, "burst")
    prod.suspend(); model.suspend()
    expect(prod, model, "suspend")
    prod.resume(drop=True); model.resume(drop=True)
    expect(prod, model, "drop")
    assert prod.state() == model.state == 'idle'
    prod.burst(2, DEACTIVATABLE); model.burst(2, DEACTIVATABLE)
    expect(prod, model, "after drop")
    prod.close(8)


@pytest.mark.parametrize("seed", range(12))
def test_random_scripts_match_model(xs, rec, seed):
    """Differential run over random scripts of bursts, device progress, suspends and
    resumes at both levels."""
    rnd = random.Random(seed)
    thr = rnd.choice([1, 2, 4, 8])
    batch = rnd.randint(1, thr)
    level = rnd.choice([1, 2])
    prod, model = both(xs, rec, thr, batch, level)
    submitted = 0
    for step in range(40):
        launched = max([int(t[1:].rstrip('*')) for t in model.trace if t.startswith('L')], default=0)
        action = rnd.choice(['burst', 'burst', 'complete', 'complete', 'complete', 'suspend', 'resume'])
        if action == 'burst':
            n = rnd.randint(1, 6)
            props = rnd.choice([NONE, DEACTIVATABLE, DEACTIVATABLE, IDEMPOTENT]) if level == 2 else NONE
            prod.burst(n, props); model.burst(n, props)
            submitted += n
        elif action == 'complete' and launched > model.done:
            upto = rnd.randint(model.done + 1, launched)
            prod.complete(upto); model.complete(upto)
        elif action == 'suspend':
            prod.suspend(); model.suspend()
        elif action == 'resume':
            prod.resume(); model.resume()
        expect(prod, model, f"seed {seed} step {step} {action}")
    prod.resume(); model.resume()
    prod.complete(submitted); model.complete(submitted)
    expect(prod, model, "final")
    assert prod.state() == model.state == 'idle'
    prod.close(submitted)
