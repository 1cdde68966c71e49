"""Drives an XQueue core over the recording hardware queue of oracle/xqueue_probe.cpp and
reads back the trace of adapter calls. Two cores can be driven with the same verbs:

* the shipped one: xsched_amd/lib/libpreempt.so + oracle/libxqueue_probe.so;
* the REFERENCE's: oracle/_ref/libxqueue_ref.so, one library holding the reference's own
  preempt/, sched/ (without the daemon client), protocol/ and utils/ sources compiled where
  they lie, plus the same recording queue compiled against the reference's headers.

Also holds the scripts (fixed and seeded random ones) both the golden generator and the
tests run. Test helper."""
import ctypes
import os
import random
import time
from ctypes import POINTER, byref, c_int, c_int64, c_size_t, c_uint64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE_LIB = os.path.join(ROOT, "oracle", "libxqueue_probe.so")
PREEMPT_LIB = os.path.join(ROOT, "xsched_amd", "lib", "libpreempt.so")
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libxqueue_ref.so")

NONE, DEACTIVATABLE, IDEMPOTENT = 0, 1, 2  # kCommandProperty* values
APP_MANAGED, POLICY_UNKNOWN = 1, 0


def _proto(api, rec):
    api.XQueueCreate.argtypes = [POINTER(c_uint64), c_uint64, c_int64, c_int64]
    api.XQueueDestroy.argtypes = [c_uint64]
    api.XQueueSetLaunchConfig.argtypes = [c_uint64, c_int64, c_int64]
    api.XQueueSubmit.argtypes = [c_uint64, c_uint64]
    api.XQueueSuspend.argtypes = [c_uint64, c_int64]
    api.XQueueResume.argtypes = [c_uint64, c_int64]
    api.XQueueQuery.argtypes = [c_uint64, POINTER(c_int)]
    api.HwQueueDestroy.argtypes = [c_uint64]
    api.XHintSetScheduler.argtypes = [c_int, c_int]
    rec.RecQueueCreate.argtypes = [POINTER(c_uint64), c_int]
    rec.RecCommandCreate.argtypes = [POINTER(c_uint64), c_int64, c_int]
    rec.RecQueueComplete.argtypes = [c_uint64, c_int64]
    rec.RecQueueSetGate.argtypes = [c_uint64, c_int]
    rec.RecQueueTrace.argtypes = [c_uint64, ctypes.c_char_p, c_size_t]
    rec.RecQueueTrace.restype = c_size_t


class Core:
    """One loaded XQueue core: `api` exports the XQueue C API, `rec` the recording queue."""

    def __init__(self, api, rec):
        self.api, self.rec = api, rec
        _proto(api, rec)
        assert api.XHintSetScheduler(APP_MANAGED, POLICY_UNKNOWN) == 0

    @classmethod
    def product(cls):
        api = ctypes.CDLL(PREEMPT_LIB, mode=ctypes.RTLD_LOCAL)
        return cls(api, ctypes.CDLL(PROBE_LIB, mode=ctypes.RTLD_LOCAL))

    @classmethod
    def reference(cls):
        os.environ.setdefault("XLOG_LEVEL", "ERRO")
        lib = ctypes.CDLL(REF_LIB, mode=ctypes.RTLD_LOCAL)
        return cls(lib, lib)


def ok(res):
    assert res == 0, f"XResult {res}"


class Session:
    """One XQueue over one recording queue; the same verbs as oracle.xqueue_model."""

    def __init__(self, core, threshold, batch, level):
        self.core, self.api, self.rec = core, core.api, core.rec
        hwq, xq = c_uint64(), c_uint64()
        ok(self.rec.RecQueueCreate(byref(hwq), 2))
        ok(self.api.XQueueCreate(byref(xq), hwq.value, level, 0))
        self.hwq, self.xq = hwq.value, xq.value
        ok(self.api.XQueueSetLaunchConfig(self.xq, threshold, batch))

    def burst(self, n, props=NONE):
        # The first command of a burst holds the launch thread in BeforeLaunch() until the
        # whole burst is buffered.
        self.rec.RecQueueSetGate(self.hwq, 0)
        for i in range(n):
            cmd = c_uint64()
            self.rec.RecCommandCreate(byref(cmd), props, 1 if i == 0 else 0)
            ok(self.api.XQueueSubmit(self.xq, cmd.value))
        self.rec.RecQueueSetGate(self.hwq, 1)

    def complete(self, upto):
        self.rec.RecQueueComplete(self.hwq, upto)

    def suspend(self):
        ok(self.api.XQueueSuspend(self.xq, 0))

    def resume(self, drop=False):
        ok(self.api.XQueueResume(self.xq, 1 if drop else 0))

    def trace(self):
        buf = ctypes.create_string_buffer(1 << 16)
        self.rec.RecQueueTrace(self.hwq, buf, 1 << 16)
        return buf.value.decode().split()

    def state(self):
        st = c_int()
        ok(self.api.XQueueQuery(self.xq, byref(st)))
        return {1: 'idle', 2: 'ready'}[st.value]

    def settle(self, want=None, quiet=0.03, limit=3.0):
        """Trace once it has stopped changing (or equals `want` and stays so)."""
        deadline = time.time() + limit
        got = self.trace()
        if want is not None:
            while got != want and time.time() < deadline:
                time.sleep(0.001)
                got = self.trace()
            time.sleep(quiet)
            return self.trace()
        last_change = time.time()
        while time.time() - last_change < quiet and time.time() < deadline:
            time.sleep(0.002)
            now = self.trace()
            if now != got:
                got, last_change = now, time.time()
        return got

    def apply(self, action):
        verb = action[0]
        if verb == 'burst':
            self.burst(action[1], action[2])
        elif verb == 'complete':
            self.complete(action[1])
        elif verb == 'suspend':
            self.suspend()
        elif verb == 'resume':
            self.resume(bool(action[1]))
        else:
            raise ValueError(verb)

    def close(self, last_idx):
        self.complete(last_idx + 1000)
        ok(self.api.XQueueDestroy(self.xq))
        ok(self.api.HwQueueDestroy(self.hwq))


def apply_model(model, action):
    verb = action[0]
    if verb == 'burst':
        model.burst(action[1], action[2])
    elif verb == 'complete':
        model.complete(action[1])
    elif verb == 'suspend':
        model.suspend()
    elif verb == 'resume':
        model.resume(bool(action[1]))


# ---- scripts -------------------------------------------------------------------------

def fixed_scripts():
    """name -> (threshold, batch, level, [actions])."""
    out = {}
    for thr, batch in [(8, 4), (16, 8), (4, 2), (1, 1), (5, 5)]:
        n = 3 * thr + 2
        out[f"stalled_device_{thr}_{batch}"] = (
            thr, batch, 1, [['burst', n, NONE]] + [['complete', i] for i in range(1, n + 1)])
    out["level2_replay_log"] = (4, 2, 2, [['burst', 7, DEACTIVATABLE], ['suspend'], ['resume', 0]]
                                + [['complete', i] for i in (1, 3, 5, 7)])
    out["level2_mixed_properties"] = (
        8, 4, 2, [['burst', n, p] for p, n in [(DEACTIVATABLE, 3), (NONE, 1), (IDEMPOTENT, 2),
                                               (DEACTIVATABLE, 2), (NONE, 2)]]
        + [['complete', i] for i in range(1, 11)])
    out["resume_drop_commands"] = (2, 1, 2, [['burst', 6, DEACTIVATABLE], ['suspend'], ['resume', 1],
                                             ['burst', 2, DEACTIVATABLE], ['complete', 8]])
    out["level1_suspend_during_window_wait"] = (
        4, 2, 1, [['burst', 9, NONE], ['suspend'], ['complete', 2], ['resume', 0], ['complete', 4],
                  ['suspend'], ['resume', 0], ['complete', 9]])
    return out


def random_script(seed, model_cls, steps=40):
    """Seeded script; the model is only used to keep `complete` targets legal (never beyond
    what has been launched)."""
    rnd = random.Random(seed)
    thr = rnd.choice([1, 2, 4, 8])
    batch = rnd.randint(1, thr)
    level = rnd.choice([1, 2])
    model = model_cls(thr, batch, level)
    actions = []
    submitted = 0
    for _ in range(steps):
        launched = max([int(t[1:].rstrip('*')) for t in model.trace if t.startswith('L')], default=0)
        verb = rnd.choice(['burst', 'burst', 'complete', 'complete', 'complete', 'suspend', 'resume'])
        if verb == 'burst':
            n = rnd.randint(1, 6)
            props = rnd.choice([NONE, DEACTIVATABLE, DEACTIVATABLE, IDEMPOTENT]) if level == 2 else NONE
            act = ['burst', n, props]
            submitted += n
        elif verb == 'complete':
            if launched <= model.done:
                continue
            act = ['complete', rnd.randint(model.done + 1, launched)]
        elif verb == 'suspend':
            act = ['suspend']
        else:
            act = ['resume', 0]
        apply_model(model, act)
        actions.append(act)
    actions += [['resume', 0], ['complete', submitted]]
    return thr, batch, level, actions


def last_index(actions):
    return sum(a[1] for a in actions if a[0] == 'burst')
