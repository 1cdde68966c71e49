"""ctypes view of oracle/sched_driver.cpp, for either build (ref_* over the reference's
sources, probe_* over this repository's classes). Test helper."""
import ctypes
import os
import struct
from ctypes import (POINTER, c_char_p, c_int, c_int8, c_int64, c_size_t, c_uint8, c_uint32, c_uint64,
                    c_void_p)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libsched_ref.so")
PROBE_LIB = os.path.join(ROOT, "oracle", "libsched_probe.so")

# record name -> list of (offset, size) of the bytes that carry fields; everything else
# is alignment padding, which the reference leaves uninitialised.
FIELDS = {
    "hint_priority": [(0, 4), (8, 8), (16, 4)],
    "hint_utilization": [(0, 4), (4, 4), (8, 8), (16, 4)],
    "hint_timeslice": [(0, 4), (8, 8)],
    "hint_deadline": [(0, 4), (8, 8), (16, 8)],
    "hint_kdeadline": [(0, 4), (8, 8)],
    "hint_laxity": [(0, 4), (8, 8), (16, 8), (24, 4), (28, 4)],
    "hint_window_active": [(0, 4), (4, 4), (8, 8)],
    "event_hint_priority": [(0, 8), (8, 8), (16, 4), (24, 8), (32, 4)],
    "event_process_create": [(0, 264)],
    "event_process_destroy": [(0, 8)],
    "event_terminate": [(0, 8)],
    "event_xqueue_create": [(0, 8), (8, 8), (16, 8), (24, 4), (32, 8), (40, 8)],
    "event_xqueue_config": [(0, 8), (8, 8), (16, 8), (24, 4), (32, 8), (40, 8)],
    "event_xqueue_destroy": [(0, 16)],
    "event_xqueue_idle": [(0, 16)],
    "event_xqueue_ready": [(0, 24)],
    "event_operation_complete": [(0, 16)],
    "operation_config": [(0, 8), (8, 4), (12, 4), (16, 8), (24, 4), (32, 8), (40, 8)],
    "operation_terminate": [(0, 8), (8, 4), (12, 4)],
    "operation_sched": None,  # no padding: every byte carries data
}


class SchedDriver:
    def __init__(self, path, prefix):
        self.lib = ctypes.CDLL(path)
        self.prefix = prefix

    def fn(self, name, restype=None, argtypes=None):
        f = getattr(self.lib, self.prefix + name)
        if restype is not None:
            f.restype = restype
        if argtypes is not None:
            f.argtypes = argtypes
        return f

    # ---- policies ----
    def policy(self, ptype):
        return _Policy(self, ptype)

    # ---- wire records ----
    def record(self, name, *args):
        """Bytes of one record. Integer arguments are passed as 64-bit values unless the
        function takes them as int (see sched_driver.cpp)."""
        f = self.fn("bytes_" + name, c_size_t, RECORD_ARGS[name] + [c_void_p, c_size_t])
        buf = ctypes.create_string_buffer(1024)
        n = f(*args, buf, 1024)
        assert 0 < n <= 1024
        return buf.raw[:n]

    def sched_operation(self, op_id, pid, running, suspended):
        f = self.fn("bytes_operation_sched", c_size_t,
                    [c_uint64, c_int, POINTER(c_uint64), c_int, POINTER(c_uint64), c_int, c_void_p, c_size_t])
        r = (c_uint64 * max(1, len(running)))(*running)
        s = (c_uint64 * max(1, len(suspended)))(*suspended)
        buf = ctypes.create_string_buffer(4096)
        n = f(op_id, pid, r, len(running), s, len(suspended), buf, 4096)
        return buf.raw[:n]

    def event_roundtrip(self, data):
        f = self.fn("event_roundtrip", c_size_t, [c_char_p, c_void_p, c_size_t])
        buf = ctypes.create_string_buffer(1024)
        n = f(data, buf, 1024)
        return buf.raw[:n]

    def operation_roundtrip(self, data):
        f = self.fn("operation_roundtrip", c_size_t, [c_char_p, c_void_p, c_size_t])
        buf = ctypes.create_string_buffer(4096)
        n = f(data, buf, 4096)
        return buf.raw[:n]

    def hint_event(self, hint_bytes):
        f = self.fn("bytes_event_hint", c_size_t, [c_char_p, c_void_p, c_size_t])
        buf = ctypes.create_string_buffer(1024)
        n = f(hint_bytes, buf, 1024)
        assert 0 < n <= 1024
        return buf.raw[:n]

    # ---- local scheduler ----
    def local(self, ptype):
        return _Local(self, ptype)

    # ---- names ----
    def policy_type_by_name(self, name):
        return self.fn("policy_type_by_name", c_int, [c_char_p])(name.encode())

    def policy_name(self, t):
        return self.fn("policy_name", c_char_p, [c_int])(t).decode()

    def scheduler_type_by_name(self, name):
        return self.fn("scheduler_type_by_name", c_int, [c_char_p])(name.encode())

    def scheduler_name(self, t):
        return self.fn("scheduler_name", c_char_p, [c_int])(t).decode()

    def level_name(self, t):
        return self.fn("level_name", c_char_p, [c_int])(t).decode()

    def platform_name(self, t):
        return self.fn("platform_name", c_char_p, [c_int])(t).decode()

    def make_device(self, t, i):
        return self.fn("make_device", c_uint64, [c_int, c_uint32])(t, i)


RECORD_ARGS = {
    "hint_priority": [c_uint64, c_int],
    "hint_utilization": [c_int, c_uint64, c_int],
    "hint_timeslice": [c_int64],
    "hint_deadline": [c_uint64, c_int64],
    "hint_kdeadline": [c_uint64],
    "hint_laxity": [c_uint64, c_int64, c_int, c_int],
    "hint_window_active": [c_int, c_uint64],
    "event_hint_priority": [c_uint64, c_int],
    "event_process_create": [c_char_p],
    "event_process_destroy": [c_int],
    "event_terminate": [],
    "event_xqueue_create": [c_uint64, c_uint64, c_int, c_int64, c_int64],
    "event_xqueue_config": [c_uint64, c_uint64, c_int, c_int64, c_int64],
    "event_xqueue_destroy": [c_uint64],
    "event_xqueue_idle": [c_uint64],
    "event_xqueue_ready": [c_uint64, c_int64],
    "event_operation_complete": [c_uint64],
    "operation_config": [c_uint64, c_int, c_uint64, c_int, c_int64, c_int64],
    "operation_terminate": [],
}


class _Policy:
    def __init__(self, drv, ptype):
        self.drv = drv
        self.h = drv.fn("policy_create", c_void_p, [c_int])(ptype)

    def close(self):
        self.drv.fn("policy_destroy", None, [c_void_p])(self.h)

    def priority(self, xq, prio):
        self.drv.fn("policy_hint_priority", None, [c_void_p, c_uint64, c_int])(self.h, xq, prio)

    def laxity(self, xq, lax, lp, cp):
        self.drv.fn("policy_hint_laxity", None, [c_void_p, c_uint64, c_int64, c_int, c_int])(self.h, xq, lax, lp, cp)

    def hint(self, hint_bytes):
        assert self.drv.fn("policy_recv_hint", c_int, [c_void_p, c_char_p])(self.h, hint_bytes) == 1

    def sched_processes(self, queues):
        """queues: list of (handle, device, ready, ready_time_us, pid, suspended) ->
        (decisions, timers); decisions: 1 suspend, 0 resume, -1 not touched"""
        n = len(queues)
        f = self.drv.fn("policy_sched_processes", c_int,
                        [c_void_p, c_int, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint8),
                         POINTER(c_int64), POINTER(c_int), POINTER(c_uint8), POINTER(c_int8),
                         POINTER(c_int64), c_int])
        h = (c_uint64 * n)(*[q[0] for q in queues])
        d = (c_uint64 * n)(*[q[1] for q in queues])
        r = (c_uint8 * n)(*[1 if q[2] else 0 for q in queues])
        t = (c_int64 * n)(*[q[3] for q in queues])
        pid = (c_int * n)(*[q[4] for q in queues])
        sus = (c_uint8 * n)(*[1 if q[5] else 0 for q in queues])
        dec = (c_int8 * n)()
        timers = (c_int64 * 16)()
        nt = f(self.h, n, h, d, r, t, pid, sus, dec, timers, 16)
        return list(dec), list(timers)[:min(nt, 16)]

    def sched(self, queues):
        """queues: list of (handle, device, ready, ready_time_us) -> (decisions, timers)"""
        n = len(queues)
        f = self.drv.fn("policy_sched", c_int,
                        [c_void_p, c_int, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint8),
                         POINTER(c_int64), POINTER(c_int8), POINTER(c_int64), c_int])
        h = (c_uint64 * n)(*[q[0] for q in queues])
        d = (c_uint64 * n)(*[q[1] for q in queues])
        r = (c_uint8 * n)(*[1 if q[2] else 0 for q in queues])
        t = (c_int64 * n)(*[q[3] for q in queues])
        dec = (c_int8 * n)()
        timers = (c_int64 * 16)()
        nt = f(self.h, n, h, d, r, t, dec, timers, 16)
        return list(dec), list(timers)[:min(nt, 16)]


def with_pid(event_bytes, pid):
    """The same event as sent by process `pid` (EventMeta is {int32 type, int32 pid})."""
    return event_bytes[:4] + struct.pack("<i", pid) + event_bytes[8:]


def parse_sched_operation(data):
    """(id, type, pid, running list, suspended list) of a SchedOperation's wire bytes:
    {uint64 id, int32 type, int32 pid, uint64 size, uint64 running_cnt,
    uint64 suspended_cnt, uint64 handles[]}."""
    op_id, op_type, pid, size, n_run, n_sus = struct.unpack_from("<QiiQQQ", data)
    assert size == len(data) == 40 + 8 * (n_run + n_sus)
    handles = struct.unpack_from("<%dQ" % (n_run + n_sus), data, 40)
    return op_id, op_type, pid, list(handles[:n_run]), list(handles[n_run:])


class _Local:
    """A LocalScheduler whose executor records operations."""

    def __init__(self, drv, ptype):
        self.drv = drv
        self.h = drv.fn("local_create", c_void_p, [c_int])(ptype)

    def close(self):
        self.drv.fn("local_destroy", None, [c_void_p])(self.h)

    def run(self):
        self.drv.fn("local_run", None, [c_void_p])(self.h)

    def stop(self):
        self.drv.fn("local_stop", None, [c_void_p])(self.h)

    def set_policy(self, ptype):
        self.drv.fn("local_set_policy", None, [c_void_p, c_int])(self.h, ptype)

    def recv(self, event_bytes):
        assert self.drv.fn("local_recv_event", c_int, [c_void_p, c_char_p])(self.h, event_bytes) == 1

    def take(self):
        """Wire bytes of the operations executed since the last call, in order."""
        f = self.drv.fn("local_take_operations", c_size_t, [c_void_p, c_void_p, c_size_t])
        need = f(self.h, None, 0)
        buf = ctypes.create_string_buffer(max(1, need))
        assert f(self.h, buf, need) == need
        ops, off = [], 0
        while off < need:
            (size,) = struct.unpack_from("<Q", buf.raw, off)
            ops.append(buf.raw[off + 8:off + 8 + size])
            off += 8 + size
        return ops

    def round(self, events):
        """Exactly one scheduling round over `events`: they are queued while no worker
        runs, followed by a terminate event, so the worker that is then started folds
        all of them into the status, runs the policy once, executes and exits."""
        for e in events:
            self.recv(e)
        self.recv(self.drv.record("event_terminate"))
        self.run()
        self.stop()
        return self.take()


def masked(name, data):
    """Bytes with the padding zeroed."""
    fields = FIELDS[name]
    if fields is None:
        return data
    out = bytearray(len(data))
    for off, size in fields:
        out[off:off + size] = data[off:off + size]
    return bytes(out)


def ref():
    return SchedDriver(REF_LIB, "ref_") if os.path.exists(REF_LIB) else None


def probe():
    return SchedDriver(PROBE_LIB, "probe_")
