"""Helper process for tests/test_daemon.py: one XSched client talking to xserver
(XSCHED_SCHEDULER=GLB). Roles:
  busy <prio> <seconds>   one host queue at priority <prio> that is busy for <seconds>
  idle <prio> <seconds>   one host queue at priority <prio> with no work, kept for <seconds>
  quick <prio> <count>    one host queue at priority <prio>; submits <count> quick kernels,
                          reports how many had run after 0.3 s and after everything finished
Prints one JSON line."""
import json
import os
import sys
import time
from ctypes import byref, c_uint64

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import xsched_amd as xs  # noqa: E402


def stats(hwq):
    e, s, r = c_uint64(), c_uint64(), c_uint64()
    xs.check(xs.halhost().HostQueueGetStats(hwq, byref(e), byref(s), byref(r)))
    return e.value


def main():
    role, prio, arg = sys.argv[1], int(sys.argv[2]), float(sys.argv[3])
    p, h = xs.preempt(), xs.halhost()
    hwq = xs.host_queue_create()
    xq = xs.xqueue_create(hwq)
    xs.check(p.XHintPriority(xq, prio))
    out = {"role": role, "pid": os.getpid()}
    if role == "busy":
        @xs.HostKernelFn
        def slow(a, wg, n):
            time.sleep(arg)
        cmd = c_uint64()
        xs.check(h.HostKernelCommandCreate(byref(cmd), slow, None, 1, 0))
        xs.check(p.XQueueSubmit(xq, cmd.value))
        print(json.dumps({"event": "busy-started", "pid": os.getpid()}), flush=True)
        xs.check(p.XQueueWaitAll(xq))
    elif role == "idle":
        print(json.dumps({"event": "busy-started", "pid": os.getpid()}), flush=True)
        time.sleep(arg)
    else:
        @xs.HostKernelFn
        def quick(a, wg, n):
            pass
        # Scheduling is asynchronous: give the daemon's answer to the priority hint time to
        # arrive before the first submission.
        time.sleep(0.2)
        for _ in range(int(arg)):
            cmd = c_uint64()
            xs.check(h.HostKernelCommandCreate(byref(cmd), quick, None, 1, 0))
            xs.check(p.XQueueSubmit(xq, cmd.value))
        time.sleep(0.3)
        out["executed_early"] = stats(hwq)
        xs.check(p.XQueueWaitAll(xq))
        out["executed_final"] = stats(hwq)
    xs.check(p.XQueueDestroy(xq))
    xs.check(p.HwQueueDestroy(hwq))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
