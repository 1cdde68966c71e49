"""Helper process for tests/test_gpu_daemon.py: one XSched client on the MI355X talking to
xserver (XSCHED_SCHEDULER=GLB). Usage:
    gpu_daemon_client.py <priority> <log2 n> <commands> <gap_us> <start_delay_s>
One Level-2 XQueue on its own stream submits <commands> guarded in-place AXPYs, <gap_us>
apart (0 = back to back), and prints one JSON line with the adapter's counters and whether
the result equals the oracle's bit for bit."""
import json
import os
import sys
import time
from ctypes import byref, c_uint64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import numpy as np  # noqa: E402
import torch  # noqa: E402

import oracle  # noqa: E402
import xsched_amd as xs  # noqa: E402


def main():
    prio, lg, commands, gap_us, delay = (int(sys.argv[1]), int(sys.argv[2]), int(sys.argv[3]),
                                         int(sys.argv[4]), float(sys.argv[5]))
    n = 1 << lg
    p, h = xs.preempt(), xs.halhip()
    x_h = oracle.fill_uniform(prio, 1, 0, n)
    y_h = oracle.fill_uniform(prio, 2, 0, n)
    x = torch.from_numpy(x_h).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    stream = torch.cuda.Stream()
    hwq = xs.hip_queue_create(stream.cuda_stream)
    xq = xs.xqueue_create(hwq, xs.kPreemptLevelDeactivate)
    xs.check(p.XQueueSetLaunchConfig(xq, 2, 1))
    xs.check(p.XHintPriority(xq, prio))
    print(json.dumps({"event": "ready", "pid": os.getpid()}), flush=True)
    sys.stdin.readline()  # the test says go once every client is ready
    time.sleep(delay)
    t0 = time.perf_counter()
    for _ in range(commands):
        cmd = c_uint64()
        xs.check(h.HipAxpyCommandCreate(byref(cmd), 0.5, x.data_ptr(), y.data_ptr(), n, 1))
        xs.check(p.XQueueSubmit(xq, cmd.value))
        if gap_us:
            xs.check(p.XQueueWaitAll(xq))
            time.sleep(gap_us * 1e-6)
    xs.check(p.XQueueWaitAll(xq))
    elapsed = time.perf_counter() - t0
    stats = (c_uint64 * 8)()
    xs.check(h.HipQueueGetStats(hwq, stats))
    # AXPY is element-wise, so three slices of 2^16 elements tell as much as the whole array
    # (thousands of passes over the whole array would take the CPU minutes).
    got = y.cpu().numpy()
    exact = True
    for first in (0, (n // 2) & ~15, n - min(n, 1 << 16)):
        sl = slice(first, first + min(n, 1 << 16))
        want = oracle.axpy(0.5, x_h[sl], y_h[sl], commands)
        exact = exact and bool(np.array_equal(got[sl].view(np.uint32), want.view(np.uint32)))
    xs.check(p.XQueueDestroy(xq))
    xs.check(p.HwQueueDestroy(hwq))
    print(json.dumps({"event": "done", "priority": prio, "elapsed_s": elapsed, "bit_exact": exact,
                      "launches": stats[0], "replays": stats[1], "deactivations": stats[2],
                      "reactivations": stats[3]}), flush=True)


if __name__ == "__main__":
    main()
