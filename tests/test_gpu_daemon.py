"""GPU: two client PROCESSES share the MI355X under the scheduler daemon. Their events go to
xserver over the datagram channel, xserver's local scheduler runs HPF over the queues of both
processes, and the suspend / resume operations come back to the process that owns the queue,
where they deactivate and reactivate a Level-2 hardware queue (reference
sched/src/scheduler/global.cpp, service/server/src/server.cpp). The low-priority process must
get deactivated while the high-priority one has work, and both results must be bit-exact."""
import json
import os
import subprocess
import sys
import tempfile
import time

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
XSERVER = os.path.join(ROOT, "xsched_amd", "lib", "xserver")
CLIENT = os.path.join(ROOT, "tests", "gpu_daemon_client.py")


def test_two_gpu_processes_hpf_through_the_daemon(gpu):
    assert os.path.exists(XSERVER), "xserver has not been built"
    sock_dir = tempfile.mkdtemp(prefix="xsched-gpu-")
    server = subprocess.Popen([XSERVER, "HPF"], env=dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="WARN"))
    try:
        deadline = time.time() + 5
        while not os.path.exists(os.path.join(sock_dir, "xsched-1.sock")) and time.time() < deadline:
            time.sleep(0.01)
        assert os.path.exists(os.path.join(sock_dir, "xsched-1.sock")), "xserver did not come up"
        env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XSCHED_SCHEDULER="GLB", XLOG_LEVEL="WARN")
        env.pop("XSCHED_POLICY", None)

        def client(*args):
            return subprocess.Popen([sys.executable, CLIENT, *map(str, args)], env=env,
                                    stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)

        print("case daemon: background process 2^26 x 3000, foreground process 2^20 x 60 every 3 ms", flush=True)
        bg = client(1, 26, 3000, 0, 0.0)          # ~0.13 ms per command, back to back: ~0.4 s
        assert json.loads(bg.stdout.readline())["event"] == "ready"
        fg = client(2, 20, 60, 3000, 0.02)
        assert json.loads(fg.stdout.readline())["event"] == "ready"
        for proc in (bg, fg):
            proc.stdin.write("go\n")
            proc.stdin.flush()
        f = json.loads(fg.communicate(timeout=100)[0].strip().splitlines()[-1])
        b = json.loads(bg.communicate(timeout=100)[0].strip().splitlines()[-1])
        print("fg", f, "\nbg", b, flush=True)
        assert fg.returncode == 0 and bg.returncode == 0
        assert f["bit_exact"] and b["bit_exact"]
        assert f["deactivations"] == 0, "the high-priority queue was suspended"
        # The background needs ~0.4 s; the foreground becomes ready 60 times in the first
        # 0.2 s of it.
        assert b["deactivations"] > 0 and b["reactivations"] > 0, \
            "the daemon never suspended the low-priority process's queue"
    finally:
        server.terminate()
        try:
            server.wait(timeout=5)
        except subprocess.TimeoutExpired:
            server.kill()
