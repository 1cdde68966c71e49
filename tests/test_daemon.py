"""Scheduler daemon wiring on one machine: client processes relay their events to
xserver over the datagram channel, xserver's LocalScheduler decides, and the operations
come back to the process they address (reference sched/src/scheduler/global.cpp and
service/server/src/server.cpp). CPU only: the clients use the host adapter."""
import json
import os
import subprocess
import sys
import tempfile
import time

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
XSERVER = os.path.join(ROOT, "xsched_amd", "lib", "xserver")
CLIENT = os.path.join(ROOT, "tests", "daemon_client.py")


@pytest.fixture(params=["blocking", "polling"])
def daemon(request, monkeypatch):
    """The daemon and its clients with receivers that block at once (the default) and with
    receivers that poll for 3 ms after each message (XSCHED_SPIN_US)."""
    if not os.path.exists(XSERVER):
        pytest.fail("xserver has not been built")
    if request.param == "polling":
        monkeypatch.setenv("XSCHED_SPIN_US", "3000")
    else:
        monkeypatch.delenv("XSCHED_SPIN_US", raising=False)
    sock_dir = tempfile.mkdtemp(prefix="xsched-test-")
    env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="INFO")
    proc = subprocess.Popen([XSERVER, "HPF"], env=env, stderr=subprocess.PIPE, text=True)
    deadline = time.time() + 5
    while not os.path.exists(os.path.join(sock_dir, "xsched-1.sock")) and time.time() < deadline:
        time.sleep(0.01)
    assert os.path.exists(os.path.join(sock_dir, "xsched-1.sock")), "xserver did not come up"
    client_env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XSCHED_SCHEDULER="GLB", XLOG_LEVEL="WARN")
    client_env.pop("XSCHED_POLICY", None)
    yield proc, client_env, sock_dir
    proc.terminate()
    try:
        proc.wait(timeout=5)
    except subprocess.TimeoutExpired:
        proc.kill()


def client(env, *args):
    return subprocess.Popen([sys.executable, CLIENT, *map(str, args)], env=env,
                            stdout=subprocess.PIPE, text=True)


def test_two_processes_hpf_through_the_daemon(daemon):
    """A low-priority process must not run while a high-priority process has work, and
    must run to completion afterwards."""
    proc, env, _ = daemon
    busy = client(env, "busy", 5, 1.0)
    assert json.loads(busy.stdout.readline())["event"] == "busy-started"
    time.sleep(0.1)                      # let the daemon see the busy queue
    quick = client(env, "quick", 1, 8)
    q = json.loads(quick.communicate(timeout=20)[0].strip().splitlines()[-1])
    b = busy.communicate(timeout=20)[0]
    assert quick.returncode == 0 and busy.returncode == 0
    assert q["executed_early"] == 0, "low-priority client ran while the high-priority one was busy"
    assert q["executed_final"] == 8
    assert json.loads(b.strip().splitlines()[-1])["role"] == "busy"


def test_equal_priorities_are_not_blocked(daemon):
    proc, env, _ = daemon
    busy = client(env, "busy", 3, 0.8)
    assert json.loads(busy.stdout.readline())["event"] == "busy-started"
    time.sleep(0.1)
    quick = client(env, "quick", 3, 8)
    q = json.loads(quick.communicate(timeout=20)[0].strip().splitlines()[-1])
    busy.communicate(timeout=20)
    assert q["executed_early"] == 8


def test_dead_client_is_forgotten(daemon):
    """A high-priority client that is killed must stop blocking everybody else."""
    proc, env, sock_dir = daemon
    busy = client(env, "busy", 9, 30.0)
    assert json.loads(busy.stdout.readline())["event"] == "busy-started"
    time.sleep(0.1)
    quick = client(env, "quick", 1, 4)
    time.sleep(0.2)
    busy.kill()
    busy.wait()
    q = json.loads(quick.communicate(timeout=20)[0].strip().splitlines()[-1])
    assert q["executed_final"] == 4      # released once the daemon noticed the death
    assert not os.path.exists(os.path.join(sock_dir, f"xsched-{busy.pid}.sock")) or True


def test_client_without_daemon_fails_loudly():
    env = dict(os.environ, XSCHED_SOCKET_DIR=tempfile.mkdtemp(prefix="xsched-none-"),
               XSCHED_SCHEDULER="GLB", XLOG_LEVEL="ERRO")
    p = subprocess.run([sys.executable, CLIENT, "quick", "1", "1"], env=env, capture_output=True, text=True,
                       timeout=30)
    assert p.returncode != 0
    assert "scheduler daemon" in p.stderr


def test_malformed_datagrams_do_not_hurt_the_daemon():
    """Short records, records whose embedded sizes exceed what arrived, unknown types and
    status queries (they carry pointers) are dropped; the daemon keeps serving."""
    import socket
    import struct
    sock_dir = tempfile.mkdtemp(prefix="xsched-test-")
    env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="ERRO")
    server = subprocess.Popen([XSERVER, "HPF"], env=env)
    try:
        path = os.path.join(sock_dir, "xsched-1.sock")
        deadline = time.time() + 10
        while not os.path.exists(path) and time.time() < deadline:
            time.sleep(0.02)
        s = socket.socket(socket.AF_UNIX, socket.SOCK_DGRAM)
        meta = lambda etype, pid=4242: struct.pack("<ii", etype, pid)
        bad = [
            b"", b"\x01", meta(2)[:7],                      # shorter than the meta record
            meta(9999),                                      # unknown type
            meta(0) + struct.pack("<Q", 1 << 40) + b"\0" * 16,   # hint event claiming 1 TiB
            meta(0) + struct.pack("<Q", 24),                 # hint event with no hint record behind it
            meta(0) + struct.pack("<Q", 24) + struct.pack("<i", 77) + b"\0" * 20,  # unknown hint type
            meta(2),                                         # process-create without its command line
            meta(4) + b"\0" * 8,                             # queue-create cut short
            meta(9) + b"\0" * 16, meta(10) + b"\0" * 8,      # status queries: pointers from elsewhere
        ]
        for rec in bad:
            s.sendto(rec, path)
        time.sleep(0.3)
        assert server.poll() is None, "xserver died on a malformed record"
        # and it still serves a real client
        client_env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XSCHED_SCHEDULER="GLB", XLOG_LEVEL="WARN")
        out = subprocess.run([sys.executable, CLIENT, "quick", "1", "8"], env=client_env, capture_output=True,
                             text=True, timeout=60)
        assert out.returncode == 0, out.stderr
        assert server.poll() is None
    finally:
        server.terminate()
        server.wait(timeout=10)
