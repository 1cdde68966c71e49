"""The daemon's HTTP control plane (reference service/server/src/server.cpp:28-39 routes,
:204-543 handlers; JSON field names of service/common/src/convert.cpp:7-17): the routes the
reference's command-line client uses, driven here with http.client against a running xserver
and a client process on the host adapter. CPU only."""
import http.client
import json
import os
import socket
import subprocess
import tempfile
import time

import pytest

from test_daemon import XSERVER, client

STATUS_FIELDS = {"handle", "device", "level", "pid", "threshold", "batch_size", "ready", "suspended"}


def free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


@pytest.fixture()
def daemon_http():
    if not os.path.exists(XSERVER):
        pytest.fail("xserver has not been built")
    sock_dir = tempfile.mkdtemp(prefix="xsched-test-")
    port = free_port()
    env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="INFO")
    env.pop("XSCHED_SERVER_ADDR", None)
    proc = subprocess.Popen([XSERVER, "HPF", str(port)], env=env, stderr=subprocess.PIPE, text=True)
    deadline = time.time() + 5
    up = False
    while time.time() < deadline and not up:
        try:
            socket.create_connection(("127.0.0.1", port), timeout=0.2).close()
            up = os.path.exists(os.path.join(sock_dir, "xsched-1.sock"))
        except OSError:
            time.sleep(0.02)
    assert up, "xserver's control plane did not come up"
    client_env = dict(os.environ, XSCHED_SOCKET_DIR=sock_dir, XSCHED_SCHEDULER="GLB", XLOG_LEVEL="WARN")
    client_env.pop("XSCHED_POLICY", None)
    yield port, client_env
    proc.terminate()
    try:
        proc.wait(timeout=5)
    except subprocess.TimeoutExpired:
        proc.kill()


def call(port, method, path, body=None):
    conn = http.client.HTTPConnection("127.0.0.1", port, timeout=5)
    headers = {"Content-Type": "application/json"} if body is not None else {}
    conn.request(method, path, body=None if body is None else json.dumps(body), headers=headers)
    resp = conn.getresponse()
    text = resp.read().decode()
    conn.close()
    return resp.status, (json.loads(text) if text else None)


def busy_client(port, env, prio=5, seconds=3.0, role="busy"):
    busy = client(env, role, prio, seconds)
    pid = json.loads(busy.stdout.readline())["pid"]
    deadline = time.time() + 3
    while time.time() < deadline:
        status, body = call(port, "GET", "/xqueues")
        mine = [q for q in body["xqueues"] if q["pid"] == pid]
        if mine:
            return busy, pid, mine[0]
        time.sleep(0.02)
    raise AssertionError("the daemon never listed the client's queue")


def test_empty_daemon_lists_nothing_and_reports_its_policy(daemon_http):
    port, _ = daemon_http
    assert call(port, "GET", "/xqueues") == (200, {"xqueues": [], "processes": []})
    assert call(port, "GET", "/policy") == (200, {"policy": 1})          # kPolicyHighestPriorityFirst
    assert call(port, "GET", "/nothing-here")[0] == 404
    assert call(port, "GET", "/xqueue/zz")[0] == 400
    assert call(port, "GET", "/xqueue/0xabc")[0] == 404


def test_queue_listing_and_lookup(daemon_http):
    port, env = daemon_http
    busy, pid, listed = busy_client(port, env)
    try:
        assert set(listed) == STATUS_FIELDS
        assert listed["level"] == 1 and listed["threshold"] == 16 and listed["batch_size"] == 8
        assert listed["suspended"] is False
        status, body = call(port, "GET", "/xqueues")
        assert [p["pid"] for p in body["processes"]] == [pid]
        assert "daemon_client.py" in body["processes"][0]["cmdline"]
        for spelling in ("%x", "0x%x", "%X"):
            status, one = call(port, "GET", "/xqueue/" + spelling % listed["handle"])
            assert status == 200
            assert one["xqueue"]["handle"] == listed["handle"] and one["process"]["pid"] == pid
    finally:
        busy.kill()
        busy.wait()
    # a dead process disappears from the listing (the daemon reaps it)
    deadline = time.time() + 5
    while time.time() < deadline and call(port, "GET", "/xqueues")[1]["xqueues"]:
        time.sleep(0.05)
    assert call(port, "GET", "/xqueues")[1] == {"xqueues": [], "processes": []}


def test_config_reaches_the_owning_process(daemon_http):
    port, env = daemon_http
    busy, pid, listed = busy_client(port, env, role="idle", seconds=20.0)   # a busy queue takes its new configuration once it drains
    path = "/config/%x" % listed["handle"]
    try:
        assert call(port, "POST", path) == (200, {"warning": "no change"})
        assert call(port, "POST", path + "?level=0") == (400, {"error": "invalid level"})
        assert call(port, "POST", path + "?level=4") == (400, {"error": "invalid level"})
        assert call(port, "POST", path + "?threshold=0") == (400, {"error": "invalid command threshold"})
        assert call(port, "POST", path + "?batch_size=-2") == (400, {"error": "invalid command batch size"})
        assert call(port, "POST", path + "?threshold=8") == (400, {"error": "batch size must be less than threshold"})
        assert call(port, "POST", "/config/123456?threshold=4") == (404, {"error": "XQueue not found"})
        assert call(port, "POST", "/config/0")[0] == 400

        assert call(port, "POST", path + "?threshold=6&batch_size=3") == (200, {"info": "success"})
        deadline = time.time() + 3
        seen = None
        while time.time() < deadline:
            seen = call(port, "GET", "/xqueue/%x" % listed["handle"])[1]["xqueue"]
            if seen["threshold"] == 6:
                break
            time.sleep(0.02)
        assert (seen["threshold"], seen["batch_size"], seen["level"]) == (6, 3, 1)
    finally:
        busy.kill()
        busy.wait()


def test_policy_switch(daemon_http):
    port, _ = daemon_http
    assert call(port, "POST", "/policy")[0] == 400
    assert call(port, "POST", "/policy?policy=0")[0] == 400
    assert call(port, "POST", "/policy?policy=99")[0] == 400
    assert call(port, "POST", "/policy?policy=4") == (200, {"info": "success"})   # utilization partition
    deadline = time.time() + 2
    while time.time() < deadline and call(port, "GET", "/policy")[1]["policy"] != 4:
        time.sleep(0.02)
    assert call(port, "GET", "/policy") == (200, {"policy": 4})


def test_hint_validation(daemon_http):
    port, _ = daemon_http
    post = lambda body: call(port, "POST", "/hint", body)  # noqa: E731
    assert post({})[1] == {"error": "missing hint type"}
    assert post({"hint_type": 0})[1] == {"error": "invalid hint type"}
    assert post({"hint_type": 1, "priority": 3})[1] == {"error": "invalid handle"}
    assert post({"hint_type": 1, "handle": 5})[1] == {"error": "missing priority"}
    assert post({"hint_type": 1, "handle": 5, "priority": 1000})[1] == {"error": "invalid priority"}
    assert post({"hint_type": 2, "utilization": 30})[1] == {"error": "handle or pid is required"}
    assert post({"hint_type": 2, "pid": 7})[1] == {"error": "missing utilization"}
    assert post({"hint_type": 2, "pid": 7, "utilization": 101})[1] == {"error": "invalid utilization"}
    assert post({"hint_type": 3})[1] == {"error": "missing timeslice"}
    assert post({"hint_type": 3, "timeslice": 0})[1] == {"error": "invalid timeslice"}
    assert post({"hint_type": 3, "timeslice": 5000}) == (200, {"info": "success"})
    assert post({"hint_type": 2, "pid": 7, "utilization": 40}) == (200, {"info": "success"})
    status, _ = call(port, "POST", "/hint")
    assert status == 400
    conn = http.client.HTTPConnection("127.0.0.1", port, timeout=5)
    conn.request("POST", "/hint", body="{not json")
    assert conn.getresponse().status == 400
    conn.close()


def test_priority_hint_over_http_changes_who_runs(daemon_http):
    """A priority hint posted to the daemon is what the policy acts on: a queue that the
    daemon is told to rank below a busy one does not run until the busy one is done."""
    port, env = daemon_http
    busy, pid, listed = busy_client(port, env, prio=3, seconds=1.0)
    quick = client(env, "quick", 3, 8)            # same priority: would run at once
    try:
        deadline = time.time() + 3
        handle = None
        while time.time() < deadline and handle is None:
            for q in call(port, "GET", "/xqueues")[1]["xqueues"]:
                if q["pid"] != pid:
                    handle = q["handle"]
            time.sleep(0.01)
        assert handle is not None
        time.sleep(0.05)                          # after the client's own priority hint
        assert call(port, "POST", "/hint", {"hint_type": 1, "handle": handle, "priority": -5}) == (200, {"info": "success"})
        q = json.loads(quick.communicate(timeout=20)[0].strip().splitlines()[-1])
        busy.communicate(timeout=20)
        assert q["executed_early"] == 0 and q["executed_final"] == 8
    finally:
        for p in (busy, quick):
            if p.poll() is None:
                p.kill()
                p.wait()


def test_malformed_requests_do_not_hurt_the_daemon(daemon_http):
    """Garbage, an oversized request, a half-sent request and an unknown method are answered
    with an error or dropped; the daemon keeps serving."""
    port, _ = daemon_http

    def raw(data, wait=True):
        s = socket.create_connection(("127.0.0.1", port), timeout=3)
        try:
            s.sendall(data)
            if not wait:
                return b""
            s.settimeout(3)
            try:
                return s.recv(4096)
            except OSError:
                return b""
        finally:
            s.close()

    assert raw(b"\x00\xff\x10 not http at all\r\n\r\n").split(b" ")[1] in (b"400", b"404")
    assert raw(b"BREW /policy HTTP/1.1\r\nHost: x\r\n\r\n").split(b" ")[1] in (b"404", b"405", b"400")
    assert raw(b"POST /hint HTTP/1.1\r\nContent-Length: 99999999\r\n\r\n{}").split(b" ")[1] in (b"400", b"413")
    big = b"GET /" + b"a" * 100000 + b" HTTP/1.1\r\n\r\n"
    try:
        reply = raw(big)
    except OSError:
        reply = b""
    assert reply == b"" or reply.split(b" ")[1] in (b"400", b"413", b"414")
    raw(b"GET /xqueues HTT", wait=False)          # hangs up in the middle of the request line
    assert call(port, "GET", "/policy") == (200, {"policy": 1})
