"""The daemon's HTTP control plane (reference service/server/src/server.cpp:28-39 routes,
:204-543 handlers; JSON field names of service/common/src/convert.cpp:7-17): the routes the
reference's command-line client uses, driven here with http.client against a running xserver
and a client process on the host adapter. CPU only.

What the daemon has to say - routes, field names, status codes, every literal answer - is not
typed into this file: it comes from tests/golden/http_contract.json, which
tests/golden/make_http_contract.py extracts from the text of the reference's two source files.
The tests say which request should draw which of the reference's answers (by a word of it) and
check that every answer of a handler that a client can provoke has been drawn."""
import http.client
import json
import os
import socket
import subprocess
import tempfile
import time

import pytest

from test_daemon import XSERVER, client

CONTRACT = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "http_contract.json")))
STATUS_FIELDS = set(CONTRACT["status_fields"])


def said(handler, word):
    """The one (status, body) among the reference's literal answers of `handler` that has `word` in it."""
    hits = [(status, body) for status, body in CONTRACT["handlers"][handler]["answers"]
            if body is not None and any(word in str(v) for v in body.values())]
    assert len(hits) == 1, (handler, word, hits)
    return hits[0]


def bare(handler):
    """Status codes that `handler` answers without a body."""
    return {status for status, body in CONTRACT["handlers"][handler]["answers"] if body is None}


def all_answers(handler, but=()):
    return {(status, json.dumps(body, sort_keys=True)) for status, body in CONTRACT["handlers"][handler]["answers"]
            if body is not None and not any(w in str(v) for w in but for v in body.values())}


class Drawn(set):
    """(status, body) pairs a test has drawn from the daemon, for the coverage check."""
    def take(self, answer):
        self.add((answer[0], json.dumps(answer[1], sort_keys=True)))
        return answer


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
    status, listing = call(port, "GET", "/xqueues")
    assert status == 200 and sorted(listing) == CONTRACT["handlers"]["GetXQueues"]["response_keys"]
    assert all(v == [] for v in listing.values())
    status, policy = call(port, "GET", "/policy")
    assert status == 200 and sorted(policy) == CONTRACT["handlers"]["GetSchedulerPolicy"]["response_keys"]
    assert policy["policy"] == 1                                         # kPolicyHighestPriorityFirst
    assert call(port, "GET", "/nothing-here")[0] == 404
    assert {call(port, "GET", "/xqueue/zz")[0], call(port, "GET", "/xqueue/0xabc")[0]} == bare("GetXQueue") == {400, 404}
    # every route the reference registers is served (a route that is not would answer 404 to everything)
    assert sorted(map(tuple, CONTRACT["routes"])) == [("GET", "/policy"), ("GET", "/xqueue/:handle"), ("GET", "/xqueues"),
                                                      ("POST", "/config/:handle"), ("POST", "/hint"), ("POST", "/policy")]
    assert call(port, "POST", "/hint", {})[0] != 404 and call(port, "POST", "/policy")[0] != 404
    assert call(port, "POST", "/config/1f")[0] != 405


def test_queue_listing_and_lookup(daemon_http):
    port, env = daemon_http
    busy, pid, listed = busy_client(port, env)
    try:
        assert set(listed) == STATUS_FIELDS
        for field, kind in CONTRACT["status_fields"].items():
            assert isinstance(listed[field], bool if kind == "boolean" else int) and (kind == "boolean" or not isinstance(listed[field], bool)), field
        assert listed["level"] == 1 and listed["threshold"] == 16 and listed["batch_size"] == 8
        assert listed["suspended"] is False
        status, body = call(port, "GET", "/xqueues")
        assert [p["pid"] for p in body["processes"]] == [pid]
        assert sorted(body["processes"][0]) == CONTRACT["handlers"]["GetXQueues"]["process_keys"]
        assert "daemon_client.py" in body["processes"][0]["cmdline"]
        for spelling in ("%x", "0x%x", "%X"):
            status, one = call(port, "GET", "/xqueue/" + spelling % listed["handle"])
            assert status == 200 and sorted(one) == CONTRACT["handlers"]["GetXQueue"]["response_keys"]
            assert sorted(one["process"]) == CONTRACT["handlers"]["GetXQueue"]["process_keys"]
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
        handler, drawn = "PostXQueueConfig", Drawn()
        assert sorted(p for p in CONTRACT["handlers"][handler]["query_parameters"]) == ["batch_size", "level", "threshold"]
        assert drawn.take(call(port, "POST", path)) == said(handler, "no change")
        assert drawn.take(call(port, "POST", path + "?level=0")) == said(handler, "level")
        assert drawn.take(call(port, "POST", path + "?level=4")) == said(handler, "level")
        assert drawn.take(call(port, "POST", path + "?threshold=0")) == said(handler, "invalid command threshold")
        assert drawn.take(call(port, "POST", path + "?batch_size=-2")) == said(handler, "invalid command batch size")
        assert drawn.take(call(port, "POST", path + "?threshold=8")) == said(handler, "less than")
        assert drawn.take(call(port, "POST", "/config/123456?threshold=4")) == said(handler, "not found")
        assert call(port, "POST", "/config/0")[0] in bare(handler)

        assert drawn.take(call(port, "POST", path + "?threshold=6&batch_size=3")) == said(handler, "success")
        assert drawn == all_answers(handler), "an answer of the reference's handler was never drawn"
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
    handler = "PostSchedulerPolicy"
    assert CONTRACT["handlers"][handler]["query_parameters"] == ["policy"] and bare(handler) == {400}
    assert call(port, "POST", "/policy")[0] in bare(handler)
    assert call(port, "POST", "/policy?policy=0")[0] in bare(handler)
    assert call(port, "POST", "/policy?policy=99")[0] in bare(handler)
    assert call(port, "POST", "/policy?policy=4") == said(handler, "success")   # utilization partition
    deadline = time.time() + 2
    while time.time() < deadline and call(port, "GET", "/policy")[1]["policy"] != 4:
        time.sleep(0.02)
    assert call(port, "GET", "/policy") == (200, {"policy": 4})


def test_hint_validation(daemon_http):
    port, _ = daemon_http
    handler, drawn = "PostHint", Drawn()
    post = lambda body: drawn.take(call(port, "POST", "/hint", body))  # noqa: E731
    assert set(CONTRACT["handlers"][handler]["request_keys"]) == {"hint_type", "handle", "priority", "pid", "utilization",
                                                                  "timeslice", "display"}
    assert post({}) == said(handler, "missing hint type")
    assert post({"hint_type": 0}) == said(handler, "invalid hint type")
    assert post({"hint_type": 99}) == said(handler, "invalid hint type")
    assert post({"hint_type": 1, "priority": 3}) == said(handler, "invalid handle")
    assert post({"hint_type": 1, "handle": 5}) == said(handler, "missing priority")
    assert post({"hint_type": 1, "handle": 5, "priority": 1000}) == said(handler, "invalid priority")
    assert post({"hint_type": 2, "utilization": 30}) == said(handler, "is required")
    assert post({"hint_type": 2, "pid": 7}) == said(handler, "missing utilization")
    assert post({"hint_type": 2, "pid": 7, "utilization": 101}) == said(handler, "invalid utilization")
    assert post({"hint_type": 3}) == said(handler, "missing timeslice")
    assert post({"hint_type": 3, "timeslice": 0}) == said(handler, "invalid timeslice")
    assert post({"hint_type": 3, "timeslice": 5000}) == said(handler, "success")
    assert post({"hint_type": 2, "pid": 7, "utilization": 40}) == said(handler, "success")
    window_active = 7                                  # kHintTypeWindowActive, the last hint the handler knows
    assert post({"hint_type": window_active, "display": 1}) == said(handler, "missing pid")
    assert post({"hint_type": window_active, "pid": 7}) == said(handler, "missing display")
    assert post({"hint_type": window_active, "pid": 7, "display": 1}) == said(handler, "success")
    # everything the handler can say has been said, but for the line behind its switch that no request reaches
    assert drawn == all_answers(handler, but=("internal server error",))
    status, _ = call(port, "POST", "/hint")
    assert status in bare(handler)
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
        assert call(port, "POST", "/hint", {"hint_type": 1, "handle": handle, "priority": -5}) == said("PostHint", "success")
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


def test_a_client_that_drips_its_request_does_not_hold_the_control_plane(daemon_http):
    """One thread serves every client: a request has a deadline as a whole (3 s), not only per
    read. A client that sends a byte every half second gets 408 and is dropped; the next
    client is served."""
    port, _ = daemon_http
    s = socket.create_connection(("127.0.0.1", port), timeout=10)
    started = time.time()
    reply = b""
    try:
        for byte in b"POST /hint HTTP/1.1\r\nContent-Length: 30\r\n\r\n{\"hint_type\": 3,":
            try:
                s.sendall(bytes([byte]))
            except OSError:
                break
            time.sleep(0.5 if time.time() - started > 0.2 else 0.01)
            if time.time() - started > 8:
                break
            s.settimeout(0.001)
            try:
                reply = s.recv(4096)
                if reply:
                    break
            except OSError:
                pass
        if not reply:
            s.settimeout(3)
            try:
                reply = s.recv(4096)
            except OSError:
                reply = b""
    finally:
        s.close()
    assert time.time() - started < 6, "the dripping client was served for longer than the request deadline"
    assert reply == b"" or reply.split(b" ")[1] == b"408"
    assert call(port, "GET", "/policy") == (200, {"policy": 1})
