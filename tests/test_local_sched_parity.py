"""The LocalScheduler of this repository (event queue, worker, Status mirror, operation
ids, policy switch, timers) and through it every policy (HPF, LAX, HHPF, CHPF, UP, PUP,
KEDF, AWF, CFS, MLFQ) against
(a) golden vectors recorded from the reference's own LocalScheduler
    (tests/golden/local_sched_vectors.json, written by
    tests/golden/make_local_sched_vectors.py from oracle/_ref/libsched_ref.so), and
(b) the live reference build, when oracle/_ref is present in this checkout.
Operations are compared exactly: id, pid, running set, suspended set, round by round."""
import json
import os
import time

import pytest

import local_sched_scripts as scripts
import sched_driver_api as api

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "local_sched_vectors.json")


def untuple(x):
    """Scripts as JSON gives them back (tuples become lists)."""
    return json.loads(json.dumps(x))


def as_script(js):
    return {"policy": js["policy"],
            "rounds": [[tuple(tuple(f) if isinstance(f, list) else f for f in e) for e in r]
                       for r in js["rounds"]]}


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def probe():
    if not os.path.exists(api.PROBE_LIB):
        pytest.fail("oracle/libsched_probe.so missing: run __graft_entry__.build()")
    os.environ["XLOG_LEVEL"] = "ERRO"
    return api.probe()


@pytest.fixture(scope="module")
def ref():
    r = api.ref()
    if r is None:
        pytest.skip("oracle/_ref not built here (reference tree absent)")
    os.environ["XLOG_LEVEL"] = "ERRO"
    return r


def test_fixture_covers_the_current_scripts(golden):
    current = scripts.all_scripts()
    assert set(golden) == set(current)
    for name, script in current.items():
        assert golden[name]["script"] == untuple(script), name


def test_fixture_is_not_trivial(golden):
    ops = [op for entry in golden.values() for rnd in entry["operations"] for op in rnd]
    assert len(ops) > 2500
    assert sum(1 for op in ops if op[3]) > 900        # rounds with something suspended
    assert sum(1 for op in ops if op[0] == 0) > 10    # operations for a process never announced
    assert max(op[0] for op in ops) > 30


@pytest.mark.parametrize("name", sorted(scripts.all_scripts()))
def test_operations_match_golden(probe, golden, name):
    entry = golden[name]
    assert scripts.play(probe, as_script(entry["script"])) == entry["operations"]


def test_operations_against_live_reference(probe, ref):
    for seed in range(200, 206):
        for policy in (scripts.HPF, scripts.LAX) + tuple(scripts.RANDOM_POLICIES.values()):
            script = scripts.random_script(seed, policy)
            assert scripts.play(probe, script) == scripts.play(ref, script), (seed, policy)


def test_wall_clock_policies_against_live_reference(probe, ref):
    """The time-sliced policies (queue and process shares with slices that end, fair share,
    feedback levels) on scripts whose pauses keep every comparison far from its threshold."""
    for name, script in scripts.more_policy_scripts().items():
        assert scripts.play(probe, script) == scripts.play(ref, script), name


def test_process_priority_policy_with_real_processes(probe, ref, monkeypatch):
    """CHPF reads /proc/<pid>/sched: this process and pid 1 run at a normal Linux priority
    (120, which the policy counts as -120), a pid that does not exist counts as 0 and wins."""
    monkeypatch.setattr(scripts, "PIDS", (os.getpid(), 1, 4190003))
    seen_suspended = 0
    for seed in range(400, 404):
        script = scripts.random_script(seed, scripts.CHPF)
        mine = scripts.play(probe, script)
        assert mine == scripts.play(ref, script), seed
        seen_suspended += sum(1 for rnd in mine for op in rnd if op[3])
    assert seen_suspended > 20


def timed_laxity_states(drv):
    """Two ready XQueues under LAX on a live worker: 3 has default priority, 4 has a laxity
    of 150 ms with a low priority before and a high one after. Returns the distinct
    (running, suspended) states seen up to 40 ms and up to 500 ms."""
    sched = drv.local(scripts.LAX)
    try:
        now_us = int(time.time() * 1e6)
        pid = scripts.owner(3)
        assert scripts.owner(4) != pid
        events = [("pc", pid, "bg"), ("pc", scripts.owner(4), "fg"),
                  ("qc", 3, ("dev", 1, 0), 2, 4, 2), ("qc", 4, ("dev", 1, 0), 2, 4, 2),
                  ("lax", pid, 4, 150_000, -3, 6)]
        for e in events:
            sched.recv(scripts.event_bytes(drv, e, {}))
        for xq in (3, 4):
            sched.recv(api.with_pid(drv.record("event_xqueue_ready", xq, now_us), scripts.owner(xq)))
        sched.run()
        time.sleep(0.04)
        early = sched.take()
        time.sleep(0.46)
        sched.stop()
        late = sched.take()
    finally:
        sched.close()

    def states(ops):
        seen = []
        for op in ops:
            _, _, op_pid, running, suspended = api.parse_sched_operation(op)
            s = (op_pid, tuple(running), tuple(suspended))
            if s not in seen:
                seen.append(s)
        return seen
    return states(early), states(early + late)


def test_laxity_timer_fires(probe):
    early, both = timed_laxity_states(probe)
    p3, p4 = scripts.owner(3), scripts.owner(4)
    assert early == [(p3, (3,), ()), (p4, (), (4,))]
    assert both == early + [(p3, (), (3,)), (p4, (4,), ())]


def test_laxity_timer_against_live_reference(probe, ref):
    assert timed_laxity_states(probe) == timed_laxity_states(ref)
