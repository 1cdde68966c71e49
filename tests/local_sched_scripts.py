"""Event scripts for the LocalScheduler parity tests and the runner that plays one on a
LocalScheduler of either build (tests/sched_driver_api.py). Test helper.

A script is {"policy": type, "rounds": [[event, ...], ...]}; each round is played as
exactly one scheduling round (see _Local.round), so the operations that come out, their
ids included, do not depend on thread timing. Events are tuples:

    ("pc", pid, cmdline)                       process create
    ("pd", pid)                                process destroy
    ("qc", xq, device, level, threshold, batch)   XQueue create   (sent by the owner of xq)
    ("qu", xq, device, level, threshold, batch)   XQueue config update
    ("qd", xq)                                 XQueue destroy
    ("ready", xq, offset_us)                   XQueue ready since now + offset_us
    ("idle", xq)                               XQueue idle
    ("prio", pid, xq, priority)                priority hint sent by pid
    ("lax", pid, xq, laxity_us, lax_prio, crit_prio)   laxity hint sent by pid
    ("done", pid)                              completion of the last operation pid was sent
    ("policy", type)                           SetPolicy; must be the only event of its round

Every XQueue has one owner process, owner(xq); the reference asserts on a destroy sent by
anyone else (sched/src/scheduler/local.cpp:303), so scripts never do that.
"""
import random
import time

from sched_driver_api import parse_sched_operation, with_pid

HPF, LAX = 1, 8
PIDS = (1001, 1002, 1003)
SECOND = 1_000_000


def owner(xq):
    return PIDS[xq % len(PIDS)]


def fixed_scripts():
    gpu0, gpu1 = ("dev", 1, 0), ("dev", 1, 1)
    return {
        "hpf_two_processes": {"policy": HPF, "rounds": [
            [("pc", 1001, "train"), ("pc", 1002, "serve")],
            [("qc", 3, gpu0, 2, 16, 8), ("qc", 4, gpu0, 1, 4, 2)],
            [("ready", 3, 0)],
            [("prio", 1002, 4, 5), ("ready", 4, 0)],
            [("done", 1001), ("done", 1002), ("idle", 4)],
            [("ready", 4, 0), ("idle", 3)],
            [("qd", 4)],
            [("pd", 1001), ("pd", 1002)],
        ]},
        "hpf_two_devices": {"policy": HPF, "rounds": [
            [("pc", 1001, "a"), ("pc", 1002, "b"), ("pc", 1003, "c")],
            [("qc", 0, gpu0, 1, 4, 2), ("qc", 1, gpu1, 1, 4, 2), ("qc", 2, gpu0, 2, 8, 4), ("qc", 3, gpu1, 2, 8, 4)],
            [("prio", 1003, 0, 3), ("prio", 1003, 1, -3), ("prio", 1003, 2, 1), ("prio", 1003, 3, 1)],
            [("ready", 0, 0), ("ready", 1, 0), ("ready", 2, 0), ("ready", 3, 0)],
            [("idle", 0)],
            [("qu", 1, gpu0, 1, 2, 1)],
            [("idle", 3), ("ready", 0, 0)],
        ]},
        "hpf_ready_before_create_and_unknown_process": {"policy": HPF, "rounds": [
            [("ready", 5, 0)],
            [("qc", 5, gpu0, 1, 4, 2), ("ready", 6, 0), ("prio", 1001, 6, 2)],
            [("pc", 1003, "late"), ("pc", 1001, "late too")],
            [("idle", 6)],
            [("pd", 1003)],
            [("ready", 5, 0), ("ready", 6, 0)],
            [("pc", 1003, "again"), ("done", 1001)],
        ]},
        "lax_critical_and_relaxed": {"policy": LAX, "rounds": [
            [("pc", 1001, "bg"), ("pc", 1002, "fg")],
            [("qc", 3, gpu0, 2, 16, 8), ("qc", 4, gpu0, 2, 4, 2)],
            [("lax", 1002, 4, 3600 * SECOND, -2, 7)],
            [("ready", 3, 0), ("ready", 4, 0)],          # 4 is far from its limit: low priority
            [("idle", 4)],
            [("ready", 4, -2 * 3600 * SECOND)],          # 4 is past its limit: critical
            [("lax", 1002, 3, SECOND, 9, 9)],
            [("lax", 1002, 3, -1, -4, -4)],              # negative laxity: never critical
            [("idle", 3), ("idle", 4)],
        ]},
        "switch_policy": {"policy": HPF, "rounds": [
            [("pc", 1001, "a"), ("pc", 1002, "b")],
            [("qc", 3, gpu0, 1, 4, 2), ("qc", 4, gpu0, 1, 4, 2), ("ready", 3, 0), ("ready", 4, 0)],
            [("prio", 1001, 3, 4)],
            [("policy", LAX)],
            [("lax", 1001, 4, 3600 * SECOND, 6, 6)],
            [("policy", HPF)],
            [("prio", 1001, 4, -1)],
        ]},
    }


def random_script(seed, policy):
    rng = random.Random(seed)
    devices = [("dev", 1, 0), ("dev", 1, 1), ("dev", 2, 0)]
    queues = list(range(6))
    rounds = [[("pc", pid, "proc %d" % pid) for pid in PIDS if rng.random() < 0.8]]
    for _ in range(40):
        events = []
        for _ in range(rng.randint(1, 4)):
            xq = rng.choice(queues)
            kind = rng.choices(["qc", "qu", "qd", "ready", "idle", "hint", "done", "pc", "pd"],
                               [3, 1, 1, 6, 5, 4, 2, 1, 1])[0]
            if kind in ("qc", "qu"):
                events.append((kind, xq, rng.choice(devices), rng.randint(1, 3), rng.choice([2, 4, 16]),
                               rng.choice([1, 2, 8])))
            elif kind == "qd":
                events.append(("qd", xq))
            elif kind == "ready":
                events.append(("ready", xq, rng.choice([0, -2 * 3600 * SECOND])))
            elif kind == "idle":
                events.append(("idle", xq))
            elif kind == "hint":
                if policy == LAX and rng.random() < 0.8:
                    events.append(("lax", rng.choice(PIDS), xq, rng.choice([-1, SECOND, 3600 * SECOND]),
                                   rng.randint(-8, 8), rng.randint(-8, 8)))
                else:
                    events.append(("prio", rng.choice(PIDS), xq, rng.randint(-8, 8)))
            elif kind == "done":
                events.append(("done", rng.choice(PIDS)))
            elif kind == "pc":
                events.append(("pc", rng.choice(PIDS), "proc again"))
            else:
                events.append(("pd", rng.choice(PIDS)))
        rounds.append(events)
    return {"policy": policy, "rounds": rounds}


def all_scripts():
    scripts = fixed_scripts()
    for seed in range(6):
        scripts["random_hpf_%d" % seed] = random_script(seed, HPF)
        scripts["random_lax_%d" % seed] = random_script(100 + seed, LAX)
    return scripts


def event_bytes(drv, event, last_id):
    """Wire bytes of one script event, or None when it has nothing to send."""
    kind = event[0]
    dev = lambda d: drv.make_device(d[1], d[2])
    if kind == "pc":
        return with_pid(drv.record("event_process_create", event[2].encode()), event[1])
    if kind == "pd":
        return with_pid(drv.record("event_process_destroy", event[1]), event[1])
    if kind == "qc":
        return with_pid(drv.record("event_xqueue_create", event[1], dev(event[2]), *event[3:]), owner(event[1]))
    if kind == "qu":
        return with_pid(drv.record("event_xqueue_config", event[1], dev(event[2]), *event[3:]), owner(event[1]))
    if kind == "qd":
        return with_pid(drv.record("event_xqueue_destroy", event[1]), owner(event[1]))
    if kind == "ready":
        now_us = int(time.time() * 1e6)
        return with_pid(drv.record("event_xqueue_ready", event[1], now_us + event[2]), owner(event[1]))
    if kind == "idle":
        return with_pid(drv.record("event_xqueue_idle", event[1]), owner(event[1]))
    if kind == "prio":
        return with_pid(drv.record("event_hint_priority", event[2], event[3]), event[1])
    if kind == "lax":
        return with_pid(drv.hint_event(drv.record("hint_laxity", *event[2:])), event[1])
    if kind == "done":
        if last_id.get(event[1], 0) == 0:
            return None
        return with_pid(drv.record("event_operation_complete", last_id[event[1]]), event[1])
    raise ValueError(kind)


def play(drv, script):
    """Operations of every round as [[id, pid, running, suspended], ...] per round."""
    sched = drv.local(script["policy"])
    last_id, out = {}, []
    try:
        for events in script["rounds"]:
            if events[0][0] == "policy":
                assert len(events) == 1
                sched.set_policy(events[0][1])
                sched.stop()
                ops = sched.take()
            else:
                wire = []
                for event in events:
                    data = event_bytes(drv, event, last_id)
                    if data is not None:
                        wire.append(data)
                    if event[0] == "pd":
                        last_id.pop(event[1], None)
                ops = sched.round(wire)
            parsed = []
            for op in ops:
                op_id, op_type, pid, running, suspended = parse_sched_operation(op)
                assert op_type == 2  # kOperationSched
                if op_id:
                    last_id[pid] = op_id
                parsed.append([op_id, pid, running, suspended])
            out.append(parsed)
    finally:
        sched.close()
    return out
