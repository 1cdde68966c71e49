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
    ("ready_at", xq, time_us)                  XQueue ready since time_us after EPOCH_US (same in every run)
    ("idle", xq)                               XQueue idle
    ("prio", pid, xq, priority)                priority hint sent by pid
    ("lax", pid, xq, laxity_us, lax_prio, crit_prio)   laxity hint sent by pid
    ("util", pid, target_pid, xq, percent)     utilization hint (queue policies read xq, process ones target_pid)
    ("ts", pid, timeslice_us)                  timeslice hint
    ("ddl", pid, xq, deadline_us)              deadline hint
    ("kddl", pid, k)                           k of k-earliest-deadline-first
    ("win", pid, target_pid, display)          target_pid owns the active window of display
    ("sleep", milliseconds)                    wall-clock pause; must be the only event of its round
    ("done", pid)                              completion of the last operation pid was sent
    ("policy", type)                           SetPolicy; must be the only event of its round

Every XQueue has one owner process, owner(xq); the reference asserts on a destroy sent by
anyone else (sched/src/scheduler/local.cpp:303), so scripts never do that.
"""
import random
import time

from sched_driver_api import parse_sched_operation, with_pid

HPF, HHPF, CHPF, UP, PUP, KEDF, LAX, AWF, CFS, MLFQ = 1, 2, 3, 4, 5, 7, 8, 9, 10, 11
PIDS = (1001, 1002, 1003)
# policies whose decisions in random scripts do not depend on the wall clock (UP and PUP
# with slices of ten seconds)
RANDOM_POLICIES = {"hhpf": HHPF, "kedf": KEDF, "awf": AWF, "up": UP, "pup": PUP}
SECOND = 1_000_000
EPOCH_US = 1_700_000_000 * SECOND


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
    if policy in (UP, PUP):
        rounds.append([("ts", PIDS[0], 10 * SECOND)])  # slices that never end within a test
    hour = 3600 * SECOND
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
            elif kind == "ready" and policy == KEDF:
                events.append(("ready_at", xq, rng.choice([0, 500, 20_000, -hour])))
            elif kind == "ready":
                events.append(("ready", xq, rng.choice([0, -2 * 3600 * SECOND])))
            elif kind == "idle":
                events.append(("idle", xq))
            elif kind == "hint":
                if policy == LAX and rng.random() < 0.8:
                    events.append(("lax", rng.choice(PIDS), xq, rng.choice([-1, SECOND, 3600 * SECOND]),
                                   rng.randint(-8, 8), rng.randint(-8, 8)))
                elif policy == KEDF and rng.random() < 0.9:
                    if rng.random() < 0.25:
                        events.append(("kddl", rng.choice(PIDS), rng.randint(0, 4)))
                    else:
                        events.append(("ddl", rng.choice(PIDS), xq, rng.choice([500, 1000, 50_000, SECOND])))
                elif policy == AWF and rng.random() < 0.9:
                    events.append(("win", rng.choice(PIDS), rng.choice(PIDS + (0,)), rng.randint(0, 2)))
                elif policy in (UP, PUP) and rng.random() < 0.9:
                    events.append(("util", rng.choice(PIDS), rng.choice(PIDS + (0,)), xq,
                                   rng.choice([-5, 0, 10, 30, 70, 100, 105])))
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


def more_policy_scripts():
    """The policies beyond HPF and LAX. The time-sliced ones decide by the wall clock;
    their scripts keep every comparison far from its threshold (slices of ten seconds
    that never end within a test, or of 100 us followed by a pause of tens of milliseconds)."""
    gpu0, gpu1 = ("dev", 1, 0), ("dev", 1, 1)
    HOUR = 3600 * SECOND
    three = [("pc", 1001, "a"), ("pc", 1002, "b"), ("pc", 1003, "c")]
    six_queues = [("qc", q, gpu0 if q < 4 else gpu1, 1, 4, 2) for q in range(6)]
    return {
        "hhpf_one_bar_for_all_devices": {"policy": HHPF, "rounds": [
            three, six_queues,
            [("prio", 1001, 0, 2), ("prio", 1001, 4, 7), ("prio", 1001, 5, -300), ("prio", 1001, 1, 300)],
            [("ready", 0, 0), ("ready", 5, 0)],
            [("ready", 4, 0)],
            [("idle", 4), ("ready", 1, 0)],
            [("idle", 1), ("idle", 0), ("idle", 5)],
        ]},
        # 1001-1003 are not expected to exist under /proc: all priorities read as 0, nobody waits;
        # priority hints mean nothing to this policy (real processes: see the live test)
        "chpf_processes_without_proc_entry": {"policy": CHPF, "rounds": [
            three, six_queues,
            [("ready", 0, 0), ("prio", 1001, 1, 9)],
            [("ready", 1, 0), ("ready", 5, 0)],
            [("idle", 0)],
        ]},
        "kedf_k1_then_k3": {"policy": KEDF, "rounds": [
            three, six_queues,
            [("ddl", 1001, 0, 50_000), ("ddl", 1001, 1, 10_000), ("ddl", 1001, 2, 30_000), ("ddl", 1001, 4, 5_000)],
            [("ready_at", 0, 0), ("ready_at", 1, 0), ("ready_at", 2, 0)],
            [("ready_at", 4, 1000), ("ready_at", 3, -HOUR)],
            [("kddl", 1002, 3)],
            [("kddl", 1002, 0), ("idle", 1)],
            [("ddl", 1003, 3, 1), ("lax", 1003, 3, 5, 1, 1)],
            [("qd", 4), ("kddl", 1002, 2)],
        ]},
        "awf_active_window_per_display": {"policy": AWF, "rounds": [
            three, six_queues,
            [("ready", 0, 0), ("ready", 1, 0), ("ready", 2, 0)],
            [("win", 1003, owner(1), 0)],
            [("win", 1003, owner(2), 1)],
            [("win", 1003, owner(0), 0)],
            [("win", 1003, 0, 0), ("idle", 0), ("idle", 2)],
            [("ready", 5, 0)],
            [("pd", owner(2))],
        ]},
        "up_slices_that_never_end": {"policy": UP, "rounds": [
            three, six_queues,
            [("ts", 1001, 10 * SECOND), ("util", 1001, 0, 1, 30), ("util", 1001, 0, 3, 70), ("util", 1001, 0, 4, 101)],
            [("ready", 0, 0)],
            [("ready", 1, 0), ("ready", 3, 0)],
            [("idle", 1)],
            [("ready", 1, 0), ("idle", 3)],
            [("idle", 1)],
            [("ready", 3, 0), ("util", 1002, 0, 0, 50)],
            [("qd", 3)],
            [("ready", 0, 0)],
        ]},
        "up_slices_that_always_end": {"policy": UP, "rounds": [
            three, six_queues,
            [("ts", 1001, 100), ("util", 1001, 0, 1, 30), ("util", 1001, 0, 3, 70), ("util", 1001, 0, 5, 0)],
            [("ready", 1, 0), ("ready", 3, 0), ("ready", 5, 0), ("ready", 2, 0)],
            [("sleep", 20)], [("done", 1001)],
            [("sleep", 20)], [("done", 1002)],
            [("sleep", 20)], [("idle", 5)],
            [("sleep", 20)], [("idle", 1), ("idle", 3)],
            [("sleep", 20)], [("ready", 3, 0)],
        ]},
        "pup_slices_that_never_end": {"policy": PUP, "rounds": [
            three, six_queues,
            [("ts", 1001, 10 * SECOND), ("util", 1001, 1002, 0, 40), ("util", 1001, 0, 0, 90), ("util", 1001, 1003, 0, 150)],
            [("ready", 0, 0)],
            [("ready", 1, 0), ("ready", 2, 0)],
            [("idle", 0), ("idle", 3)],
            [("ready", 3, 0)],
            [("idle", 1), ("idle", 4)],
            [("pd", 1003)],
            [("ready", 4, 0)],
        ]},
        "pup_slices_that_always_end": {"policy": PUP, "rounds": [
            three, six_queues,
            [("ts", 1001, 100), ("ts", 1001, 50), ("util", 1001, 1001, 0, 10)],
            [("ready", 0, 0), ("ready", 1, 0), ("ready", 2, 0)],
            [("sleep", 20)], [("done", 1001)],
            [("sleep", 20)], [("done", 1001)],
            [("sleep", 20)], [("idle", 1), ("idle", 4)],
            [("sleep", 20)], [("done", 1001)],
            [("sleep", 20)], [("idle", 0), ("idle", 3), ("idle", 2), ("idle", 5)],
            [("sleep", 20)], [("ready", 2, 0)],
        ]},
        "cfs_weights_and_turns": {"policy": CFS, "rounds": [
            three, [("qc", 0, gpu0, 1, 4, 2), ("qc", 1, gpu0, 1, 4, 2), ("qc", 4, gpu1, 1, 4, 2)],
            [("prio", 1001, 1, 8)],                   # weight 1024 * 1.2^8 = 4403: its clock runs 4.3 times slower
            [("ready", 0, 0)],
            [("sleep", 40)], [("ready", 1, 0), ("ready", 4, 0)],    # 0 has run 40 ms; 1 starts at 0's clock... and wins ties by order
            [("sleep", 40)], [("done", 1001)],
            [("sleep", 120)], [("done", 1001)],
            [("sleep", 40)], [("idle", 0)],
            [("sleep", 40)], [("ready", 0, 0)],
        ]},
        "mlfq_drop_and_rise": {"policy": MLFQ, "rounds": [
            three, [("qc", 0, gpu0, 1, 4, 2), ("qc", 1, gpu0, 1, 4, 2), ("qc", 4, gpu1, 1, 4, 2)],
            [("ready", 0, 0)],
            [("sleep", 2)], [("ready", 1, 0)],          # 0 has used 2 of its 10 ms
            [("sleep", 14)], [("done", 1001)],          # 0 used 16 ms: drops to level 1, 1 runs
            [("sleep", 14)], [("done", 1001)],          # 1 used 14 ms: drops too; 0 has been pending longer
            [("sleep", 3)], [("ready", 4, 0)],
            [("sleep", 30)], [("done", 1001)],          # 0 used 33 of 20 ms at level 1: drops to 2
            [("sleep", 140)], [("done", 1001)],         # everybody's level is older than 100 ms
        ]},
    }


def all_scripts():
    scripts = fixed_scripts()
    scripts.update(more_policy_scripts())
    for seed in range(6):
        scripts["random_hpf_%d" % seed] = random_script(seed, HPF)
        scripts["random_lax_%d" % seed] = random_script(100 + seed, LAX)
    for seed in range(3):
        for name, policy in RANDOM_POLICIES.items():
            scripts["random_%s_%d" % (name, seed)] = random_script(300 + seed, policy)
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
    if kind == "ready_at":
        return with_pid(drv.record("event_xqueue_ready", event[1], EPOCH_US + event[2]), owner(event[1]))
    if kind == "idle":
        return with_pid(drv.record("event_xqueue_idle", event[1]), owner(event[1]))
    if kind == "prio":
        return with_pid(drv.record("event_hint_priority", event[2], event[3]), event[1])
    if kind == "lax":
        return with_pid(drv.hint_event(drv.record("hint_laxity", *event[2:])), event[1])
    if kind == "util":
        return with_pid(drv.hint_event(drv.record("hint_utilization", event[2], event[3], event[4])), event[1])
    if kind == "ts":
        return with_pid(drv.hint_event(drv.record("hint_timeslice", event[2])), event[1])
    if kind == "ddl":
        return with_pid(drv.hint_event(drv.record("hint_deadline", event[2], event[3])), event[1])
    if kind == "kddl":
        return with_pid(drv.hint_event(drv.record("hint_kdeadline", event[2])), event[1])
    if kind == "win":
        return with_pid(drv.hint_event(drv.record("hint_window_active", event[2], event[3])), event[1])
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
            if events[0][0] == "sleep":
                assert len(events) == 1
                time.sleep(events[0][1] / 1000.0)
                ops = []
            elif events[0][0] == "policy":
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
