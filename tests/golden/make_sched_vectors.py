#!/usr/bin/env python3
"""Writes tests/golden/sched_vectors.json from the REFERENCE build of
oracle/sched_driver.cpp (oracle/_ref/libsched_ref.so, compiled from the reference's own
policy / wire-record sources in this container). The fixture holds inputs and the
reference's outputs only: scheduling decisions of HPF and LAX for seeded scenarios, and
the field bytes of every event / operation / hint record for fixed arguments.

    python tests/golden/make_sched_vectors.py
"""
import json
import os
import random
import sys

os.environ["XLOG_LEVEL"] = "ERRO"  # the reference logs every hint at INFO

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import sched_driver_api as api  # noqa: E402

HPF, LAX = 1, 8
PID = 4242  # records carry the producing pid; the fixture stores it and the test patches it in


def hpf_scenarios(rnd, count):
    out = []
    for _ in range(count):
        n = rnd.randint(1, 8)
        handles = rnd.sample(range(0x1000, 0x2000), n)
        queues = [(h, rnd.choice([0x200000001, 0x200000002]), rnd.random() < 0.6, 0) for h in handles]
        hints = [(h, rnd.choice([-400, -255, -3, 0, 1, 2, 5, 255, 300])) for h in handles if rnd.random() < 0.8]
        out.append({"queues": queues, "hints": hints})
    return out


def lax_scenarios(rnd, count, now_us):
    out = []
    far = 3600 * 10**6
    for _ in range(count):
        n = rnd.randint(1, 6)
        handles = rnd.sample(range(0x1000, 0x2000), n)
        queues = []
        hints = []
        for h in handles:
            ready = rnd.random() < 0.7
            # ready long ago (laxity used up) or in the far future (laxity not used up):
            # both are unambiguous whatever the exact "now" of the run is.
            ready_time = now_us - far if rnd.random() < 0.5 else now_us + far
            queues.append((h, 0x200000001, ready, ready_time))
            if rnd.random() < 0.75:
                hints.append((h, rnd.choice([1000, 50000, 10**6]), rnd.choice([-5, 0, 1]), rnd.choice([2, 7, 9])))
        out.append({"queues": queues, "hints": hints})
    return out


def main():
    drv = api.ref()
    assert drv is not None, "build oracle/_ref first (make -C oracle ref)"
    rnd = random.Random(20240607)
    import time
    now_us = int(time.time() * 1e6)  # LAX reads the system clock; ready times are +-1 h around it

    vec = {"pid_note": "meta.pid bytes are replaced by the test with its own pid", "hpf": [], "lax": [],
           "records": {}, "names": {}}
    for sc in hpf_scenarios(rnd, 60):
        p = drv.policy(HPF)
        for h, prio in sc["hints"]:
            p.priority(h, prio)
        dec, timers = p.sched(sc["queues"])
        p.close()
        vec["hpf"].append({"queues": sc["queues"], "hints": sc["hints"], "decisions": dec, "timers": timers})
    for sc in lax_scenarios(rnd, 60, now_us):
        p = drv.policy(LAX)
        for h, lax, lp, cp in sc["hints"]:
            p.laxity(h, lax, lp, cp)
        dec, timers = p.sched(sc["queues"])
        p.close()
        # store ready times relative to "now" so the fixture can be replayed at any time
        rel = [(h, d, r, t - now_us) for (h, d, r, t) in sc["queues"]]
        vec["lax"].append({"queues_rel": rel, "hints": sc["hints"], "decisions": dec,
                           "timers_rel": [t - now_us for t in timers]})

    args = {
        "hint_priority": [0x1122334455667788, -7],
        "hint_utilization": [77, 0x1122334455667788, 35],
        "hint_timeslice": [5000],
        "hint_deadline": [0x1122334455667788, 123456],
        "hint_kdeadline": [3],
        "hint_laxity": [0x1122334455667788, 1000, -255, 9],
        "event_hint_priority": [0x1122334455667788, 12],
        "event_process_create": [b"python bench.py --gpus 1"],
        "event_process_destroy": [PID],
        "event_terminate": [],
        "event_xqueue_create": [0xAABBCCDDEEFF0011, 0x2000000C1, 2, 8, 4],
        "event_xqueue_config": [0xAABBCCDDEEFF0011, 0x2000000C1, 1, 16, 8],
        "event_xqueue_destroy": [0xAABBCCDDEEFF0011],
        "event_xqueue_idle": [0xAABBCCDDEEFF0011],
        "event_xqueue_ready": [0xAABBCCDDEEFF0011, 1717171717000000],
        "event_operation_complete": [99],
        "operation_config": [17, PID, 0xAABBCCDDEEFF0011, 2, 8, -1],
        "operation_terminate": [],
    }
    for name, a in args.items():
        data = api.masked(name, drv.record(name, *a))
        vec["records"][name] = {"args": [x.decode() if isinstance(x, bytes) else x for x in a],
                                "hex": data.hex()}
    so = drv.sched_operation(5, PID, [0x30, 0x10, 0x20], [0x50, 0x40])
    vec["records"]["operation_sched"] = {"args": [5, PID, [0x30, 0x10, 0x20], [0x50, 0x40]], "hex": so.hex()}
    so0 = drv.sched_operation(6, PID, [], [])
    vec["records"]["operation_sched_empty"] = {"args": [6, PID, [], []], "hex": so0.hex()}

    vec["names"]["policy"] = {str(t): drv.policy_name(t) for t in range(0, 13)}
    vec["names"]["policy_by_name"] = {n: drv.policy_type_by_name(n) for n in
                                      ["HPF", "hpf", "LAX", "lax", "KEDF", "CFS", "nope", ""]}
    vec["names"]["scheduler"] = {str(t): drv.scheduler_name(t) for t in range(0, 5)}
    vec["names"]["scheduler_by_name"] = {n: drv.scheduler_type_by_name(n) for n in ["APP", "lcl", "GLB", "x"]}
    vec["names"]["level"] = {str(t): drv.level_name(t) for t in range(0, 5)}
    vec["names"]["platform"] = {str(t): drv.platform_name(t) for t in range(0, 9)}
    vec["names"]["make_device"] = {"2,193": drv.make_device(2, 193), "1,0": drv.make_device(1, 0)}
    vec["producer_pid"] = os.getpid()

    with open(os.path.join(HERE, "sched_vectors.json"), "w") as f:
        json.dump(vec, f, separators=(",", ":"))
    print("wrote sched_vectors.json:", len(vec["hpf"]), "HPF and", len(vec["lax"]), "LAX scenarios,",
          len(vec["records"]), "records")


if __name__ == "__main__":
    main()
