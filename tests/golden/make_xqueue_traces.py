#!/usr/bin/env python3
"""Writes tests/golden/xqueue_traces.json from the REFERENCE's XQueue core
(oracle/_ref/libxqueue_ref.so: the reference's own preempt/, sched/, protocol/ and utils/
sources compiled in this container, over the recording hardware queue of
oracle/xqueue_probe.cpp). For every script the fixture holds the inputs (launch
configuration and the list of actions) and, after each action, the reference's outputs: the
trace of calls it made on the adapter and the XQueue state it reports.

    python tests/golden/make_xqueue_traces.py
"""
import json
import os
import sys

os.environ["XLOG_LEVEL"] = "ERRO"

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, ROOT)
import xqueue_trace_driver as drv  # noqa: E402
from oracle.xqueue_model import XQueueModel  # noqa: E402  (only bounds `complete` targets)

RANDOM_SEEDS = range(24)


def run(core, thr, batch, level, actions):
    s = drv.Session(core, thr, batch, level)
    steps = []
    for act in actions:
        s.apply(act)
        trace = s.settle(quiet=0.05)
        steps.append({"action": act, "trace_len": len(trace), "state": s.state()})
    final = s.trace()
    s.close(drv.last_index(actions))
    # the trace only grows, so the per-step prefix lengths and the final trace hold it all
    return {"threshold": thr, "batch": batch, "level": level, "steps": steps, "trace": final}


def main():
    core = drv.Core.reference()
    out = {}
    for name, (thr, batch, level, actions) in drv.fixed_scripts().items():
        out[name] = run(core, thr, batch, level, actions)
    for seed in RANDOM_SEEDS:
        thr, batch, level, actions = drv.random_script(seed, XQueueModel)
        out[f"random_{seed}"] = run(core, thr, batch, level, actions)
    # every script twice: a fixture is only worth keeping if the reference repeats itself
    for name, rec in out.items():
        again = run(core, rec["threshold"], rec["batch"], rec["level"], [s["action"] for s in rec["steps"]])
        assert again == rec, f"reference not deterministic on {name}"
    path = os.path.join(HERE, "xqueue_traces.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(f"wrote {path}: {len(out)} scripts, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
