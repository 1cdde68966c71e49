#!/usr/bin/env python3
"""Writes tests/golden/local_sched_vectors.json from the REFERENCE's own LocalScheduler
(sched/src/scheduler/local.cpp compiled where it lies into oracle/_ref/libsched_ref.so, in
this container). The fixture holds, for every script of tests/local_sched_scripts.py, the
script itself and the operations the reference scheduler executed in each round:
[operation id, pid, running XQueues, suspended XQueues].

    python tests/golden/make_local_sched_vectors.py
"""
import json
import os
import sys

os.environ["XLOG_LEVEL"] = "ERRO"

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import local_sched_scripts as scripts  # noqa: E402
import sched_driver_api as api  # noqa: E402


def main():
    ref = api.ref()
    if ref is None:
        sys.exit("oracle/_ref/libsched_ref.so not built (needs the reference tree)")
    out = {}
    for name, script in scripts.all_scripts().items():
        first, second = scripts.play(ref, script), scripts.play(ref, script)
        assert first == second, "script %s is not deterministic on the reference" % name
        out[name] = {"script": script, "operations": first}
    path = os.path.join(HERE, "local_sched_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
        f.write("\n")
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "scripts")


if __name__ == "__main__":
    main()
