"""The interception shim on the GPU: an unmodified HIP program gives the same results with and
without the shim in front of the runtime, and the shim's counters show that its stream work
really went through XQueues.

`shim_app` and `shim_app_plain` are built from tests/shim_app.hip; the first is linked against
libshimhip.so ahead of the HIP runtime. Each check of the program prints a checksum and compares
it with a value computed on the host, so "ok" lines are results that are right, and equal output
of the two programs is the parity statement."""
import os
import re
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "xsched_amd", "lib")
MODULE = os.path.join(LIB, "shim_module.co")
CHECKS = 14  # lines the program prints, "done" included


def run(binary, args, env_extra, timeout=120):
    env = dict(os.environ)
    for k in list(env):
        if k.startswith("XSCHED_"):
            del env[k]
    env.update(env_extra)
    print(f"running {binary} {args} with {env_extra}", flush=True)
    proc = subprocess.run([os.path.join(LIB, binary)] + args, env=env, capture_output=True, text=True,
                          timeout=timeout)
    assert proc.returncode == 0, (proc.returncode, proc.stdout[-2000:], proc.stderr[-2000:])
    return proc.stdout, proc.stderr


def stats_of(stderr):
    m = re.search(r"\[xsched shim\] (.*)", stderr)
    assert m, stderr[-2000:]
    return {k: int(v) for k, v in (item.split("=") for item in m.group(1).split())}


def shim_env(level, **more):
    env = {"XSCHED_AUTO_XQUEUE": "ON", "XSCHED_AUTO_XQUEUE_LEVEL": str(level), "XSCHED_SCHEDULER": "LCL",
           "XSCHED_POLICY": "HPF", "XSCHED_SHIM_STATS": "1", "XLOG_LEVEL": "WARN"}
    env.update(more)
    return env


@pytest.fixture(scope="module")
def plain_output():
    out, _ = run("shim_app_plain", [MODULE], {})
    lines = out.strip().splitlines()
    assert len(lines) == CHECKS and lines[-1] == "done", out
    for line in lines[:-1]:
        assert line.endswith(" ok"), line
    return out


@pytest.mark.parametrize("level,threshold,batch", [(1, 16, 8), (1, 2, 1), (2, 16, 8)])
def test_same_results_through_xqueues(plain_output, level, threshold, batch):
    out, err = run("shim_app", [MODULE], shim_env(level, XSCHED_AUTO_XQUEUE_THRESHOLD=str(threshold),
                                                  XSCHED_AUTO_XQUEUE_BATCH_SIZE=str(batch)))
    assert out == plain_output
    s = stats_of(err)
    # 3 saxpy + 2 argument shapes + 301 counter kernels + 2 spins + 4 adds on streams (checks 4-6)
    # + 2 * 400 from the threads + 3 module launches; the one null-stream launch goes straight through
    assert s["kernel_cmds"] == 3 + 2 + 301 + (1 + 2) + (1 + 1) + (1 + 1 + 1) + 800 + 3
    assert s["kernel_drained"] == 0 and s["kernel_direct"] == 1
    assert s["known_kernels"] >= 7 + 2
    assert s["event_cmds"] == 3 and s["event_waits"] == 1
    # pinned and device-to-device copies and every fill are commands; pageable copies drain
    assert s["mem_cmds"] >= 2 + 4 + 4 and s["mem_drained"] >= 5


def test_without_auto_xqueue_everything_passes_through(plain_output):
    out, err = run("shim_app", [MODULE], {"XSCHED_SHIM_STATS": "1", "XLOG_LEVEL": "WARN"})
    assert out == plain_output
    s = stats_of(err)
    assert s["kernel_cmds"] == 0 and s["mem_cmds"] == 0 and s["event_cmds"] == 0
    assert s["kernel_direct"] > 1000


def test_launch_cost_through_the_shim():
    """us per launch of a tiny kernel, with and without the shim (printed for the record)."""
    def bench(binary, env):
        out, _ = run(binary, ["--bench", "20000"], env)
        m = re.search(r"submit_us_per_launch=([\d.]+) total_us_per_launch=([\d.]+)", out)
        assert m, out
        return float(m.group(1)), float(m.group(2))
    plain = bench("shim_app_plain", {})
    through = bench("shim_app", shim_env(1))
    print(f"launch cost: plain submit {plain[0]:.2f} us, total {plain[1]:.2f} us per launch; "
          f"through the shim submit {through[0]:.2f} us, total {through[1]:.2f} us", file=sys.stderr, flush=True)
    assert through[1] < 60.0  # a regression guard, not a claim; typical values are far below
