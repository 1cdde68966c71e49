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
CHECKS = 20  # lines the program prints, "done" and the error codes included


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
        assert line.endswith(" ok") or line.startswith("    error codes"), line
    codes = [line for line in lines if line.startswith("    error codes")][0].split()[2:]
    assert all(int(c) != 0 for c in codes), "the runtime accepted an invalid launch"
    return out


@pytest.mark.parametrize("level,threshold,batch", [(1, 16, 8), (1, 2, 1), (2, 16, 8)])
def test_same_results_through_xqueues(plain_output, level, threshold, batch):
    out, err = run("shim_app", [MODULE], shim_env(level, XSCHED_AUTO_XQUEUE_THRESHOLD=str(threshold),
                                                  XSCHED_AUTO_XQUEUE_BATCH_SIZE=str(batch)))
    assert out == plain_output
    s = stats_of(err)
    # 3 saxpy + 2 argument shapes + 301 counter kernels + 2 spins + 4 adds on streams (checks 4-6)
    # + 2 * 400 from the threads + 3 module launches; the one null-stream launch goes straight through
    # + 2 around the captured graph (the three captured launches are recorded by the runtime)
    # + 3 ordinary launches among the ordered-only calls (the cooperative and the ext launch drain)
    assert s["kernel_cmds"] == 3 + 2 + 301 + (1 + 2) + (1 + 1) + (1 + 1 + 1) + 800 + 2 + 40 + 3 + 50 + 3
    assert s["guarded_cmds"] == 50   # the launches of the kernel that has the guard compiled in
    assert s["kernel_drained"] == 2 + 2 + 3 and s["kernel_direct"] == 1 + 3   # refused launches; cooperative and ext launch; 3 ext launches before a sync
    assert s["known_kernels"] >= 7 + 2
    assert s["event_cmds"] == 3 and s["event_waits"] == 1
    # pinned and device-to-device copies and every fill are commands; pageable copies drain
    assert s["mem_cmds"] >= 2 + 4 + 4 and s["mem_drained"] >= 5


def test_program_with_compressed_device_code(plain_output):
    """Large applications ship their code objects compressed; the launches must still become
    commands (their argument layouts are read after unpacking), not drain-and-launch."""
    out, err = run("shim_app_packed", [MODULE], shim_env(2))
    assert out == plain_output
    s = stats_of(err)
    assert s["kernel_cmds"] == 1212 and s["kernel_drained"] == 7 and s["guarded_cmds"] == 50


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


def test_unmodified_binary_under_ld_preload(plain_output):
    """The way a user runs a program that was not linked against the shim."""
    shim = os.path.join(LIB, "libshimhip.so")
    preload = " ".join(x for x in (os.environ.get("LD_PRELOAD", ""), shim) if x)
    out, err = run("shim_app_plain", [MODULE], shim_env(1, LD_PRELOAD=preload))
    assert out == plain_output
    s = stats_of(err)
    assert s["kernel_cmds"] > 1000 and s["kernel_drained"] == 7


def _percentiles(out):
    m = re.search(r"probe n=(\d+) p50_us=([\d.]+) p99_us=([\d.]+) max_us=([\d.]+)", out)
    assert m, out
    return float(m.group(2)), float(m.group(3))


def test_two_unmodified_processes_under_the_daemon():
    """Two processes that know nothing of XSched, one filling the device with back-to-back
    kernels (priority 0), one launching a short kernel every 2 ms (priority 1), both through the
    shim and the scheduler daemon with HPF (reference examples/Linux/1_transparent_sched). The
    low-priority process's queue must get suspended while the other has work. Twice: with an
    ordinary load kernel, which a suspension can only keep from being launched again, and with
    one that has the guard compiled in (a zeroed XGuardArgs as its last argument in the
    program's own launches), which a deactivation makes leave the device and the reactivation
    replays; every work-group of it must still count itself exactly once per launch. The
    latencies of the short kernel are printed for the record."""
    import tempfile
    import time
    xserver = os.path.join(LIB, "xserver")
    sock_dir = tempfile.mkdtemp(prefix="xsched-shim-")
    base = {k: v for k, v in os.environ.items() if not k.startswith("XSCHED_")}
    probe_args = ["--probe", "300", "2000"]

    def start(binary, args, extra):
        print(f"starting {binary} {args} with {extra}", flush=True)
        return subprocess.Popen([os.path.join(LIB, binary)] + args, env=dict(base, **extra),
                                stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)

    def next_to(load_binary, load_args, load_env, probe_binary, probe_env):
        """Runs the probe while the load runs; returns (probe out, probe err, load out, load err)."""
        load = start(load_binary, load_args, load_env)
        assert load.stdout.readline().strip() == "ready"
        probe = start(probe_binary, probe_args, probe_env)
        probe_out, probe_err = probe.communicate(timeout=60)
        load_out, load_err = load.communicate(timeout=60)
        assert probe.returncode == 0 and load.returncode == 0, (probe_err[-1000:], load_out[-500:], load_err[-1000:])
        return probe_out, probe_err, load_out, load_err

    alone, _ = run("shim_app_plain", probe_args, {})
    # hardware scheduling only
    native = {kind: next_to("shim_app_plain", [flag, "1.6"], {}, "shim_app_plain", {})
              for kind, flag in (("plain", "--load"), ("guarded", "--load-guarded"))}

    server = subprocess.Popen([xserver, "HPF"], env=dict(base, XSCHED_SOCKET_DIR=sock_dir, XLOG_LEVEL="WARN"))
    try:
        deadline = time.time() + 5
        while not os.path.exists(os.path.join(sock_dir, "xsched-1.sock")) and time.time() < deadline:
            time.sleep(0.01)
        assert os.path.exists(os.path.join(sock_dir, "xsched-1.sock")), "xserver did not come up"
        common = {"XSCHED_SOCKET_DIR": sock_dir, "XSCHED_SCHEDULER": "GLB", "XSCHED_AUTO_XQUEUE": "ON",
                  "XSCHED_AUTO_XQUEUE_LEVEL": "2", "XSCHED_SHIM_STATS": "1", "XLOG_LEVEL": "WARN"}
        low = dict(common, XSCHED_AUTO_XQUEUE_PRIORITY="0", XSCHED_AUTO_XQUEUE_THRESHOLD="2",
                   XSCHED_AUTO_XQUEUE_BATCH_SIZE="1")
        high = dict(common, XSCHED_AUTO_XQUEUE_PRIORITY="1")
        under = {kind: next_to("shim_app", [flag, "1.6"], low, "shim_app", high)
                 for kind, flag in (("plain", "--load"), ("guarded", "--load-guarded"))}
    finally:
        server.terminate()
        try:
            server.wait(timeout=5)
        except subprocess.TimeoutExpired:
            server.kill()

    a = _percentiles(alone)
    print(f"short kernel alone: p50/p99 {a[0]:.0f}/{a[1]:.0f} us", file=sys.stderr, flush=True)
    for kind in ("plain", "guarded"):
        n, x = _percentiles(native[kind][0]), _percentiles(under[kind][0])
        ls, ps = stats_of(under[kind][3]), stats_of(under[kind][1])
        print(f"{kind} load: short kernel p50/p99 us next to it without XSched {n[0]:.0f}/{n[1]:.0f}, under XSched "
              f"{x[0]:.0f}/{x[1]:.0f}; load without XSched: {native[kind][2].strip().splitlines()[-1]} | under XSched: "
              f"{under[kind][2].strip().splitlines()[-1]}; its queue: deactivations {ls['deactivations']}, "
              f"replayed launches {ls['replays']}, guarded commands {ls['guarded_cmds']}", file=sys.stderr, flush=True)
        assert ps["deactivations"] == 0, "the high-priority process was suspended"
        assert ls["deactivations"] > 50 and ls["reactivations"] > 50, "the daemon never suspended the low-priority process"
        assert ps["kernel_cmds"] >= 300 and ls["kernel_cmds"] >= 32
    gs = stats_of(under["guarded"][3])
    assert gs["guarded_cmds"] == gs["kernel_cmds"] and gs["replays"] > 0, "no guarded launch was flushed and replayed"
    assert "work_groups_not_exactly_once=0" in under["guarded"][2] and "work_groups_not_exactly_once=0" in native["guarded"][2]
    # what the guard is for: the short kernel no longer waits for the load's 5 ms kernel to finish
    assert _percentiles(under["guarded"][0])[1] < _percentiles(native["guarded"][0])[0] / 3


@pytest.mark.parametrize("level", [1, 2])
def test_program_that_releases_nothing_exits_cleanly(level):
    """Streams, events and memory are never released and one stream still has work when main()
    returns: the process must end with the program's own exit code."""
    out, _ = run("shim_app_plain", ["--leak"], {})
    assert "leak counter=100" in out
    out, err = run("shim_app", ["--leak"], shim_env(level))
    assert "leak counter=100" in out
    assert stats_of(err)["kernel_cmds"] == 102


def test_pytorch_program_under_the_preloaded_shim():
    """A PyTorch-ROCm training loop on side streams (tests/shim_torch_workload.py; compressed
    code objects, rocBLAS kernels launched from loaded modules, the caching allocator's events)
    prints bit-identical losses and weights with the shim preloaded, and its launches were
    XQueue commands."""
    script = os.path.join(ROOT, "tests", "shim_torch_workload.py")

    def torch_run(extra):
        env = {k: v for k, v in os.environ.items() if not k.startswith("XSCHED_")}
        env.update(extra)
        print(f"running {script} with {extra}", flush=True)
        proc = subprocess.run([sys.executable, script], env=env, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, (proc.stdout[-2000:], proc.stderr[-3000:])
        return proc.stdout, proc.stderr

    plain, _ = torch_run({})
    assert plain.strip().endswith("done")
    shim = os.path.join(LIB, "libshimhip.so")
    preload = " ".join(x for x in (os.environ.get("LD_PRELOAD", ""), shim) if x)
    for level in (1, 2):
        out, err = torch_run(shim_env(level, LD_PRELOAD=preload))
        assert out == plain
        s = stats_of(err)
        print(f"level {level}: {s}", file=sys.stderr, flush=True)
        assert s["kernel_cmds"] > 500 and s["kernel_drained"] == 0
        assert s["event_waits"] >= 1 and s["mem_cmds"] > 0
