"""The XQueue core, the local scheduler and the host adapter under ThreadSanitizer: their
sources are compiled with -fsanitize=thread together with tests/tsan_driver.cpp (no shared
library in between, so every access is instrumented) and driven from several threads through
the public C API. No data race may be reported and every guarded work-group must have taken
effect exactly once. CPU only."""
import os
import subprocess

import xsched_amd.build as b

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_core_scheduler_and_host_adapter_under_thread_sanitizer(tmp_path):
    exe = str(tmp_path / "tsan_driver")
    srcs = [os.path.join(b.CSRC, rel) for rel in b.PREEMPT_SRCS + b.HOST_SRCS]
    srcs.append(os.path.join(ROOT, "tests", "tsan_driver.cpp"))
    # the sanitizer runtime is linked statically: it then does not mind other preloaded libraries
    build = subprocess.run(["g++", "-std=c++20", "-O1", "-g", "-fsanitize=thread", "-static-libtsan", "-pthread",
                            "-I", b.INC] + srcs + ["-o", exe], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 exitcode=66 second_deadlock_stack=1", XLOG_LEVEL="ERRO")
    env.pop("LD_PRELOAD", None)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600, env=env)
    assert "ThreadSanitizer" not in run.stderr, run.stderr[-6000:]
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert run.stdout.strip().endswith("done"), run.stdout
