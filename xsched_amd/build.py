"""Build driver for the native libraries.

    python -m xsched_amd.build [--only host|hip|oracle|all] [--debug-log]

Produces, under xsched_amd/lib/:
    libpreempt.so   XQueue core, scheduler, policies, C API           (g++)
    libhalhost.so   CPU hardware-queue adapter                         (g++)
    libhalhip.so    MI355X HIP adapter: Level-1/Level-2 queue, guarded
                    kernels, benchmark harness                         (hipcc, gfx950)
    libshimhip.so   HIP interception shim: stream work of an unmodified
                    HIP program becomes XQueue commands                (g++)
    shim_app, shim_app_plain, shim_app_packed
                    the shim's test program with the shim, without it, and
                    with compressed device code                        (hipcc)
    xserver         scheduler daemon                                   (g++)
    traffic_probe   counter-run driver for the AXPY kernel             (hipcc)
and, under oracle/, the checker libraries (see oracle/Makefile).

Everything is compiled for gfx950 only; hipcc cross-compiles without a GPU.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xsched_amd", "csrc")
LIB = os.path.join(ROOT, "xsched_amd", "lib")
OBJ = os.path.join(ROOT, "build", "obj")
INC = os.path.join(ROOT, "include")

CXXFLAGS = ["-std=c++20", "-O2", "-g", "-fPIC", "-Wall", "-Wextra", "-pthread",
            "-I", INC]
# Packed-FP32 instruction selection is switched off for all device code.
HIPFLAGS = ["--offload-arch=gfx950", "-std=c++20", "-O3", "-fPIC", "-pthread", "-I", INC,
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Wno-unused-command-line-argument"]

PREEMPT_SRCS = [
    "protocol/log.cpp", "protocol/names.cpp",
    "sched/protocol.cpp", "sched/policy.cpp", "sched/policy_extra.cpp", "sched/local.cpp", "sched/global.cpp",
    "sched/channel.cpp",
    "preempt/xcommand.cpp", "preempt/ring_queue.cpp", "preempt/xqueue.cpp", "preempt/agent.cpp",
]
HOST_SRCS = ["host/host_queue.cpp", "host/host_bench.cpp"]
SERVER_SRCS = ["service/xserver.cpp", "service/http.cpp"]
SHIM_SRCS = ["shim/code_object.cpp", "shim/hip_shim.cpp"]
HIP_SRCS = ["hip/hip_queue.hip", "hip/hip_command.hip", "hip/kernels_axpy.hip",
            "hip/kernels_gemm.hip", "hip/kernels_hist.hip", "bench/harness.hip"]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError("build step failed: " + cmd[0] + " " + cmd[-1])
    # hipcc's host pass does not know the packed-fp32 feature name; that warning is noise.
    noise = ("is not a recognized feature for this target", "warning generated", "warnings generated")
    for line in (proc.stdout + proc.stderr).splitlines():
        if line.strip() and not any(n in line for n in noise):
            sys.stderr.write(line + "\n")


def _compile_all(compiler, flags, srcs, jobs):
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    cmds = []
    for rel in srcs:
        src = os.path.join(CSRC, rel)
        if not os.path.exists(src):
            continue
        obj = os.path.join(OBJ, rel.replace("/", "_") + ".o")
        objs.append(obj)
        cmds.append([compiler] + flags + ["-c", src, "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, cmds))
    return objs


def build_host(extra, jobs):
    os.makedirs(LIB, exist_ok=True)
    flags = CXXFLAGS + extra
    objs = _compile_all("g++", flags, PREEMPT_SRCS, jobs)
    _run(["g++", "-shared", "-o", os.path.join(LIB, "libpreempt.so")] + objs + ["-pthread"])
    rpath = ["-L", LIB, "-Wl,-rpath,$ORIGIN"]
    objs = _compile_all("g++", flags, HOST_SRCS, jobs)
    _run(["g++", "-shared", "-o", os.path.join(LIB, "libhalhost.so")] + objs + rpath
         + ["-lpreempt", "-pthread"])
    objs = _compile_all("g++", flags, SERVER_SRCS, jobs)
    if objs:
        _run(["g++", "-o", os.path.join(LIB, "xserver")] + objs
             + ["-L", LIB, "-Wl,-rpath,$ORIGIN", "-lpreempt", "-pthread"])


def build_hip(extra, jobs):
    os.makedirs(LIB, exist_ok=True)
    objs = _compile_all("hipcc", HIPFLAGS + extra, HIP_SRCS, jobs)
    if not objs:
        return
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-o", os.path.join(LIB, "libhalhip.so")]
         + objs + ["-L", LIB, "-Wl,-rpath,$ORIGIN", "-lpreempt", "-pthread"])
    # The shim is host code against the HIP headers. libamdhip64 is named after the adapter so
    # that a program linked against the shim finds the runtime's entry points behind the shim's.
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    shim_flags = CXXFLAGS + extra + ["-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include")]
    shim_objs = _compile_all("g++", shim_flags, SHIM_SRCS, jobs)
    _run(["g++", "-shared", "-o", os.path.join(LIB, "libshimhip.so")] + shim_objs
         + ["-L", LIB, "-Wl,-rpath,$ORIGIN", "-lhalhip", "-lpreempt",
            "-L", os.path.join(rocm, "lib"), "-Wl,--no-as-needed", "-lamdhip64", "-Wl,--as-needed", "-ldl", "-pthread"])
    app = os.path.join(ROOT, "tests", "shim_app.hip")
    if os.path.exists(app):
        common = ["hipcc"] + HIPFLAGS + [app, "-pthread"]
        _run(common + ["-o", os.path.join(LIB, "shim_app_plain")])
        _run(common + ["-o", os.path.join(LIB, "shim_app"), "-L", LIB, "-Wl,-rpath,$ORIGIN",
                       "-Wl,--no-as-needed", "-lshimhip"])
        # the same program with its device code compressed, as large applications ship it
        _run(common + ["--offload-compress", "-o", os.path.join(LIB, "shim_app_packed"), "-L", LIB,
                       "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed", "-lshimhip"])
    user = os.path.join(ROOT, "tests", "user_guarded_kernel.hip")
    if os.path.exists(user):
        _run(["hipcc"] + HIPFLAGS + extra + ["-shared", user, "-o", os.path.join(LIB, "libuserguarded.so")])
    mod = os.path.join(ROOT, "tests", "shim_module.hip")
    if os.path.exists(mod):
        _run(["hipcc", "--offload-arch=gfx950", "-O3", "--genco", mod, "-o", os.path.join(LIB, "shim_module.co")])
    probe = os.path.join(CSRC, "bench", "traffic_probe.hip")
    if os.path.exists(probe):
        _run(["hipcc"] + HIPFLAGS + extra + [probe, "-o", os.path.join(LIB, "traffic_probe"),
             "-L", LIB, "-Wl,-rpath,$ORIGIN", "-lhalhip", "-lpreempt", "-pthread"])


def build_oracle():
    mk = os.path.join(ROOT, "oracle", "Makefile")
    if os.path.exists(mk):
        _run(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "-j8", "all"])


def build(only="all", debug_log=False, jobs=8):
    extra = ["-DXSCHED_DEBUG_LOG"] if debug_log else []
    if only in ("all", "host"):
        build_host(extra, jobs)
    if only in ("all", "hip"):
        build_hip(extra, jobs)
    if only in ("all", "oracle"):
        build_oracle()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", default="all", choices=["all", "host", "hip", "oracle"])
    ap.add_argument("--debug-log", action="store_true")
    ap.add_argument("-j", type=int, default=8)
    a = ap.parse_args()
    build(a.only, a.debug_log, a.j)
    print("built into", LIB)
