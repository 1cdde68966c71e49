"""The headline workload on CPU cores, through the public C API only (oracle/host_bench.cpp),
over two host loops: the reference's own XQueue core + local scheduler + HPF policy
(where that build is present) and the shipped core. Both must leave bit-identical foreground
output: k in-place AXPYs of the seeded arrays, checked against the kernel oracle."""
import ctypes
import os
from ctypes import POINTER, byref, c_double, c_int, c_int64, c_uint64

import numpy as np
import pytest

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBS = {
    "reference": (os.path.join(ROOT, "oracle", "_ref", "libxqueue_ref.so"), "hostbench_run_fg_bg_axpy"),
    "shipped": (os.path.join(ROOT, "oracle", "libhostbench.so"), "hostbench_run_fg_bg_axpy"),
}
FG_N, BG_N, SAMPLES = 1 << 12, 1 << 16, 20


def expected_checksum():
    x = oracle.fill_uniform(0, 0, 0, FG_N)
    y = oracle.fill_uniform(0, 1, 0, FG_N)
    y = oracle.axpy(0.5, x, y, times=2 * SAMPLES)  # alone phase + contended phase
    return int(y[::97].view(np.uint32).astype(np.uint64).sum())


@pytest.mark.parametrize("which", ["reference", "shipped"])
def test_host_loops_agree_bit_for_bit(which):
    path, sym = LIBS[which]
    if not os.path.exists(path):
        if which == "reference":
            pytest.skip("reference build not present")
        pytest.fail(f"{path} missing: run __graft_entry__.build()")
    os.environ.setdefault("XLOG_LEVEL", "ERRO")
    fn = getattr(ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL), sym)
    fn.restype = c_int
    fn.argtypes = [c_uint64, c_uint64, c_int64, c_int, c_int, c_int, POINTER(c_double), POINTER(c_double),
                   POINTER(c_uint64), POINTER(c_double), POINTER(c_uint64)]
    alone, cont = (c_double * SAMPLES)(), (c_double * SAMPLES)()
    cmds, secs, chk = c_uint64(), c_double(), c_uint64()
    assert fn(BG_N, FG_N, 1000, SAMPLES, 8, 4, alone, cont, byref(cmds), byref(secs), byref(chk)) == 0
    assert all(v > 0 for v in list(alone) + list(cont))
    assert cmds.value > 0, "background made no progress under contention"
    assert chk.value == expected_checksum()
