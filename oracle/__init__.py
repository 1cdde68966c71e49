"""ORACLE - test infrastructure only (see oracle/kernels.c).

ctypes access to the plain-C restatement of the path's arithmetic. Imported by
tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py; never by
the xsched_amd package.
"""
import ctypes
import os
from ctypes import POINTER, c_double, c_float, c_int, c_size_t, c_uint16, c_uint32, c_uint64, c_void_p

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_DIR, "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle` (or __graft_entry__.build())")
        L = ctypes.CDLL(path)
        L.oracle_vecadd.argtypes = [c_void_p, c_void_p, c_void_p, c_size_t]
        L.oracle_axpy.argtypes = [c_float, c_void_p, c_void_p, c_size_t]
        L.oracle_gemm_bf16.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]
        L.oracle_histogram.argtypes = [c_void_p, c_size_t, c_void_p, c_uint32]
        L.oracle_percentile.argtypes = [c_void_p, c_size_t, c_double]
        L.oracle_percentile.restype = c_double
        L.oracle_f32_to_bf16.argtypes = [c_float]
        L.oracle_f32_to_bf16.restype = c_uint16
        L.oracle_stream_key.argtypes = [c_uint64, c_uint64]
        L.oracle_stream_key.restype = c_uint64
        L.oracle_bits.argtypes = [c_uint64, c_uint64]
        L.oracle_bits.restype = c_uint64
        L.oracle_fill_uniform.argtypes = [c_void_p, c_uint64, c_uint64, c_uint64]
        L.oracle_fill_normal_bf16.argtypes = [c_void_p, c_uint64, c_uint64, c_uint64]
        L.oracle_zipf_table.argtypes = [c_void_p, c_uint32, c_double]
        L.oracle_fill_zipf.argtypes = [c_void_p, c_uint64, c_uint64, c_uint64, c_void_p, c_uint32]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(c_void_p)


def vecadd(a, b):
    a = np.ascontiguousarray(a, np.float32); b = np.ascontiguousarray(b, np.float32)
    c = np.empty_like(a)
    lib().oracle_vecadd(_p(a), _p(b), _p(c), a.size)
    return c


def axpy(alpha, x, y, times=1):
    """y <- fma(alpha, x, y), applied `times` times; returns the new y."""
    x = np.ascontiguousarray(x, np.float32)
    y = np.array(y, np.float32, copy=True)
    for _ in range(times):
        lib().oracle_axpy(float(alpha), _p(x), _p(y), x.size)
    return y


def gemm_bf16(a_bits, b_bits, M, N, K, want_f32=False):
    """a_bits/b_bits: uint16 arrays holding bf16 bit patterns, row-major."""
    a_bits = np.ascontiguousarray(a_bits, np.uint16); b_bits = np.ascontiguousarray(b_bits, np.uint16)
    c = np.empty(M * N, np.uint16)
    cf = np.empty(M * N, np.float32) if want_f32 else None
    lib().oracle_gemm_bf16(_p(a_bits), _p(b_bits), _p(c), _p(cf) if want_f32 else None, M, N, K)
    return (c.reshape(M, N), cf.reshape(M, N)) if want_f32 else c.reshape(M, N)


def histogram(keys, n_bins, bins=None):
    keys = np.ascontiguousarray(keys, np.int32)
    out = np.zeros(n_bins, np.uint32) if bins is None else np.array(bins, np.uint32, copy=True)
    lib().oracle_histogram(_p(keys), keys.size, _p(out), n_bins)
    return out


def percentile(samples, p):
    d = np.array(samples, np.float64, copy=True)
    return lib().oracle_percentile(_p(d), d.size, float(p))


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def stream_key(seed, stream):
    return lib().oracle_stream_key(seed, stream)


def bits(key, i):
    """Raw 64 bits of the stream with key `key` at index i."""
    return lib().oracle_bits(key, i)


def fill_uniform(seed, stream, first, count):
    out = np.empty(count, np.float32)
    lib().oracle_fill_uniform(_p(out), first, count, stream_key(seed, stream))
    return out


def fill_normal_bf16(seed, stream, first, count):
    out = np.empty(count, np.uint16)
    lib().oracle_fill_normal_bf16(_p(out), first, count, stream_key(seed, stream))
    return out


def zipf_table(n_bins=65536, s=1.1):
    t = np.empty(n_bins, np.uint32)
    lib().oracle_zipf_table(_p(t), n_bins, s)
    return t


def fill_zipf(seed, stream, first, count, table=None, n_bins=65536):
    table = zipf_table(n_bins) if table is None else table
    out = np.empty(count, np.int32)
    lib().oracle_fill_zipf(_p(out), first, count, stream_key(seed, stream), _p(table), n_bins)
    return out
