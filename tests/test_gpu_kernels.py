"""GPU parity: the guarded kernels, launched through the C ABI and an XQueue, against
the CPU oracle on the same seeded inputs. Integer and fp32-AXPY results must be
bit-exact; the bf16 GEMM is bit-exact where the arithmetic is exact (small-integer
inputs) and within a stated tolerance otherwise."""
import ctypes
from ctypes import byref, c_uint64, c_void_p

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


class Queue:
    """One stream + HwQueue + XQueue."""

    def __init__(self, xs, torch, level=1, threshold=8, batch=4):
        self.xs, self.torch = xs, torch
        self.stream = torch.cuda.Stream()
        self.hwq = xs.hip_queue_create(self.stream.cuda_stream)
        self.xq = xs.xqueue_create(self.hwq, level)
        xs.check(xs.preempt().XQueueSetLaunchConfig(self.xq, threshold, batch))

    def submit(self, cmd):
        self.xs.check(self.xs.preempt().XQueueSubmit(self.xq, cmd))

    def wait(self):
        self.xs.check(self.xs.preempt().XQueueWaitAll(self.xq))

    def close(self):
        p = self.xs.preempt()
        self.xs.check(p.XQueueDestroy(self.xq))
        self.xs.check(p.HwQueueDestroy(self.hwq))


def axpy_cmd(xs, alpha, x, y, n, guard):
    cmd = c_uint64()
    xs.check(xs.halhip().HipAxpyCommandCreate(byref(cmd), alpha, x.data_ptr(), y.data_ptr(), n, guard))
    return cmd.value


def gemm_cmd(xs, a, b, c, M, N, K, guard):
    cmd = c_uint64()
    xs.check(xs.halhip().HipGemmBf16CommandCreate(byref(cmd), a.data_ptr(), b.data_ptr(), c.data_ptr(),
                                                  M, N, K, guard))
    return cmd.value


def hist_cmd(xs, keys, n, bins, n_bins, guard):
    cmd = c_uint64()
    xs.check(xs.halhip().HipHistogramCommandCreate(byref(cmd), keys.data_ptr(), n, bins.data_ptr(),
                                                   n_bins, guard))
    return cmd.value


@pytest.mark.parametrize("n", [0, 1, 3, 5, 1023, 4096, 4097, (1 << 20) + 7, 1 << 22])
@pytest.mark.parametrize("level,guard", [(1, 0), (1, 2), (2, 1), (2, 3), (1, 3)])
def test_axpy_bit_exact(xs, gpu, n, level, guard):
    torch = gpu
    print(f"case axpy n={n} level={level} guard={guard}", flush=True)
    x_h = oracle.fill_uniform(0, 1, 0, max(n, 1))[:n]
    y_h = oracle.fill_uniform(0, 2, 0, max(n, 1))[:n]
    x = torch.from_numpy(x_h.copy()).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, level)
    times = 3
    for _ in range(times):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, guard))
    q.wait()
    torch.cuda.synchronize()
    want = oracle.axpy(0.5, x_h, y_h, times)
    got = y.cpu().numpy()
    q.close()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n", [1, 1024, 2048, 3 * 1024 + 1, 7 * 1024, 7 * 1024 * 513 + 2, (1 << 21) + 4099])
@pytest.mark.parametrize("grid,steps", [("waves", 2), ("waves", 3), ("waves", 7), ("chunk", 1), ("chunk", 2), ("chunk", 3)])
def test_axpy_guarded_grids_and_chunk_sizes(xs, gpu, monkeypatch, grid, steps, n):
    """Both grids of a guarded AXPY with chunks of several steps, at lengths around the
    chunk and step borders (a last chunk that is not full, 0..3 trailing scalars, fewer
    chunks than waves, more steps in a chunk than the waves keep in flight)."""
    torch = gpu
    monkeypatch.setenv("XSCHED_HIP_AXPY_GRID", grid)
    monkeypatch.setenv("XSCHED_HIP_AXPY_STEPS", str(steps))
    print(f"case axpy-grid n={n} grid={grid} steps={steps}", flush=True)
    x_h = oracle.fill_uniform(21, 1, 0, n)
    y_h = oracle.fill_uniform(21, 2, 0, n)
    x = torch.from_numpy(x_h.copy()).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, 2)
    for _ in range(2):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
    q.wait()
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    q.close()
    want = oracle.axpy(0.5, x_h, y_h, 2)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("steps,n", [(1, (1 << 23) + 7), (3, 8192 * 3072 + 1029), (2, 8192 * 2048)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_axpy_long_arrays(xs, gpu, monkeypatch, steps, n, level, guard):
    """From 8192 chunks on a plain launch runs on the long-lived waves as well (shorter arrays
    use one wave per chunk): lengths just past that border, with one and several steps per
    chunk, a ragged end and an exact fit."""
    torch = gpu
    monkeypatch.setenv("XSCHED_HIP_AXPY_STEPS", str(steps))
    print(f"case axpy-long n={n} steps={steps} level={level} guard={guard}", flush=True)
    x_h = oracle.fill_uniform(23, 1, 0, n)
    y_h = oracle.fill_uniform(23, 2, 0, n)
    x = torch.from_numpy(x_h).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, level)
    for _ in range(2):
        q.submit(axpy_cmd(xs, 0.5, x, y, n, guard))
    q.wait()
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    q.close()
    want = oracle.axpy(0.5, x_h, y_h, 2)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_axpy_at_the_full_size_of_the_headline_configuration(xs, gpu):
    """2^28 elements, where the grid sits exactly on the progress map's limit of 2^18
    work-groups, and 2^28 + 5 (the chunk doubles, the end is ragged): a plain launch at level 1,
    then guarded launches at level 2 with a suspend / resume while they are in flight; every
    element against the oracle."""
    torch = gpu
    p = xs.preempt()
    n_big = (1 << 28) + 5
    x_h = oracle.fill_uniform(0, 4, 0, n_big)
    y_h = oracle.fill_uniform(0, 5, 0, n_big)
    x = torch.from_numpy(x_h).cuda()

    n = 1 << 28
    print(f"case axpy-full n={n} plain level 1", flush=True)
    y = torch.from_numpy(y_h[:n].copy()).cuda()
    q = Queue(xs, torch, 1, threshold=2, batch=1)
    q.submit(axpy_cmd(xs, 0.5, x, y, n, 0))
    q.wait()
    want = oracle.axpy(0.5, x_h[:n], y_h[:n], 1)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    q.close()

    print(f"case axpy-full n={n} guarded level 2, suspended in flight", flush=True)
    q = Queue(xs, torch, 2, threshold=2, batch=1)
    q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
    q.submit(axpy_cmd(xs, 0.5, x, y, n, 1))
    xs.check(p.XQueueSuspend(q.xq, xs.kQueueSuspendFlagSyncHwQueue))
    xs.check(p.XQueueResume(q.xq, xs.kQueueResumeFlagNone))
    q.wait()
    want = oracle.axpy(0.5, x_h[:n], want, 2)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    stats = (ctypes.c_uint64 * 8)()
    xs.check(xs.halhip().HipQueueGetStats(q.hwq, stats))
    assert stats[2] == 1 and stats[3] == 1   # one deactivation, one reactivation
    q.close()
    del y, want

    print(f"case axpy-full n={n_big} guarded level 2", flush=True)
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, 2, threshold=2, batch=1)
    q.submit(axpy_cmd(xs, 0.5, x, y, n_big, 1))
    q.wait()
    want = oracle.axpy(0.5, x_h, y_h, 1)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    q.close()


def test_axpy_general_alpha_and_unaligned(xs, gpu):
    """alpha whose product is inexact (one rounding: fma) and a pointer that is only
    4-byte aligned (scalar fallback kernel)."""
    torch = gpu
    n = 100003
    x_h = oracle.fill_uniform(3, 1, 0, n + 1)
    y_h = oracle.fill_uniform(3, 2, 0, n + 1)
    x = torch.from_numpy(x_h.copy()).cuda()
    y = torch.from_numpy(y_h.copy()).cuda()
    q = Queue(xs, torch, 2)
    alpha = 0.3337
    q.submit(axpy_cmd(xs, alpha, x, y, n, 1))          # aligned
    q.wait()
    want = oracle.axpy(np.float32(alpha), x_h[:n], y_h[:n])
    assert np.array_equal(y.cpu().numpy()[:n].view(np.uint32), want.view(np.uint32))
    xo, yo = x[1:], y[1:]                               # misaligned by 4 bytes
    y_before = y.cpu().numpy().copy()
    q.submit(axpy_cmd(xs, alpha, xo, yo, n, 1))
    q.wait()
    want2 = oracle.axpy(np.float32(alpha), x_h[1:n + 1], y_before[1:n + 1])
    got = y.cpu().numpy()
    q.close()
    assert np.array_equal(got[1:n + 1].view(np.uint32), want2.view(np.uint32))
    assert got[0] == y_before[0]


@pytest.fixture(params=["sweep", "merge"])
def hist_layout(request, monkeypatch):
    """The histogram merges its per-group counts in one of two ways, chosen by the number
    of keys when the command is created: an atomic sweep by the counting kernel itself
    (small inputs) or packed partial histograms summed by a second kernel (2^25 keys and
    more). "merge" forces the second one at every size."""
    if request.param == "merge":
        monkeypatch.setenv("XSCHED_HIP_HIST_MERGE_MIN_KEYS", "1")
    else:
        monkeypatch.setenv("XSCHED_HIP_HIST_MERGE_MIN_KEYS", str(1 << 40))
    return request.param


@pytest.mark.parametrize("n,n_bins", [(0, 65536), (1, 65536), (1000, 65536), (65536 + 13, 65536),
                                      (1 << 20, 65536), (300000, 1000), (5000, 7), (70000, 32769),
                                      (4096 * 300 + 1, 65535)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_histogram_bit_exact(xs, gpu, hist_layout, n, n_bins, level, guard):
    torch = gpu
    print(f"case hist {hist_layout} n={n} bins={n_bins} level={level} guard={guard}", flush=True)
    table = oracle.zipf_table(n_bins)
    keys_h = oracle.fill_zipf(0, 1, 0, max(n, 1), table, n_bins)[:n]
    keys = torch.from_numpy(np.ascontiguousarray(keys_h) if n else np.zeros(1, np.int32)).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, level)
    q.submit(hist_cmd(xs, keys, n, bins, n_bins, guard))
    q.submit(hist_cmd(xs, keys, n, bins, n_bins, guard))   # accumulates: bins are not cleared
    q.wait()
    got = bins.cpu().numpy().view(np.uint32)
    q.close()
    want = oracle.histogram(keys_h, n_bins)
    want = oracle.histogram(keys_h, n_bins, want)
    assert int(got.sum()) == 2 * n
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n_bins,offset", [(65536, 0), (65536, 1), (1001, 0), (40000, 1)])
def test_histogram_counters_wrap_independently(xs, gpu, hist_layout, n_bins, offset):
    """Bins that start just below 2^32 wrap on their own, as uint32 counters do in the
    oracle: the write-out adds two neighbouring counters with one 64-bit atomic and must
    take back a carry that leaks from the lower into the upper one. Also with a bins array
    that is only 4-byte aligned (offset 1), where the write-out uses 32-bit atomics."""
    torch = gpu
    n = (1 << 20) + 13
    print(f"case hist-wrap {hist_layout} bins={n_bins} offset={offset}", flush=True)
    table = oracle.zipf_table(n_bins)
    keys_h = oracle.fill_zipf(3, 1, 0, n, table, n_bins)
    keys = torch.from_numpy(keys_h).cuda()
    rnd = np.random.default_rng(5)
    start = (0xFFFFFFFF - rnd.integers(0, 3, n_bins)).astype(np.uint32)   # 0..2 below wrapping
    start[rnd.random(n_bins) < 0.3] = 0
    store = torch.zeros(n_bins + 2, dtype=torch.int32, device="cuda")
    bins = store[offset:offset + n_bins]
    bins.copy_(torch.from_numpy(start.view(np.int32)))
    q = Queue(xs, torch, 2)
    q.submit(hist_cmd(xs, keys, n, bins, n_bins, 1))
    q.wait()
    got = bins.cpu().numpy().view(np.uint32)
    guard_words = store.cpu().numpy()
    q.close()
    want = oracle.histogram(keys_h, n_bins, start)
    assert np.array_equal(got, want)
    assert guard_words[offset + n_bins:].tolist() == [0] * (2 - offset), "wrote beyond the bins array"
    if offset:
        assert guard_words[0] == 0


@pytest.mark.parametrize("lo,hi", [(32768, 65536), (0, 65536), (100, 101), (40000, 40003)])
def test_histogram_any_distribution(xs, gpu, hist_layout, lo, hi):
    """Distributions the kernel is not tuned for: every key in the upper half of the key
    space (the on-chip list of such keys overflows and the work-group re-reads its chunk),
    uniform keys, one single bin, three neighbouring bins."""
    torch = gpu
    n = (1 << 22) + 5
    print(f"case hist-dist {hist_layout} [{lo},{hi})", flush=True)
    keys_h = np.random.default_rng(lo).integers(lo, hi, n).astype(np.int32)
    keys = torch.from_numpy(keys_h).cuda()
    bins = torch.zeros(65536, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, 2)
    q.submit(hist_cmd(xs, keys, n, bins, 65536, 1))
    q.wait()
    got = bins.cpu().numpy().view(np.uint32)
    q.close()
    assert np.array_equal(got, oracle.histogram(keys_h, 65536))


@pytest.mark.parametrize("case", ["zipf", "one low bin", "one high bin", "both halves of a word", "ballot bin",
                                  "half heavy"])
def test_histogram_merge_layout_at_its_own_size(xs, gpu, case):
    """2^25 keys take the two-kernel layout by themselves, 131072 keys per counting group.
    Its 16-bit halves overflow when one bin takes 65536 keys of a group: the group must
    notice and recount. "both halves of a word": bins 7232 and 40000 share a packed word."""
    torch = gpu
    n, n_bins = 1 << 25, 65536
    print(f"case hist-merge {case}", flush=True)
    rng = np.random.default_rng(11)
    if case == "zipf":
        keys_h = oracle.fill_zipf(5, 1, 0, n, oracle.zipf_table(n_bins), n_bins)
    elif case == "one low bin":
        keys_h = np.full(n, 100, np.int32)
    elif case == "one high bin":
        keys_h = np.full(n, 40000, np.int32)
    elif case == "both halves of a word":
        keys_h = np.where(rng.random(n) < 0.5, 7232, 40000).astype(np.int32)
    elif case == "ballot bin":
        keys_h = np.where(rng.random(n) < 0.9, 0, rng.integers(0, n_bins, n)).astype(np.int32)
    else:
        # groups in the first half of the array overflow, the others do not
        keys_h = rng.integers(0, n_bins, n).astype(np.int32)
        keys_h[:n // 2][rng.random(n // 2) < 0.7] = 12345
    keys = torch.from_numpy(keys_h).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    q = Queue(xs, torch, 2)
    q.submit(hist_cmd(xs, keys, n, bins, n_bins, 1))
    q.submit(hist_cmd(xs, keys, n, bins, n_bins, 0))
    q.wait()
    got = bins.cpu().numpy().view(np.uint32)
    q.close()
    want = oracle.histogram(keys_h, n_bins)
    assert np.array_equal(got.astype(np.uint64), want.astype(np.uint64) * 2)


def _gemm_case(xs, torch, a_bits, b_bits, M, N, K, level, guard):
    a = torch.from_numpy(a_bits.view(np.int16).reshape(M, K)).cuda()
    b = torch.from_numpy(b_bits.view(np.int16).reshape(K, N)).cuda()
    c = torch.zeros(M, N, dtype=torch.int16, device="cuda")
    q = Queue(xs, torch, level)
    q.submit(gemm_cmd(xs, a, b, c, M, N, K, guard))
    q.wait()
    got = c.cpu().numpy().view(np.uint16)
    q.close()
    return got


@pytest.fixture(params=[128, 256])
def gemm_tile(request, monkeypatch):
    """The GEMM works on 256x256 tiles of C, or on 128x128 tiles when the large ones would not
    fill the device (every shape of these tests) or do not fit the shape. The variable forces
    one of them where the shape allows both."""
    monkeypatch.setenv("XSCHED_HIP_GEMM_TILE", str(request.param))
    return request.param


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (256, 512, 128), (512, 256, 192)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_gemm_exact_on_small_integers(xs, gpu, gemm_tile, M, N, K, level, guard):
    """Inputs are integers in [-4, 4]: every product and partial sum is an integer below
    2^24, so fp32 accumulation is exact in any order and the bf16 result is determined;
    any indexing or layout mistake changes it."""
    print(f"case gemm-int M={M} N={N} K={K} level={level} guard={guard}", flush=True)
    rng = np.random.default_rng(7)
    a_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b_i = rng.integers(-4, 5, (K, N)).astype(np.float32)
    a_bits, b_bits = oracle.f32_to_bf16_bits(a_i), oracle.f32_to_bf16_bits(b_i)
    got = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, level, guard)
    want_int = a_i.astype(np.int64) @ b_i.astype(np.int64)
    want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K)
    assert np.array_equal(want, oracle.f32_to_bf16_bits(want_int.astype(np.float32)).reshape(M, N))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (384, 128, 128), (128, 640, 192), (896, 384, 64)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_gemm_shapes_that_only_small_tiles_fit(xs, gpu, M, N, K, level, guard):
    """M or N a multiple of 128 but not of 256; integers as above, so the result is determined."""
    print(f"case gemm-int-small M={M} N={N} K={K} level={level} guard={guard}", flush=True)
    rng = np.random.default_rng(8)
    a_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b_i = rng.integers(-4, 5, (K, N)).astype(np.float32)
    a_bits, b_bits = oracle.f32_to_bf16_bits(a_i), oracle.f32_to_bf16_bits(b_i)
    got = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, level, guard)
    want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (64, 64, 16), (65, 63, 17), (127, 129, 65), (130, 70, 33),
                                   (256, 128, 100), (200, 256, 64), (128, 128, 8), (1, 300, 129), (300, 1, 250)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_gemm_any_shape(xs, gpu, M, N, K, level, guard):
    """Shapes the fast kernels do not take (M or N no multiple of 128, K no multiple of 64) go
    to the any-shape kernel: integers as above, so the result is determined; the matrices lie
    in larger buffers whose other elements must come back untouched."""
    torch = gpu
    print(f"case gemm-any M={M} N={N} K={K} level={level} guard={guard}", flush=True)
    rng = np.random.default_rng(9)
    a_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b_i = rng.integers(-4, 5, (K, N)).astype(np.float32)
    a_bits, b_bits = oracle.f32_to_bf16_bits(a_i), oracle.f32_to_bf16_bits(b_i)
    want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K)
    pad = 3   # elements in front: the matrices start at odd multiples of two bytes
    a = torch.from_numpy(np.concatenate([np.full(pad, 0x7FC0, np.uint16), a_bits.ravel(), np.full(64, 0x7FC0, np.uint16)]).view(np.int16)).cuda()
    b = torch.from_numpy(np.concatenate([np.full(pad, 0x7FC0, np.uint16), b_bits.ravel(), np.full(64, 0x7FC0, np.uint16)]).view(np.int16)).cuda()
    c = torch.full((pad + M * N + 64,), 0x1234, dtype=torch.int16, device="cuda")
    cmd = c_uint64()
    xs.check(xs.halhip().HipGemmBf16CommandCreate(byref(cmd), a.data_ptr() + 2 * pad, b.data_ptr() + 2 * pad,
                                                  c.data_ptr() + 2 * pad, M, N, K, guard))
    q = Queue(xs, torch, level)
    q.submit(cmd.value)
    q.wait()
    got = c.cpu().numpy().view(np.uint16)
    q.close()
    assert np.array_equal(got[pad:pad + M * N].reshape(M, N), want.reshape(M, N))
    assert np.all(got[:pad] == 0x1234) and np.all(got[pad + M * N:] == 0x1234)


@pytest.mark.parametrize("M,N,K", [(129, 128, 64), (200, 256, 64), (1000, 384, 128), (2049, 256, 192), (127, 256, 64)])
@pytest.mark.parametrize("level,guard", [(1, 0), (2, 1)])
def test_gemm_ragged_rows_are_split_between_the_kernels(xs, gpu, M, N, K, level, guard):
    """N and K as the fast kernel wants them, M not (the usual ragged dimension): the rows up to
    the last multiple of 128 go to the fast kernel, the rest to the any-shape kernel, in one
    command (M below 128: all of it to the any-shape kernel). Integers, so the result is
    determined; the rows behind the matrix in C's buffer stay untouched."""
    torch = gpu
    print(f"case gemm-split M={M} N={N} K={K} level={level} guard={guard}", flush=True)
    rng = np.random.default_rng(10)
    a_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b_i = rng.integers(-4, 5, (K, N)).astype(np.float32)
    a_bits, b_bits = oracle.f32_to_bf16_bits(a_i), oracle.f32_to_bf16_bits(b_i)
    want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K).reshape(M, N)
    a = torch.from_numpy(a_bits.view(np.int16).reshape(M, K)).cuda()
    b = torch.from_numpy(b_bits.view(np.int16).reshape(K, N)).cuda()
    c = torch.full((M + 2, N), 0x1234, dtype=torch.int16, device="cuda")
    q = Queue(xs, torch, level)
    q.submit(gemm_cmd(xs, a, b, c, M, N, K, guard))
    q.wait()
    got = c.cpu().numpy().view(np.uint16)
    q.close()
    assert np.array_equal(got[:M], want)
    assert np.all(got[M:] == 0x1234)


def test_gemm_any_shape_kernel_sums_as_the_fast_kernels_do(xs, gpu, monkeypatch):
    """Seeded normal inputs on a shape every kernel takes: the any-shape kernel (forced)
    feeds the matrix cores the same slices of 16 along K in the same order, so the bits agree."""
    M, N, K = 256, 384, 512
    print(f"case gemm-any-vs-fast M={M} N={N} K={K}", flush=True)
    a_bits = oracle.fill_normal_bf16(19, 1, 0, M * K)
    b_bits = oracle.fill_normal_bf16(19, 2, 0, K * N)
    out = {}
    for tile in (64, 128):
        monkeypatch.setenv("XSCHED_HIP_GEMM_TILE", str(tile))
        out[tile] = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, 2, 1)
    assert np.array_equal(out[64], out[128])


def test_gemm_refuses_what_no_kernel_takes(xs, gpu):
    torch = gpu
    t = torch.zeros(64, dtype=torch.int16, device="cuda")
    cmd = c_uint64()
    h = xs.halhip()
    for M, N, K in ((0, 8, 8), (8, 0, 8), (8, 8, 0), (-1, 8, 8)):
        assert h.HipGemmBf16CommandCreate(byref(cmd), t.data_ptr(), t.data_ptr(), t.data_ptr(), M, N, K, 1) == xs.kXSchedErrorInvalidValue
    assert h.HipGemmBf16CommandCreate(byref(cmd), t.data_ptr() + 1, t.data_ptr(), t.data_ptr(), 4, 4, 4, 1) == xs.kXSchedErrorInvalidValue
    # more tiles than a progress map has bytes
    assert h.HipGemmBf16CommandCreate(byref(cmd), t.data_ptr(), t.data_ptr(), t.data_ptr(), 64 * 1024, 64 * 1024 + 1, 1, 1) == xs.kXSchedErrorInvalidValue


def test_gemm_seeded_random_shapes(xs, gpu, monkeypatch):
    """Ten seeded shapes (M, N multiples of 128 up to 1152, K multiples of 64 up to 448), each
    with the tile sizes its shape allows; integer inputs, so every result is determined."""
    rng = np.random.default_rng(2024)
    for case in range(10):
        M, N = (int(v) * 128 for v in rng.integers(1, 10, 2))
        K = int(rng.integers(1, 8)) * 64
        a_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
        b_i = rng.integers(-4, 5, (K, N)).astype(np.float32)
        a_bits, b_bits = oracle.f32_to_bf16_bits(a_i), oracle.f32_to_bf16_bits(b_i)
        want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K)
        tiles = (128, 256) if M % 256 == 0 and N % 256 == 0 else (128,)
        for tile in tiles:
            print(f"case gemm-random {case}: M={M} N={N} K={K} tile={tile}", flush=True)
            monkeypatch.setenv("XSCHED_HIP_GEMM_TILE", str(tile))
            got = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, 2, 1)
            assert np.array_equal(got, want), (M, N, K, tile)


def test_gemm_both_tile_sizes_give_the_same_bits(xs, gpu, monkeypatch):
    """Seeded normal inputs, where the order of the fp32 additions shows in the last bits:
    both tile sizes feed every element's products to the matrix cores in the same order."""
    M, N, K = 512, 768, 1024
    print(f"case gemm-tiles M={M} N={N} K={K}", flush=True)
    a_bits = oracle.fill_normal_bf16(17, 1, 0, M * K)
    b_bits = oracle.fill_normal_bf16(17, 2, 0, K * N)
    out = {}
    for tile in (128, 256):
        monkeypatch.setenv("XSCHED_HIP_GEMM_TILE", str(tile))
        out[tile] = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, 2, 1)
    assert np.array_equal(out[128], out[256])


def test_gemm_rounding_to_bf16_is_the_oracles(xs, gpu, gemm_tile):
    """Every C[i][j] here is ONE product a_i * b_j (the other 63 terms of the sum are 0 * 0),
    so the fp32 accumulator holds it exactly and the stored bf16 shows the rounding alone:
    ties to even, carries into the exponent, overflow to infinity, denormal results,
    infinities and NaNs. Bit for bit the oracle's (u + 0x7FFF + lsb) >> 16 with quieted NaNs."""
    torch = gpu
    M = N = 256
    K = 64
    print("case gemm-rounding", flush=True)
    rng = np.random.default_rng(7)

    def interesting(count):
        bits = rng.integers(0, 1 << 16, count).astype(np.uint16)            # any bf16 at all
        bits[:8] = [0x0000, 0x8000, 0x7F80, 0xFF80, 0x7FC0, 0x7F81, 0x0001, 0x807F]
        bits[8:16] = [0x3F80, 0x3F81, 0x3FFF, 0x4000, 0x7F7F, 0x0080, 0x3F7F, 0xBF81]
        bits[16:96] = rng.integers(0x3F80, 0x4080, 80).astype(np.uint16)    # products around 1..4 hit ties often
        bits[96:128] = rng.integers(0x0001, 0x0100, 32).astype(np.uint16)   # denormal and tiny operands
        return bits

    a_col, b_row = interesting(M), interesting(N)
    a_bits = np.zeros((M, K), np.uint16)
    b_bits = np.zeros((K, N), np.uint16)
    a_bits[:, 5] = a_col
    b_bits[5, :] = b_row
    got = _gemm_case(xs, torch, a_bits.ravel(), b_bits.ravel(), M, N, K, 1, 0).reshape(M, N)
    want = oracle.gemm_bf16(a_bits.ravel(), b_bits.ravel(), M, N, K).reshape(M, N)

    def is_nan(h):
        return (h & 0x7FFF) > 0x7F80
    nan_want = is_nan(want)
    assert np.array_equal(is_nan(got), nan_want)
    # which NaN comes out (sign, payload) is the matrix unit's business: it answers every
    # NaN, passed through or made by inf * 0, with its default NaN, the oracle's fmaf keeps
    # the operand's. Only that it IS a NaN is compared.
    same = (got == want) | nan_want
    bad = np.argwhere(~same)
    assert bad.size == 0, [(hex(a_col[i]), hex(b_row[j]), hex(got[i, j]), hex(want[i, j])) for i, j in bad[:8]]
    assert np.count_nonzero(~nan_want) > 60000


def test_gemm_normal_inputs_within_tolerance(xs, gpu, gemm_tile):
    """Seeded N(0,1)-like inputs: the MFMA's internal summation order is not the
    oracle's, so the comparison is on values. Tolerance: one bf16 unit in the last
    place of the result (2^-8 relative) plus fp32 accumulation noise 2^-20*sqrt(K)."""
    M, N, K = 256, 256, 512
    a_bits = oracle.fill_normal_bf16(11, 1, 0, M * K)
    b_bits = oracle.fill_normal_bf16(11, 2, 0, K * N)
    got = _gemm_case(xs, gpu, a_bits, b_bits, M, N, K, 2, 1)
    want_bits, want_f32 = oracle.gemm_bf16(a_bits, b_bits, M, N, K, want_f32=True)
    got_f = oracle.bf16_bits_to_f32(got.ravel()).reshape(M, N)
    tol = np.abs(want_f32) * 2.0 ** -8 + 2.0 ** -20 * np.sqrt(K) * 16
    assert np.all(np.abs(got_f - want_f32) <= tol)
    assert np.mean(got == want_bits) > 0.95
