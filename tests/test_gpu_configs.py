"""GPU: the benchmark configurations end to end through the native harness (the same
entry points bench.py uses), at sizes the CPU oracle finishes in seconds and, for the
size-independent properties, at the full sizes. Whatever the scheduler did to the queues
(window stalls, suspensions, Level-2 flushes and replays), every output buffer must hold
exactly what `applied` uninterrupted commands produce."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

N_BINS = 65536


@pytest.fixture(scope="module")
def H(xs, gpu):
    from xsched_amd import harness
    harness.lib()
    yield harness
    # later test modules drive suspend / resume by hand: no scheduler must interfere
    xs.check(xs.preempt().XHintSetScheduler(xs.kSchedulerAppManaged, xs.kPolicyUnknown))


def lane_streams(lane_id):
    """Input streams of harness lane `lane_id` (0 = foreground, i + 1 = background i)."""
    return lane_id * 4, lane_id * 4 + 1


def check_axpy(b, which, q, lane_id, n, seed=0, first=0, count=None):
    count = n if count is None else count
    got, applied = b.read(which, q, first, count, np.float32)
    s0, s1 = lane_streams(lane_id)
    x = oracle.fill_uniform(seed, s0, first, count)
    y = oracle.fill_uniform(seed, s1, first, count)
    want = oracle.axpy(0.5, x, y, applied)
    if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
        raise AssertionError(f"axpy lane {lane_id}: output differs from {applied} uninterrupted applications: "
                             + describe_axpy_mismatch(got, x, y, applied, first))
    return applied


def describe_axpy_mismatch(got, x, y, applied, first):
    """Which 1024-element chunks differ, and whether they hold one application more or fewer."""
    bad = np.flatnonzero(got.view(np.uint32) != oracle.axpy(0.5, x, y, applied).view(np.uint32))
    chunks = np.unique((bad + first) // 1024)
    notes = []
    for k in (applied - 2, applied - 1, applied + 1, applied + 2):
        if k < 0:
            continue
        alt = oracle.axpy(0.5, x, y, k)
        notes.append("%d of them equal %d applications" % (int(np.sum(got[bad].view(np.uint32) == alt[bad].view(np.uint32))), k))
    runs = np.split(chunks, np.flatnonzero(np.diff(chunks) != 1) + 1)
    spans = ["%d-%d" % (r[0], r[-1]) if len(r) > 1 else str(r[0]) for r in runs[:12]]
    return "%d elements in %d chunks of 1024 (%s%s); %s" % (len(bad), len(chunks), ", ".join(spans),
                                                           ", ..." if len(runs) > 12 else "", "; ".join(notes))


def check_hist(b, which, q, lane_id, n, seed=0):
    got, applied = b.read(which, q, 0, N_BINS, np.uint32)
    s0, _ = lane_streams(lane_id)
    one = oracle.histogram(oracle.fill_zipf(seed, s0, 0, n), N_BINS).astype(np.uint64)
    assert int(one.sum()) == n
    assert np.array_equal(got.astype(np.uint64), (one * applied) & 0xFFFFFFFF), \
        f"histogram lane {lane_id}: bins differ from {applied} x the oracle's counts"
    return applied


def check_gemm_rows(b, which, q, lane_id, n, rows, seed=0):
    """Rows [r, r + 4) of C against the oracle (ascending-k fmaf, RNE), within the
    tolerance the MFMA summation order allows: 2^-8 relative + 2^-16 * sqrt(K) absolute."""
    s0, s1 = lane_streams(lane_id)
    bmat = oracle.fill_normal_bf16(seed, s1, 0, n * n)
    for r in rows:
        got, applied = b.read(which, q, r * n, 4 * n, np.uint16)
        a = oracle.fill_normal_bf16(seed, s0, r * n, 4 * n)
        _, want_f32 = oracle.gemm_bf16(a, bmat, 4, n, n, want_f32=True)
        gf = oracle.bf16_bits_to_f32(got).reshape(4, n)
        tol = np.abs(want_f32) * 2.0 ** -8 + 2.0 ** -16 * np.sqrt(n)
        assert np.all(np.abs(gf - want_f32) <= tol), f"gemm lane {lane_id} rows {r}..{r + 3}"
    return applied


def test_config2_level1_axpy_contention(H):
    bg_n, fg_n = 1 << 22, 1 << 16
    print(f"case cfg2 bg={bg_n} fg={fg_n}", flush=True)
    cfg = H.Config(H.HPF, 1, H.spec(H.AXPY, bg_n, 1, 1, 2, 1, 1),
                   H.spec(H.AXPY, fg_n, 0, 1, 8, 4, 2, period_us=2000), 16, 0)
    with H.Bench(cfg) as b:
        alone, _ = b.fg_alone(20)
        cont, res = b.contended(40)
        assert len(cont) == 40 and all(v > 0 for v in alone + cont)
        assert res.bg_commands > 0
        assert check_axpy(b, 1, 0, 0, fg_n) == 60
        assert check_axpy(b, 0, 0, 1, bg_n) == res.bg_commands
        assert res.stats[2] == 0, "level 1 never deactivates"


def test_config3_level2_gemm_preempted_equals_uninterrupted(H):
    bg_n, fg_n = 1024, 256
    print(f"case cfg3 bg={bg_n} fg={fg_n}", flush=True)
    cfg = H.Config(H.HPF, 1, H.spec(H.GEMM, bg_n, 1, 2, 2, 1, 1),
                   H.spec(H.GEMM, fg_n, 0, 1, 8, 4, 2, period_us=1000), 16, 0)
    with H.Bench(cfg) as b:
        b.bg_alone(1)
        clean, _ = b.read(0, 0, 0, bg_n * bg_n, np.uint16)
        cont, res = b.contended(60)
        sus, resume, pres = b.preempt(40)
        assert res.stats[2] > 0, "the scheduler never deactivated the background queue"
        # (a suspension that finds nothing in flight, between two bursts, deactivates nothing)
        assert pres.stats[2] >= res.stats[2] + 25, "the preemption loop did not deactivate it"
        after, applied = b.read(0, 0, 0, bg_n * bg_n, np.uint16)
        assert applied > 1
        assert np.array_equal(clean, after), "preempted-and-resumed GEMM differs from the uninterrupted one"
        check_gemm_rows(b, 0, 0, 1, bg_n, [0, 508, 1020])
        check_gemm_rows(b, 1, 0, 0, fg_n, [0, 252])


def test_config4_laxity_histogram_four_background_queues(H):
    bg_n, fg_n = 1 << 22, 1 << 16
    print(f"case cfg4 bg=4x{bg_n} fg={fg_n}", flush=True)
    cfg = H.Config(H.LAX, 4, H.spec(H.HIST, bg_n, 1, 2, 2, 1, 0),
                   H.spec(H.HIST, fg_n, 0, 1, 8, 4, 1, laxity_us=100, period_us=1000, lax_priority=0,
                          deadline_us=1000), 16, 0)
    with H.Bench(cfg) as b:
        cont, res = b.contended(80)
        assert res.fg_samples == 80 and 0 <= res.fg_deadline_miss <= 80
        assert res.bg_commands > 0
        total = 0
        for q in range(4):
            total += check_hist(b, 0, q, q + 1, bg_n)
        assert total == res.bg_commands
        assert check_hist(b, 1, 0, 0, fg_n) == 80


def test_config5_mixed_stress_sixteen_queues(H):
    axpy_n, gemm_n, hist_n, nq = 1 << 20, 512, 1 << 20, 16
    print("case cfg5 reduced", flush=True)
    cfg = H.StressConfig(H.HPF, nq, 2, 1, 4, 2, axpy_n, gemm_n, hist_n, 1000.0, 7)
    with H.Bench(cfg) as b:
        lat, res = b.stress(0.4)
        counts = [len(x) for x in lat]
        assert all(c > 100 for c in counts), counts          # ~400 arrivals per queue
        assert sum(counts) == res.bg_commands
        # the arrival process is the documented one: same seed, same counts on every run
        assert counts == expected_arrivals(nq, 0.4, 1000.0, 7)
        for i in range(nq):
            if i % 3 == 0:
                assert check_axpy(b, 0, i, i + 1, axpy_n, seed=7) == counts[i]
            elif i % 3 == 1:
                assert check_gemm_rows(b, 0, i, i + 1, gemm_n, [0, 256, 508], seed=7) == counts[i]
            else:
                assert check_hist(b, 0, i, i + 1, hist_n, seed=7) == counts[i]
        # highest priority is never held back by the scheduler
        assert H.pct(lat[nq - 1], 0.5) < H.pct(lat[0], 0.99) * 10 + 1e6


def expected_arrivals(nq, duration_s, mean_us, seed):
    """Arrival counts of the stress run restated from the header: interval k of queue i is
    -mean * ln(1 - u), u = top 53 bits of synthetic stream (seed, 1000 + i) at index k."""
    out = []
    for i in range(nq):
        key = oracle.stream_key(seed, 1000 + i)
        t, k = 0.0, 0
        while True:
            u = (oracle.bits(key, k) >> 11) / 9007199254740992.0
            t += -mean_us * np.log1p(-u)
            if t > duration_s * 1e6:
                break
            k += 1
        out.append(k)
    return out


def test_full_size_gemm_preempted_is_bit_identical(H):
    """8192^3 at Level 2 under the preemption loop: C never changes from the uninterrupted
    result (each tile has one summation order; abandoned tiles leave no trace)."""
    n = 8192
    print("case cfg3 full size", flush=True)
    cfg = H.Config(0, 1, H.spec(H.GEMM, n, 1, 2, 2, 1, 1), H.spec(H.GEMM, 0, 0, 1, 8, 4, 2), 16, 0)
    with H.Bench(cfg) as b:
        b.bg_alone(1)
        clean, _ = b.read(0, 0, 0, n * n, np.uint16)
        sus, resume, res = b.preempt(60)
        assert res.stats[2] >= 45 and res.stats[1] > 0, "no flush / replay happened"   # 60 suspensions, most of them with work in flight
        after, applied = b.read(0, 0, 0, n * n, np.uint16)
        assert np.array_equal(clean, after)
        check_gemm_rows(b, 0, 0, 1, n, [4096])


def test_full_size_histogram_counts_after_preemption(H):
    """2^26 Zipf keys at Level 2 under the preemption loop: the bins are an exact multiple
    of one uninterrupted pass and sum to applied * 2^26."""
    n = 1 << 26
    print("case cfg4 full size", flush=True)
    cfg = H.Config(0, 1, H.spec(H.HIST, n, 1, 2, 2, 1, 1), H.spec(H.HIST, 0, 0, 1, 8, 4, 2), 16, 0)
    with H.Bench(cfg) as b:
        b.bg_alone(1)
        one, k1 = b.read(0, 0, 0, N_BINS, np.uint32)
        assert k1 == 1 and int(one.astype(np.uint64).sum()) == n
        sus, resume, res = b.preempt(40)
        assert res.stats[2] >= 30   # 40 suspensions, most of them with work in flight
        bins, applied = b.read(0, 0, 0, N_BINS, np.uint32)
        assert np.array_equal(bins.astype(np.uint64), (one.astype(np.uint64) * applied) & 0xFFFFFFFF)
        # head of the distribution against the oracle's generator on the first 2^22 keys
        part = oracle.histogram(oracle.fill_zipf(0, 4, 0, 1 << 22), N_BINS)
        assert abs(int(one[0]) / n - int(part[0]) / (1 << 22)) < 2e-3
