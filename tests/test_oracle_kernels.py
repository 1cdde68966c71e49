"""Pins of oracle/kernels.c (CPU only): every function of the kernel oracle is held against
something that does not repeat its formula.

  * tests/golden/kernel_vectors.json was written by tests/golden/make_kernel_vectors.py with
    Python integers, fractions and 60-digit decimals (no C, no long double, no add-and-shift
    rounding): SplitMix64 anchored on its published vector, first values of every generator,
    the Zipf table, bins 0..15 of 2^22 keys, fused multiply-add results as exact rationals
    rounded once.
  * numpy for what numpy defines (mul-add at alpha = 0.5, bincount, matmul in float64).
  * closed forms of the percentile rule of the reference
    (utils/include/xsched/utils/data.h:57-65: sorted data, index = size * p, no interpolation).
  * properties of the Zipf table that follow from the distribution, not from the table's code.
"""
import json
import math
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "kernel_vectors.json")) as f:
    GOLD = json.load(f)

GAMMA = 0x9E3779B97F4A7C15


def _pair(text):
    s, t = text.split(",")
    return int(s), int(t)


# ---- generators -------------------------------------------------------------------------

def test_splitmix64_published_vector():
    # Steele, Lea, Flood: SplitMix64 seeded with 0 gives these three outputs.
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    got = [oracle.bits(0, 0), oracle.bits(GAMMA, 0), oracle.bits((2 * GAMMA) & (2**64 - 1), 0)]
    assert got == want
    assert [int(v, 16) for v in GOLD["splitmix64_published_seed0"]] == want
    # index and key add: bits(key, i) == bits(key + i, 0)
    assert oracle.bits(5, 7) == oracle.bits(12, 0)


def test_stream_keys_match_the_fixture():
    for text, want in GOLD["stream_keys"].items():
        assert oracle.stream_key(*_pair(text)) == int(want, 16), text


def test_uniform_first_values_and_range():
    for text, want in GOLD["uniform_first16_bits"].items():
        seed, stream = _pair(text)
        got = oracle.fill_uniform(seed, stream, 0, 16).view(np.uint32)
        assert [int(v) for v in got] == [int(w, 16) for w in want], text
    tail = oracle.fill_uniform(0, 0, (1 << 28) - 2, 2).view(np.uint32)
    assert [int(v) for v in tail] == [int(w, 16) for w in GOLD["uniform_at_2p28_minus_2_bits"]]
    # `first` is an offset into one stream, not a new stream
    whole = oracle.fill_uniform(3, 9, 0, 1000)
    assert np.array_equal(whole[137:], oracle.fill_uniform(3, 9, 137, 863))
    # distribution: U[-1, 1) on a grid of 2^-23
    big = oracle.fill_uniform(0, 0, 0, 1 << 20)
    assert big.min() >= -1.0 and big.max() < 1.0
    assert np.array_equal(big * 8388608.0, np.round(big * 8388608.0))
    assert abs(float(big.mean())) < 4 / math.sqrt(3 * (1 << 20))
    assert abs(float(big.astype(np.float64).var()) - 1 / 3) < 2e-3


def test_normal_bf16_first_values_and_moments():
    for text, want in GOLD["normal_bf16_first16"].items():
        seed, stream = _pair(text)
        got = oracle.fill_normal_bf16(seed, stream, 0, 16)
        assert [int(v) for v in got] == [int(w, 16) for w in want], text
    vals = oracle.bf16_bits_to_f32(oracle.fill_normal_bf16(0, 0, 0, 1 << 18)).astype(np.float64)
    assert abs(vals.mean()) < 0.01 and abs(vals.var() - 1.0) < 0.02
    assert np.abs(vals).max() <= 6.0  # a sum of twelve uniforms cannot leave [-6, 6]


def test_bf16_rounding_known_answers():
    for value_bits, want in GOLD["bf16_rne"]:
        f = np.array([int(value_bits, 16)], np.uint32).view(np.float32)[0]
        assert oracle.lib().oracle_f32_to_bf16(float(f)) == int(want, 16), value_bits
    # NaN stays NaN (quiet), infinity stays infinity
    assert oracle.lib().oracle_f32_to_bf16(float("inf")) == 0x7F80
    assert oracle.lib().oracle_f32_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0


def test_zipf_table_against_the_fixture_and_the_distribution():
    t = oracle.zipf_table(65536, 1.1)
    gold = GOLD["zipf_table_65536_s1.1"]
    assert [int(v) for v in t[:16]] == gold["first16"]
    for k, v in gold["at"].items():
        assert int(t[int(k)]) == v, k
    assert int(t.astype(np.uint64).sum()) & 0xFFFFFFFF == gold["sum_mod_2p32"]
    # what the distribution fixes, without the table's own formula:
    assert np.all(np.diff(t.astype(np.int64)) >= 0)          # a CDF is monotone
    assert int(t[-1]) == 2**32 - 1                            # and ends at 1
    h = math.fsum((k + 1) ** -1.1 for k in range(65536))     # generalised harmonic number
    assert abs(int(t[0]) / 2**32 - 1.0 / h) < 2**-31         # P(key 0) = 1 / H
    assert abs(1.0 / h - 0.138) < 0.002                      # about 13.8 % of all keys
    # P(key k) / P(key 0) = (k + 1)^-1.1, read off the table's increments
    for k in (1, 2, 9, 99, 999):
        ratio = (int(t[k]) - int(t[k - 1])) / int(t[0])
        assert abs(ratio - (k + 1) ** -1.1) < 1e-8      # two floors over t[0] ~ 5.9e8


def test_zipf_keys_first_values_and_bins_of_2p22():
    table = oracle.zipf_table(65536, 1.1)
    for text, want in GOLD["zipf_first32_keys"].items():
        seed, stream = _pair(text)
        assert [int(v) for v in oracle.fill_zipf(seed, stream, 0, 32, table)] == want, text
    for text, want in GOLD["zipf_2p22_bins"].items():
        seed, stream = _pair(text)
        keys = oracle.fill_zipf(seed, stream, 0, 1 << 22, table)
        assert keys.min() >= 0 and keys.max() <= 65535
        bins = oracle.histogram(keys, 65536)
        assert [int(v) for v in bins[:16]] == want["bins0_15"], text
        assert int(bins[16:].astype(np.uint64).sum()) == want["rest"]
        assert int(bins[65535]) == want["bin65535"]
        assert int((bins > 0).sum()) == want["nonzero_bins"]
        assert abs(want["bins0_15"][0] / (1 << 22) - 0.138) < 0.002  # bin-0 share of the draws


# ---- kernels ----------------------------------------------------------------------------

def test_vecadd_is_one_ieee_addition():
    a = oracle.fill_uniform(0, 0, 0, 4099)
    b = oracle.fill_uniform(0, 1, 0, 4099)
    assert np.array_equal(oracle.vecadd(a, b).view(np.uint32), (a + b).view(np.uint32))
    # the reference's known answer: k chained additions of ones give k
    # (platforms/example/test/src/vecadd.cpp:91-102)
    acc = np.zeros(64, np.float32)
    for _ in range(1024):
        acc = oracle.vecadd(acc, np.ones(64, np.float32))
    assert np.all(acc == 1024.0)


def test_axpy_alpha_half_equals_numpy_mul_add_bit_for_bit():
    x = oracle.fill_uniform(0, 0, 0, 100003)
    y = oracle.fill_uniform(0, 1, 0, 100003)
    got = oracle.axpy(0.5, x, y)
    want = np.float32(0.5) * x + y          # the product is exact, so fused == unfused
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # repeated application keeps agreeing (what the GPU tests rely on)
    got5, want5 = oracle.axpy(0.5, x, y, times=5), y.copy()
    for _ in range(5):
        want5 = np.float32(0.5) * x + want5
    assert np.array_equal(got5.view(np.uint32), want5.view(np.uint32))


def test_axpy_general_alpha_is_a_single_rounding():
    g = GOLD["axpy_fma_256"]
    x = oracle.fill_uniform(*_pair(g["x_stream"]), 0, 256)
    y = oracle.fill_uniform(*_pair(g["y_stream"]), 0, 256)
    differs_from_unfused = 0
    for case in g["cases"]:
        alpha = np.array([int(case["alpha_bits"], 16)], np.uint32).view(np.float32)[0]
        got = oracle.axpy(alpha, x, y).view(np.uint32)
        want = np.array([int(v, 16) for v in case["y_bits"]], np.uint32)
        assert np.array_equal(got, want), case["alpha_bits"]
        differs_from_unfused += int(np.count_nonzero(got != (alpha * x + y).view(np.uint32)))
    # the vectors do tell a fused multiply-add from multiply-then-add
    assert differs_from_unfused > 0


def test_axpy_empty_and_single():
    assert oracle.axpy(0.5, np.zeros(0, np.float32), np.zeros(0, np.float32)).size == 0
    assert oracle.axpy(2.0, np.array([3.0], np.float32), np.array([1.0], np.float32))[0] == 7.0


def test_histogram_equals_bincount_with_out_of_range_keys_and_wrap():
    rng = np.random.default_rng(5)
    keys = rng.integers(-50, 1100, size=200001).astype(np.int32)
    keys[::1000] = np.int32(-2**31)
    keys[1::1000] = np.int32(2**31 - 1)
    n_bins = 1000
    inside = keys[(keys >= 0) & (keys < n_bins)]
    want = np.bincount(inside, minlength=n_bins).astype(np.uint32)
    assert np.array_equal(oracle.histogram(keys, n_bins), want)
    # bins are added to, not cleared, and wrap modulo 2^32
    start = np.full(n_bins, 0xFFFFFFFF, np.uint32)
    got = oracle.histogram(keys, n_bins, bins=start)
    assert np.array_equal(got, (want.astype(np.uint64) + 0xFFFFFFFF).astype(np.uint32))
    assert np.array_equal(oracle.histogram(np.zeros(0, np.int32), 16), np.zeros(16, np.uint32))
    assert int(oracle.histogram(np.full(70000, 3, np.int32), 8)[3]) == 70000


def test_gemm_integer_inputs_are_exact_and_order_is_ascending_k():
    rng = np.random.default_rng(11)
    M, N, K = 24, 40, 96
    a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    b = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    c_bits, c_f32 = oracle.gemm_bf16(oracle.f32_to_bf16_bits(a).ravel(), oracle.f32_to_bf16_bits(b).ravel(),
                                     M, N, K, want_f32=True)
    exact = a.astype(np.int64) @ b.astype(np.int64)
    assert np.array_equal(c_f32.astype(np.int64), exact)
    # |sums| <= 16 * 96 = 1536 < 2^8 * 8: not all fit bf16 exactly; the rounding is the fixture-pinned one
    want_bits = np.array([oracle.lib().oracle_f32_to_bf16(float(v)) for v in exact.ravel()], np.uint16)
    assert np.array_equal(c_bits.ravel(), want_bits)
    # ascending k with one rounding per step: a sum that depends on the order.
    # 2^24 first: every following + 1 is a tie that rounds back to 2^24.
    # 2^24 last: 63 ones add up exactly, and 2^24 + 63 rounds (tie, to even) to 2^24 + 64.
    K2 = 64
    a2 = np.ones((1, K2), np.float32); b2 = np.ones((K2, 1), np.float32)
    a2[0, 0] = 2.0**8; b2[0, 0] = 2.0**16          # both exact in bf16, product 2^24
    _, f = oracle.gemm_bf16(oracle.f32_to_bf16_bits(a2).ravel(), oracle.f32_to_bf16_bits(b2).ravel(), 1, 1, K2, want_f32=True)
    assert float(f[0, 0]) == 2.0**24
    a3, b3 = a2[:, ::-1].copy(), b2[::-1, :].copy()
    _, f = oracle.gemm_bf16(oracle.f32_to_bf16_bits(a3).ravel(), oracle.f32_to_bf16_bits(b3).ravel(), 1, 1, K2, want_f32=True)
    assert float(f[0, 0]) == 2.0**24 + 64


def test_gemm_normal_inputs_within_float64_tolerance():
    M, N, K = 32, 48, 256
    a = oracle.fill_normal_bf16(0, 0, 0, M * K)
    b = oracle.fill_normal_bf16(0, 1, 0, K * N)
    _, f = oracle.gemm_bf16(a, b, M, N, K, want_f32=True)
    ref = oracle.bf16_bits_to_f32(a).astype(np.float64).reshape(M, K) @ oracle.bf16_bits_to_f32(b).astype(np.float64).reshape(K, N)
    # fp32 accumulation of K products: error below K * 2^-24 * sum |a||b|
    bound = K * 2.0**-24 * (np.abs(oracle.bf16_bits_to_f32(a).astype(np.float64).reshape(M, K))
                            @ np.abs(oracle.bf16_bits_to_f32(b).astype(np.float64).reshape(K, N)))
    assert np.all(np.abs(f.astype(np.float64) - ref) <= bound)


# ---- percentile rule ---------------------------------------------------------------------

@pytest.mark.parametrize("n,p,index", [
    (1, 0.5, 0), (1, 0.99, 0), (100, 0.99, 99), (100, 0.5, 50), (400, 0.99, 396), (20, 0.99, 19),
    (10, 0.25, 2), (7, 0.5, 3), (1000, 0.999, 999), (3, 0.0, 0),
])
def test_percentile_is_sorted_at_floor_p_times_n(n, p, index):
    # reference rule: sort, then data[size * p] with the product truncated to an index
    data = list(range(1000, 1000 + n))
    shuffled = np.random.default_rng(n).permutation(data)
    assert oracle.percentile(shuffled, p) == float(data[index])


def test_percentile_has_no_interpolation_and_handles_ties():
    assert oracle.percentile([1.0, 2.0], 0.5) == 2.0
    assert oracle.percentile([5.0, 5.0, 5.0, 9.0], 0.74) == 5.0
    assert oracle.percentile([5.0, 5.0, 5.0, 9.0], 0.75) == 9.0
