"""Writes tests/golden/kernel_vectors.json: known answers for the seeded synthetic inputs
and the victim kernels, computed WITHOUT the C oracle and without the device code.

    python tests/golden/make_kernel_vectors.py

Arithmetic used here, on purpose different from oracle/kernels.c:
  * SplitMix64 on Python integers (arbitrary precision, masked to 64 bits), anchored on the
    generator's published test vector (seed 0: E220A8397B1DCDAF, 6E789E6AA1B965F4,
    06C45D188009454F).
  * uniform values as exact fractions (u - 2^23) / 2^23, which every fp32 holds exactly.
  * bf16 rounding by comparing the exact distances to the two neighbouring bf16 values
    (fractions, ties to the even mantissa), not by the add-and-shift formula.
  * the Zipf table with 60-digit decimal arithmetic (decimal.Decimal), not long double.
  * AXPY for a general alpha as the exact rational alpha * x + y rounded once to fp32
    (fractions), which is what a fused multiply-add is defined to return.
The 2^22-key bin counts use numpy uint64 arithmetic for speed; that vectorised generator is
checked against the integer one on its first 4096 draws before it is used.
"""
import bisect
import json
import os
import struct
from decimal import Decimal, getcontext
from fractions import Fraction

import numpy as np

M64 = (1 << 64) - 1
GAMMA = 0x9E3779B97F4A7C15
STREAM_MUL = 0xD1B54A32D192ED03


def mix(z):
    """One SplitMix64 output for the state that precedes it (state += gamma, then finalise)."""
    z = (z + GAMMA) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def stream_key(seed, stream):
    return mix(seed ^ ((stream * STREAM_MUL) & M64))


def bits(key, i):
    return mix((key + i) & M64)


def f32_bits(x):
    """Bits of the fp32 nearest to the Python float / Fraction x (ties to even)."""
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def f32_value(b):
    return Fraction(struct.unpack("<f", struct.pack("<I", b))[0])


def round_fraction_to_f32_bits(q):
    """Correctly rounded fp32 of an exact rational: via float64 when that is exact enough,
    decided by exact comparison with the two neighbouring fp32 values."""
    if q == 0:
        return 0
    guess = f32_bits(float(q))  # double rounding possible: repair below
    cands = {guess}
    for d in (-1, 1):
        g = guess + d
        if 0 <= (g & 0x7FFFFFFF) < 0x7F800000:
            cands.add(g)
    # a neighbour on the other side of zero
    best = None
    for b in cands:
        dist = abs(f32_value(b) - q)
        even = (b & 1) == 0
        key = (dist, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, b)
    return best[1]


def bf16_bits_of_f32_bits(b):
    """Round an fp32 (finite) to bf16, ties to even, by exact distances."""
    lo = b & 0xFFFF0000          # truncation towards zero
    hi = lo + 0x10000            # next bf16 away from zero (may be infinity)
    v, vlo = f32_value(b), f32_value(lo)
    if (hi & 0x7F800000) == 0x7F800000:
        # next value is infinity: its place in the rounding is 2^128 with an even mantissa
        sign = -1 if b >> 31 else 1
        vhi = Fraction(sign * (1 << 128))
    else:
        vhi = f32_value(hi)
    dlo, dhi = abs(v - vlo), abs(vhi - v)
    if dlo < dhi:
        return lo >> 16
    if dhi < dlo:
        return hi >> 16
    return (lo >> 16) if ((lo >> 16) & 1) == 0 else (hi >> 16)


def uniform_bits(key, i):
    u = bits(key, i) >> 40
    return f32_bits(Fraction(u - (1 << 23), 1 << 23))


def normal_bf16(key, i):
    total = 0
    for k in range(6):
        b = bits(key, i * 6 + k)
        total += (b >> 40) + ((b >> 16) & 0xFFFFFF)
    total -= 6 << 24
    as_f32 = round_fraction_to_f32_bits(Fraction(total))        # (float)sum
    scaled = f32_bits(f32_value(as_f32) / (1 << 24))            # exact: power of two
    return bf16_bits_of_f32_bits(scaled)


def zipf_table(n_bins, s_text):
    getcontext().prec = 60
    s = Decimal(s_text)
    h, acc = [], Decimal(0)
    for k in range(1, n_bins + 1):
        acc += (Decimal(k).ln() * -s).exp()
        h.append(acc)
    two32 = Decimal(1 << 32)
    t = [min(int((two32 * v / acc).to_integral_value(rounding="ROUND_FLOOR")), 0xFFFFFFFF) for v in h]
    t[-1] = 0xFFFFFFFF
    return t


def zipf_key(table, key, i):
    u = bits(key, i) >> 32
    return min(bisect.bisect_right(table, u), len(table) - 1)


def np_mix(z):
    z = z + np.uint64(GAMMA)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def main():
    out = {}
    out["splitmix64_published_seed0"] = ["%016X" % mix(0), "%016X" % mix(GAMMA), "%016X" % mix((2 * GAMMA) & M64)]
    assert out["splitmix64_published_seed0"] == ["E220A8397B1DCDAF", "6E789E6AA1B965F4", "06C45D188009454F"]

    out["stream_keys"] = {"%d,%d" % (s, t): "%016X" % stream_key(s, t)
                          for s, t in [(0, 0), (0, 1), (0, 4), (7, 5), (7, 1003), (123456789, 2)]}

    out["uniform_first16_bits"] = {
        "%d,%d" % (s, t): ["%08X" % uniform_bits(stream_key(s, t), i) for i in range(16)]
        for s, t in [(0, 0), (0, 1), (7, 4)]}
    out["uniform_at_2p28_minus_2_bits"] = ["%08X" % uniform_bits(stream_key(0, 0), (1 << 28) - 2 + j) for j in range(2)]

    out["normal_bf16_first16"] = {
        "%d,%d" % (s, t): ["%04X" % normal_bf16(stream_key(s, t), i) for i in range(16)]
        for s, t in [(0, 0), (0, 1)]}

    table = zipf_table(65536, "1.1")
    out["zipf_table_65536_s1.1"] = {
        "first16": table[:16], "at": {str(k): table[k] for k in (100, 1000, 32767, 32768, 65534, 65535)},
        "sum_mod_2p32": sum(table) & 0xFFFFFFFF}
    key = stream_key(0, 0)
    out["zipf_first32_keys"] = {"0,0": [zipf_key(table, key, i) for i in range(32)]}

    # bins 0..15 (and the total of the rest) of 2^22 keys, streams (0,0) and (0,4)
    tab = np.array(table, np.uint64)
    with np.errstate(over="ignore"):
        for s, t in [(0, 0), (0, 4)]:
            k = stream_key(s, t)
            idx = np.arange(1 << 22, dtype=np.uint64)
            draws = np_mix(np.uint64(k) + idx) >> np.uint64(32)
            assert [int(v) for v in draws[:4096]] == [bits(k, i) >> 32 for i in range(4096)]
            keys = np.minimum(np.searchsorted(tab, draws, side="right"), 65535)
            counts = np.bincount(keys, minlength=65536)
            out.setdefault("zipf_2p22_bins", {})["%d,%d" % (s, t)] = {
                "bins0_15": [int(c) for c in counts[:16]], "rest": int(counts[16:].sum()),
                "bin65535": int(counts[65535]), "nonzero_bins": int((counts > 0).sum())}

    # AXPY with a general alpha: exact rational result rounded once
    kx, ky = stream_key(0, 0), stream_key(0, 1)
    cases = []
    for alpha in (0.5, 0.1, -1.7, 3.0e-5, 1.0 / 3.0):
        a_bits = f32_bits(alpha)
        a = f32_value(a_bits)
        res = []
        for i in range(256):
            x, y = f32_value(uniform_bits(kx, i)), f32_value(uniform_bits(ky, i))
            res.append("%08X" % round_fraction_to_f32_bits(a * x + y))
        cases.append({"alpha_bits": "%08X" % a_bits, "y_bits": res})
    out["axpy_fma_256"] = {"x_stream": "0,0", "y_stream": "0,1", "cases": cases}

    # bf16 rounding known answers (value bits -> bf16 bits), including ties and carries
    probes = [0x3F800000, 0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x3FFF8000, 0x7F7F8000,
              0x7F7F7FFF, 0x00008000, 0x00018000, 0x80008000, 0xBF808000, 0xC0FF8000, 0x3EAAAAAB]
    out["bf16_rne"] = [["%08X" % b, "%04X" % bf16_bits_of_f32_bits(b)] for b in probes]

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_vectors.json")
    with open(path, "w") as f:
        f.write("{\n" + ",\n".join(" %s: %s" % (json.dumps(k), json.dumps(out[k], sort_keys=True))
                                    for k in sorted(out)) + "\n}\n")
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
