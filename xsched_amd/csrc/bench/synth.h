// Seeded synthetic inputs of the benchmark workloads. Everything is integer
// arithmetic plus exact int -> float conversions, so the device fill kernels and
// a CPU restatement produce identical bits.
//
//   bits(seed, stream, i) = splitmix64(splitmix64(seed ^ stream * C) + i)
//   uniform[-1,1)  : top 24 bits u -> (float)u * 2^-23 - 1
//   normal-ish     : Irwin-Hall, sum of twelve 24-bit uniforms minus 6 * 2^24, scaled
//                    by 2^-24 (mean 0, variance 1), rounded to bf16 (nearest even)
//   zipf(s) key    : inverse CDF through an integer table: key = number of table
//                    entries <= u32 draw; table[k] = floor(2^32 * H(k+1)/H(n_bins))
//                    (H = generalised harmonic number, long double), last entry 2^32-1
#pragma once

#include <stdint.h>

#ifdef __HIPCC__
#define SYNTH_FN __host__ __device__ inline
#else
#define SYNTH_FN inline
#endif

SYNTH_FN uint64_t synth_splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

SYNTH_FN uint64_t synth_stream_key(uint64_t seed, uint64_t stream)
{
    return synth_splitmix64(seed ^ (stream * 0xD1B54A32D192ED03ull));
}

SYNTH_FN uint64_t synth_bits(uint64_t stream_key, uint64_t i) { return synth_splitmix64(stream_key + i); }

SYNTH_FN float synth_uniform_pm1(uint64_t stream_key, uint64_t i)
{
    const uint32_t u = (uint32_t)(synth_bits(stream_key, i) >> 40); // 24 bits
    return (float)u * (1.0f / 8388608.0f) - 1.0f;
}

SYNTH_FN uint16_t synth_f32_to_bf16_rne(float f)
{
    union { float f; uint32_t u; } v = { f };
    const uint32_t lsb = (v.u >> 16) & 1u;
    return (uint16_t)((v.u + 0x7FFFu + lsb) >> 16); // inputs are finite
}

SYNTH_FN uint16_t synth_normal_bf16(uint64_t stream_key, uint64_t i)
{
    int64_t sum = 0;
    for (int k = 0; k < 6; ++k) {
        const uint64_t b = synth_bits(stream_key, i * 6 + k);
        sum += (int64_t)(b >> 40) + (int64_t)((b >> 16) & 0xFFFFFFull);
    }
    sum -= 6ll * 16777216ll;
    return synth_f32_to_bf16_rne((float)sum * (1.0f / 16777216.0f));
}

SYNTH_FN uint32_t synth_zipf_key(const uint32_t *table, uint32_t n_bins, uint64_t stream_key, uint64_t i)
{
    const uint32_t u = (uint32_t)(synth_bits(stream_key, i) >> 32);
    uint32_t lo = 0, hi = n_bins - 1; // first index with table[idx] > u, clamped to n_bins-1
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (table[mid] > u) hi = mid; else lo = mid + 1;
    }
    return lo;
}
