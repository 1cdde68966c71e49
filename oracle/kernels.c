/* ORACLE - test infrastructure only. Plain-C restatement of the arithmetic on the
 * preemptible-queue path: the victim kernels, the seeded synthetic inputs and the
 * percentile rule. Nothing in the shipped libraries links or calls this file; it is
 * used by tests/, by the smoke check and by the CPU-baseline leg of bench.py.
 *
 * What pins each function (tests/test_oracle_kernels.py, CPU only; the known answers in
 * tests/golden/kernel_vectors.json were computed by tests/golden/make_kernel_vectors.py
 * with Python integers, fractions and decimals, not with this file):
 *   oracle_vecadd      c = a + b is one IEEE-754 operation per element: equal to numpy's
 *                      addition bit for bit, and the known-answer shape of the reference's
 *                      own test: k chained additions of ones give k
 *                      (platforms/example/test/src/vecadd.cpp:91-102).
 *   oracle_axpy        y = fma(alpha, x, y): one correctly rounded libm fmaf per element.
 *                      alpha = 0.5 (product exact): equal to numpy's multiply-then-add bit
 *                      for bit; five other alphas: equal to the exact rational
 *                      alpha * x + y rounded once (fixture), on inputs where
 *                      multiply-then-add gives different bits.
 *   oracle_gemm_bf16   triple loop, ascending k, fmaf accumulation, RNE to bf16. On
 *                      small-integer inputs (every partial sum exact) equal to integer
 *                      matmul; the summation order by a sum whose value depends on it
 *                      (2^24 + 63 ones); float64 matmul within the fp32 error bound;
 *                      oracle_f32_to_bf16 against ties, carries and the overflow to
 *                      infinity decided by exact distances (fixture).
 *   oracle_histogram   bins[key]++ ; equal to numpy.bincount, keys outside the range
 *                      ignored, bins not cleared, counters wrap modulo 2^32.
 *   oracle_percentile  sorted[floor(p*n)] - the reference's rule
 *                      (utils/include/xsched/utils/data.h:57-65); closed-form cases
 *                      (n = 1; n = 100, p = 0.99 -> index 99; p * n integral; ties).
 *   synthetic inputs   SplitMix64 against its published vector (seed 0: E220A8397B1DCDAF,
 *                      6E789E6AA1B965F4, 06C45D188009454F); stream keys, the first 16
 *                      uniform and normal values, the first 32 Zipf keys, the Zipf table
 *                      (60-digit decimals) and bins 0..15 of 2^22 keys against the
 *                      fixture; the table also against what the distribution fixes
 *                      (monotone, ends at 2^32 - 1, P(0) = 1 / H(65536, 1.1), increments
 *                      in the ratio (k + 1)^-1.1, 13.8 % of the keys in bin 0).
 * The reference has no GEMM, histogram or AXPY kernel: these three are new work
 * whose definition is the header include/xsched/hip/hal.h.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- kernels ------------------------------------------------------------------ */

void oracle_vecadd(const float *a, const float *b, float *c, size_t n)
{
    for (size_t i = 0; i < n; ++i) c[i] = a[i] + b[i];
}

void oracle_axpy(float alpha, const float *x, float *y, size_t n)
{
    for (size_t i = 0; i < n; ++i) y[i] = fmaf(alpha, x[i], y[i]);
}

static float bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7FFFu + lsb) >> 16);
}

/* C[M,N] = A[M,K] * B[K,N], row-major bf16 in/out, fp32 accumulation, k ascending.
 * c_f32 (optional) receives the unrounded fp32 accumulators. */
void oracle_gemm_bf16(const uint16_t *A, const uint16_t *B, uint16_t *C, float *c_f32,
                      int M, int N, int K)
{
    float *bt = (float *)malloc((size_t)K * N * sizeof(float)); /* B as float, transposed */
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) bt[(size_t)n * K + k] = bf16_to_f32(B[(size_t)k * N + n]);
    float *arow = (float *)malloc((size_t)K * sizeof(float));
    for (int m = 0; m < M; ++m) {
        for (int k = 0; k < K; ++k) arow[k] = bf16_to_f32(A[(size_t)m * K + k]);
        for (int n = 0; n < N; ++n) {
            const float *bcol = bt + (size_t)n * K;
            float acc = 0.f;
            for (int k = 0; k < K; ++k) acc = fmaf(arow[k], bcol[k], acc);
            if (c_f32) c_f32[(size_t)m * N + n] = acc;
            C[(size_t)m * N + n] = oracle_f32_to_bf16(acc);
        }
    }
    free(arow);
    free(bt);
}

/* bins[keys[i]] += 1; keys outside [0, n_bins) are ignored. Bins are not cleared. */
void oracle_histogram(const int32_t *keys, size_t n, uint32_t *bins, uint32_t n_bins)
{
    for (size_t i = 0; i < n; ++i) {
        uint32_t k = (uint32_t)keys[i];
        if (k < n_bins) bins[k] += 1;
    }
}

/* ---- percentile rule ------------------------------------------------------------ */

static int cmp_double(const void *a, const void *b)
{
    double x = *(const double *)a, y = *(const double *)b;
    return (x > y) - (x < y);
}

/* sorted[floor(p * n)]; sorts `data` in place. p must keep the index below n. */
double oracle_percentile(double *data, size_t n, double p)
{
    if (n == 0) return 0.0;
    qsort(data, n, sizeof(double), cmp_double);
    size_t idx = (size_t)(p * (double)n);
    if (idx >= n) idx = n - 1;
    return data[idx];
}

/* ---- seeded synthetic inputs ---------------------------------------------------
 * bits(seed, stream, i) = splitmix64(splitmix64(seed ^ stream * C) + i)            */

static uint64_t splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

uint64_t oracle_stream_key(uint64_t seed, uint64_t stream)
{
    return splitmix64(seed ^ (stream * 0xD1B54A32D192ED03ull));
}

/* raw 64 bits of a stream at index i */
uint64_t oracle_bits(uint64_t key, uint64_t i) { return splitmix64(key + i); }

/* uniform in [-1, 1): top 24 bits u -> u * 2^-23 - 1 */
void oracle_fill_uniform(float *dst, uint64_t first, uint64_t count, uint64_t key)
{
    for (uint64_t j = 0; j < count; ++j) {
        uint32_t u = (uint32_t)(splitmix64(key + first + j) >> 40);
        dst[j] = (float)u * (1.0f / 8388608.0f) - 1.0f;
    }
}

/* Irwin-Hall(12) approximation of N(0,1), rounded to bf16 */
void oracle_fill_normal_bf16(uint16_t *dst, uint64_t first, uint64_t count, uint64_t key)
{
    for (uint64_t j = 0; j < count; ++j) {
        uint64_t i = first + j;
        int64_t sum = 0;
        for (int k = 0; k < 6; ++k) {
            uint64_t b = splitmix64(key + i * 6 + (uint64_t)k);
            sum += (int64_t)(b >> 40) + (int64_t)((b >> 16) & 0xFFFFFFull);
        }
        sum -= 6ll * 16777216ll;
        dst[j] = oracle_f32_to_bf16((float)sum * (1.0f / 16777216.0f));
    }
}

/* table[k] = floor(2^32 * H(k+1) / H(n_bins)), H = generalised harmonic number of
 * exponent s, in long double; the last entry is forced to 2^32 - 1. */
void oracle_zipf_table(uint32_t *table, uint32_t n_bins, double s)
{
    long double *h = (long double *)malloc(sizeof(long double) * n_bins);
    long double acc = 0;
    for (uint32_t k = 0; k < n_bins; ++k) { acc += powl((long double)(k + 1), -(long double)s); h[k] = acc; }
    for (uint32_t k = 0; k < n_bins; ++k) {
        long double v = floorl(4294967296.0L * (h[k] / acc));
        table[k] = v >= 4294967295.0L ? 0xFFFFFFFFu : (uint32_t)v;
    }
    table[n_bins - 1] = 0xFFFFFFFFu;
    free(h);
}

/* key = first index whose table entry exceeds the 32-bit draw (clamped) */
void oracle_fill_zipf(int32_t *dst, uint64_t first, uint64_t count, uint64_t key,
                      const uint32_t *table, uint32_t n_bins)
{
    for (uint64_t j = 0; j < count; ++j) {
        uint32_t u = (uint32_t)(splitmix64(key + first + j) >> 32);
        uint32_t lo = 0, hi = n_bins - 1;
        while (lo < hi) {
            uint32_t mid = (lo + hi) >> 1;
            if (table[mid] > u) hi = mid; else lo = mid + 1;
        }
        dst[j] = (int32_t)lo;
    }
}
