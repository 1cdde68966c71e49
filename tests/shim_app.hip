// A plain HIP program that knows nothing of XSched: the interception shim's test subject.
// It is built twice from this file, once linked against libshimhip.so (shim_app) and once
// not (shim_app_plain). Both print one line per check; the lines must be equal, and equal
// to the values computed on the host below.
//
//   shim_app [module.co]          the checks (module checks only if a code object is given)
//   shim_app --bench N            N launches of a tiny kernel on one stream, us per launch
//   shim_app --bench-paced N GAP_US  N launches with GAP_US of host work between them: cost of the launch call
//   shim_app --load SECONDS       device-filling kernels back to back on one stream
//   shim_app --probe N PERIOD_US  a short kernel every PERIOD_US, launch-to-completion latency
//   shim_app --leak               leaves main() with streams, events and memory never released
//   shim_app --load-guarded SECONDS [SPLIT]  like --load with a kernel that has the XSched guard compiled in
//                                 (SPLIT times as many work-groups, each that much shorter)
//
// The guard (xsched/hip/guard.h) is the one thing here that belongs to XSched: a kernel with
// an XGuardArgs as its last parameter. The program launches it like any other kernel and
// passes zeroes, which switch the guard off; with the shim in front, the queue supplies the
// real arguments and the launch can be flushed and replayed at level 2.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "xsched/hip/guard.h"

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#define CHECK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { \
    fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); exit(2); } } while (0)

struct Pair { float a; double b; char c; };          // 24 bytes with padding
struct Wide { uint32_t v[50]; };                      // 200 bytes by value

__device__ uint32_t g_counter;

__global__ void Saxpy(float a, const float *x, float *y, size_t n)
{
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (i < n) y[i] = a * x[i] + y[i];
}

__global__ void Mixed(Pair p, short s, unsigned char u, double *out, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = p.a + p.b + p.c + s + u + i;
}

__global__ void SumWide(Wide w, uint32_t *out)
{
    uint32_t sum = 0;
    for (int i = 0; i < 50; ++i) sum += w.v[i] * (uint32_t)(i + 1);
    out[threadIdx.x] = sum + threadIdx.x;
}

__global__ void Bump() { if (threadIdx.x == 0 && blockIdx.x == 0) g_counter += 1; }

__global__ void ReadCounter(uint32_t *out) { out[0] = g_counter; }

__global__ void AddInto(uint32_t *dst, const uint32_t *src, uint32_t k, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] += src[i] + k;
}

// Long enough that work queued behind it is still pending when the host moves on.
__global__ void Spin(uint32_t *out, uint32_t iters)
{
    uint32_t v = threadIdx.x;
    for (uint32_t i = 0; i < iters; ++i) v = v * 1664525u + 1013904223u;
    out[threadIdx.x] = v;
}

// Spins for a while (milliseconds at `iters` in the millions), then stores `value` where the
// host reads it directly.
__global__ void SpinThenStore(volatile uint32_t *host_word, uint32_t iters, uint32_t value)
{
    uint32_t v = threadIdx.x;
    for (uint32_t i = 0; i < iters; ++i) v = v * 1664525u + 1013904223u;
    if (threadIdx.x == 0) *host_word = v == 0x12345u ? value + 1 : value;
}

static uint64_t Fnv(const void *data, size_t bytes)
{
    const uint8_t *p = (const uint8_t *)data;
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < bytes; ++i) { h ^= p[i]; h *= 1099511628211ull; }
    return h;
}

static void Report(const char *what, uint64_t got, uint64_t want)
{
    printf("%-28s %016llx %s\n", what, (unsigned long long)got, got == want ? "ok" : "MISMATCH");
}

static void HostFn(void *data) { *(volatile uint32_t *)data = 77; }
static void Callback(hipStream_t, hipError_t, void *data) { *(volatile uint32_t *)data += 1; }

static int Bench(int launches)
{
    hipStream_t s;
    CHECK(hipStreamCreate(&s));
    for (int i = 0; i < 200; ++i) Bump<<<1, 64, 0, s>>>();
    CHECK(hipStreamSynchronize(s));
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < launches; ++i) Bump<<<1, 64, 0, s>>>();
    const auto t1 = std::chrono::steady_clock::now();
    CHECK(hipStreamSynchronize(s));
    const auto t2 = std::chrono::steady_clock::now();
    const double submit = std::chrono::duration<double, std::micro>(t1 - t0).count() / launches;
    const double total = std::chrono::duration<double, std::micro>(t2 - t0).count() / launches;
    printf("bench launches=%d submit_us_per_launch=%.3f total_us_per_launch=%.3f\n", launches, submit, total);
    CHECK(hipStreamDestroy(s));
    return 0;
}

// The same launches with `gap_us` of host work between them, the way a framework issues
// kernels: what is timed is the launch call itself.
static int BenchPaced(int launches, int gap_us)
{
    hipStream_t s;
    CHECK(hipStreamCreate(&s));
    for (int i = 0; i < 200; ++i) Bump<<<1, 64, 0, s>>>();
    CHECK(hipStreamSynchronize(s));
    std::vector<double> cost((size_t)launches);
    using Clock = std::chrono::steady_clock;
    for (int i = 0; i < launches; ++i) {
        const auto t0 = Clock::now();
        Bump<<<1, 64, 0, s>>>();
        const auto t1 = Clock::now();
        cost[(size_t)i] = std::chrono::duration<double, std::micro>(t1 - t0).count();
        while (Clock::now() < t1 + std::chrono::microseconds(gap_us)) {}
    }
    CHECK(hipStreamSynchronize(s));
    std::sort(cost.begin(), cost.end());
    double sum = 0;
    for (double c : cost) sum += c;
    printf("bench-paced launches=%d gap_us=%d call_us_mean=%.3f p50=%.3f p99=%.3f\n", launches, gap_us, sum / launches,
           cost[cost.size() / 2], cost[cost.size() * 99 / 100]);
    CHECK(hipStreamDestroy(s));
    return 0;
}

// Every thread runs `iters` dependent steps: with 2048 x 256 threads (all resident at once)
// the device is full for about a millisecond at 30000 steps.
__global__ void Busy(uint32_t *out, uint32_t iters)
{
    uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
    for (uint32_t i = 0; i < iters; ++i) v = v * 1664525u + 1013904223u;
    if (v == 0x12345678u) out[0] = v; // keeps the loop; practically never true
}

// The guarded load: every work-group spins like Busy, looks at the preempt word every 256
// steps (about every 14 us) (and leaves without a trace when the queue has been deactivated), and counts itself in
// `runs` at the end: a work-group that took effect twice, or never, shows there.
__global__ __launch_bounds__(256)
void BusyGuarded(uint32_t *runs, uint32_t iters, XGuardArgs g)
{
    __shared__ uint32_t guard_word;
    XGuardBlock guard(g, blockIdx.x, &guard_word);
    if (!guard.Enter()) return;
    uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
    for (uint32_t done = 0; done < iters; done += 256) {
        // (not an affine map like Busy's: the compiler would fold the fixed number of steps into one)
        for (uint32_t i = 0; i < 256; ++i) v = (v ^ (v >> 13)) * 1664525u + 1013904223u;
        if (!guard.StillCurrent()) return;
    }
    if (threadIdx.x == 0) runs[blockIdx.x] += 1 + (v == 0x12345678u);
    guard.Commit();
}

// In place and not idempotent, for the checks: y = 0.5 * y + b over 1024 elements per work-group.
__global__ __launch_bounds__(256)
void AffineGuarded(float *y, float b, uint32_t n, XGuardArgs g)
{
    __shared__ uint32_t guard_word;
    XGuardBlock guard(g, blockIdx.x, &guard_word);
    if (!guard.Enter()) return;
    for (uint32_t i = blockIdx.x * 1024 + threadIdx.x; i < (blockIdx.x + 1) * 1024 && i < n; i += 256) {
        y[i] = __builtin_fmaf(0.5f, y[i], b);
    }
    guard.Commit();
}

// `split` > 1 cuts the same work into `split` times as many work-groups, each that much
// shorter: what a flush throws away is the progress of the work-groups that were running.
static int LoadGuarded(double seconds, uint32_t split)
{
    hipStream_t s;
    uint32_t *runs;
    const uint32_t kGroups = 2048 * split;
    CHECK(hipStreamCreate(&s));
    CHECK(hipMalloc(&runs, kGroups * 4));
    CHECK(hipMemset(runs, 0, kGroups * 4));
    printf("ready\n"); fflush(stdout);
    const auto t0 = std::chrono::steady_clock::now();
    uint32_t kernels = 0;
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) {
        for (int i = 0; i < 8; ++i) BusyGuarded<<<kGroups, 256, 0, s>>>(runs, 92160 / split, XGuardArgs {});   // about 5 ms: long enough that waiting for its end hurts
        CHECK(hipStreamSynchronize(s));
        kernels += 8;
    }
    const double elapsed = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::vector<uint32_t> host(kGroups);
    CHECK(hipMemcpy(host.data(), runs, kGroups * 4, hipMemcpyDeviceToHost));
    uint32_t wrong = 0;
    for (uint32_t w = 0; w < kGroups; ++w) wrong += host[w] != kernels;
    printf("load kernels=%u ms_per_kernel=%.3f work_groups_not_exactly_once=%u\n", kernels, elapsed * 1e3 / kernels, wrong);
    CHECK(hipFree(runs));
    CHECK(hipStreamDestroy(s));
    return wrong == 0 ? 0 : 4;
}

static int Load(double seconds)
{
    hipStream_t s;
    uint32_t *out;
    CHECK(hipStreamCreate(&s));
    CHECK(hipMalloc(&out, 4));
    printf("ready\n"); fflush(stdout);
    const auto t0 = std::chrono::steady_clock::now();
    uint64_t kernels = 0;
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) {
        for (int i = 0; i < 32; ++i) Busy<<<2048, 256, 0, s>>>(out, 30000);
        CHECK(hipStreamSynchronize(s));
        kernels += 32;
    }
    const double elapsed = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    printf("load kernels=%llu ms_per_kernel=%.3f\n", (unsigned long long)kernels, elapsed * 1e3 / kernels);
    CHECK(hipFree(out));
    CHECK(hipStreamDestroy(s));
    return 0;
}

static int Probe(int count, int period_us)
{
    hipStream_t s;
    uint32_t *out;
    CHECK(hipStreamCreate(&s));
    CHECK(hipMalloc(&out, 4));
    for (int i = 0; i < 20; ++i) Busy<<<256, 256, 0, s>>>(out, 5000);
    CHECK(hipStreamSynchronize(s));
    printf("ready\n"); fflush(stdout);
    std::vector<double> us(count), launch_us(count);
    for (int i = 0; i < count; ++i) {
        const auto t0 = std::chrono::steady_clock::now();
        Busy<<<256, 256, 0, s>>>(out, 5000);
        const auto t1 = std::chrono::steady_clock::now();
        CHECK(hipStreamSynchronize(s));
        us[i] = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
        launch_us[i] = std::chrono::duration<double, std::micro>(t1 - t0).count();
        std::this_thread::sleep_for(std::chrono::microseconds(period_us));
    }
    if (const char *dump = getenv("SHIM_APP_PROBE_DUMP")) {   // every sample in arrival order (total, of which the launch call), for a closer look at the tail
        if (FILE *f = fopen(dump, "w")) {
            for (int i = 0; i < count; ++i) fprintf(f, "%.1f %.1f\n", us[i], launch_us[i]);
            fclose(f);
        }
    }
    std::sort(us.begin(), us.end());
    // percentile p = sorted[floor(p * n)]
    printf("probe n=%d p50_us=%.1f p99_us=%.1f max_us=%.1f p90_us=%.1f p95_us=%.1f\n", count, us[(size_t)(0.5 * count)],
           us[(size_t)(0.99 * count)], us.back(), us[(size_t)(0.9 * count)], us[(size_t)(0.95 * count)]);
    CHECK(hipFree(out));
    CHECK(hipStreamDestroy(s));
    return 0;
}

// What many programs do: nothing is destroyed, the last work is synchronised by an event only.
static int Leak()
{
    hipStream_t s[2];
    hipEvent_t done;
    uint32_t *out, host = 0;
    CHECK(hipStreamCreate(&s[0])); CHECK(hipStreamCreateWithFlags(&s[1], hipStreamNonBlocking));
    CHECK(hipEventCreate(&done));
    CHECK(hipMalloc(&out, 4));
    uint32_t zero = 0;
    CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_counter), &zero, 4));
    for (int i = 0; i < 100; ++i) Bump<<<1, 64, 0, s[0]>>>();
    ReadCounter<<<1, 1, 0, s[0]>>>(out);
    CHECK(hipEventRecord(done, s[0]));
    Busy<<<64, 256, 0, s[1]>>>(out + 0, 1000);   // never waited for
    CHECK(hipEventSynchronize(done));
    CHECK(hipMemcpy(&host, out, 4, hipMemcpyDeviceToHost));
    printf("leak counter=%u\n", host);
    return host == 100 ? 0 : 3;
}

int main(int argc, char **argv)
{
    if (argc >= 2 && strcmp(argv[1], "--leak") == 0) return Leak();
    if (argc >= 3 && strcmp(argv[1], "--bench") == 0) return Bench(atoi(argv[2]));
    if (argc >= 4 && strcmp(argv[1], "--bench-paced") == 0) return BenchPaced(atoi(argv[2]), atoi(argv[3]));
    if (argc >= 3 && strcmp(argv[1], "--load") == 0) return Load(atof(argv[2]));
    if (argc >= 3 && strcmp(argv[1], "--load-guarded") == 0) return LoadGuarded(atof(argv[2]), argc >= 4 ? (uint32_t)atoi(argv[3]) : 1u);
    if (argc >= 4 && strcmp(argv[1], "--probe") == 0) return Probe(atoi(argv[2]), atoi(argv[3]));
    const char *module_path = argc >= 2 ? argv[1] : nullptr;
    // Under the kernel-trace profiler the program without any library of this repository in it
    // ends in a segmentation fault inside the exit handlers once it has used stream-ordered
    // allocation; a profile run passes this switch and leaves section 7d out.
    const bool skip_ordered_only = argc >= 3 && strcmp(argv[2], "--skip-ordered-only") == 0;

    constexpr size_t n = 1 << 16;
    hipStream_t s1, s2, s3;
    CHECK(hipStreamCreate(&s1));
    CHECK(hipStreamCreateWithFlags(&s2, hipStreamNonBlocking));
    CHECK(hipStreamCreateWithPriority(&s3, hipStreamDefault, 0));

    // ---- 1. fills of every width, copies from pinned and pageable memory, a kernel chain ----
    float *x, *y;
    CHECK(hipMalloc(&x, n * 4)); CHECK(hipMalloc(&y, n * 4));
    float *pinned, *pinned_out;
    CHECK(hipHostMalloc(&pinned, n * 4, hipHostMallocDefault));
    CHECK(hipHostMalloc(&pinned_out, n * 4, hipHostMallocDefault));
    std::vector<float> pageable(n), want(n);
    for (size_t i = 0; i < n; ++i) { pinned[i] = (float)(i % 97) * 0.5f; pageable[i] = (float)(i % 13); }
    CHECK(hipMemcpyAsync(x, pinned, n * 4, hipMemcpyHostToDevice, s1));
    CHECK(hipMemcpyAsync(y, pageable.data(), n * 4, hipMemcpyHostToDevice, s1));
    for (size_t i = 0; i < n; ++i) want[i] = pageable[i];
    for (int rep = 0; rep < 3; ++rep) {
        Saxpy<<<(n + 255) / 256, 256, 0, s1>>>(2.0f, x, y, n);
        for (size_t i = 0; i < n; ++i) want[i] = 2.0f * pinned[i] + want[i];
    }
    CHECK(hipMemcpyAsync(pinned_out, y, n * 4, hipMemcpyDeviceToHost, s1));
    CHECK(hipStreamSynchronize(s1));
    Report("saxpy chain", Fnv(pinned_out, n * 4), Fnv(want.data(), n * 4));

    uint8_t *fills;
    CHECK(hipMalloc(&fills, 4096));
    CHECK(hipMemsetAsync(fills, 0xAB, 1024, s1));
    CHECK(hipMemsetD8Async((hipDeviceptr_t)(fills + 1024), 0x5C, 1024, s1));
    CHECK(hipMemsetD16Async((hipDeviceptr_t)(fills + 2048), 0xBEEF, 512, s1));
    CHECK(hipMemsetD32Async((hipDeviceptr_t)(fills + 3072), (int)0xDEADC0DE, 256, s1));
    std::vector<uint8_t> fills_host(4096), fills_want(4096);
    CHECK(hipMemcpyAsync(fills_host.data(), fills, 4096, hipMemcpyDeviceToHost, s1)); // pageable destination
    memset(fills_want.data(), 0xAB, 1024); memset(fills_want.data() + 1024, 0x5C, 1024);
    for (int i = 0; i < 512; ++i) { const uint16_t v = 0xBEEF; memcpy(&fills_want[2048 + 2 * i], &v, 2); }
    for (int i = 0; i < 256; ++i) { const uint32_t v = 0xDEADC0DE; memcpy(&fills_want[3072 + 4 * i], &v, 4); }
    CHECK(hipStreamSynchronize(s1));
    Report("fills 8/16/32", Fnv(fills_host.data(), 4096), Fnv(fills_want.data(), 4096));

    // ---- 2. arguments of every shape ----------------------------------------------------------
    double *mixed_out; uint32_t *wide_out;
    CHECK(hipMalloc(&mixed_out, 512 * 8)); CHECK(hipMalloc(&wide_out, 64 * 4));
    {
        Pair p { 1.5f, -2.25, 7 };
        Wide w;
        for (int i = 0; i < 50; ++i) w.v[i] = 1000u + 17u * i;
        Mixed<<<2, 256, 0, s2>>>(p, (short)-300, (unsigned char)200, mixed_out, 512);
        SumWide<<<1, 64, 0, s2>>>(w, wide_out);
        p.a = 0; memset(&w, 0, sizeof w); // the launches must have taken copies
    }
    std::vector<double> mixed_host(512), mixed_want(512);
    std::vector<uint32_t> wide_host(64), wide_want(64);
    CHECK(hipMemcpyDtoHAsync(mixed_host.data(), (hipDeviceptr_t)mixed_out, 512 * 8, s2));
    CHECK(hipMemcpyDtoHAsync(wide_host.data(), (hipDeviceptr_t)wide_out, 64 * 4, s2));
    CHECK(hipStreamSynchronize(s2));
    for (int i = 0; i < 512; ++i) mixed_want[i] = 1.5f + -2.25 + 7 + -300 + 200 + i;
    uint32_t wsum = 0;
    for (int i = 0; i < 50; ++i) wsum += (1000u + 17u * i) * (uint32_t)(i + 1);
    for (int i = 0; i < 64; ++i) wide_want[i] = wsum + i;
    Report("struct and small scalars", Fnv(mixed_host.data(), 512 * 8), Fnv(mixed_want.data(), 512 * 8));
    Report("200-byte struct by value", Fnv(wide_host.data(), 64 * 4), Fnv(wide_want.data(), 64 * 4));

    // ---- 3. a kernel without arguments, in order with its neighbours --------------------------
    uint32_t *counter_out, counter_host = 0, zero = 0;
    CHECK(hipMalloc(&counter_out, 4));
    CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_counter), &zero, 4));
    for (int i = 0; i < 300; ++i) Bump<<<1, 64, 0, s3>>>();
    ReadCounter<<<1, 1, 0, s3>>>(counter_out);
    CHECK(hipMemcpyAsync(&counter_host, counter_out, 4, hipMemcpyDeviceToHost, s3));
    CHECK(hipStreamSynchronize(s3));
    Report("300 argument-less launches", counter_host, 300);

    // ---- 4. events across streams -------------------------------------------------------------
    uint32_t *a, *b, *spin;
    CHECK(hipMalloc(&a, n * 4)); CHECK(hipMalloc(&b, n * 4)); CHECK(hipMalloc(&spin, 256 * 4));
    CHECK(hipMemsetD32Async((hipDeviceptr_t)a, 5, n, s1));
    CHECK(hipMemsetD32Async((hipDeviceptr_t)b, 1, n, s2));
    CHECK(hipStreamSynchronize(s1)); CHECK(hipStreamSynchronize(s2));
    hipEvent_t start, produced, stop;
    CHECK(hipEventCreate(&start)); CHECK(hipEventCreate(&produced)); CHECK(hipEventCreate(&stop));
    CHECK(hipEventRecord(start, s1));
    Spin<<<1, 256, 0, s1>>>(spin, 2000000);                   // a few milliseconds
    AddInto<<<n / 256, 256, 0, s1>>>(a, b, 10, n);            // a = 5 + 1 + 10 = 16
    CHECK(hipEventRecord(produced, s1));
    CHECK(hipStreamWaitEvent(s2, produced, 0));
    AddInto<<<n / 256, 256, 0, s2>>>(b, a, 100, n);           // b = 1 + 16 + 100 = 117, only after s1
    CHECK(hipEventRecord(stop, s2));
    const hipError_t early = hipEventQuery(stop);
    CHECK(hipEventSynchronize(stop));
    float ms = -1.f;
    CHECK(hipEventElapsedTime(&ms, start, stop));
    std::vector<uint32_t> b_host(n);
    CHECK(hipMemcpy(b_host.data(), b, n * 4, hipMemcpyDeviceToHost));
    uint64_t bad = 0;
    for (size_t i = 0; i < n; ++i) bad += b_host[i] != 117;
    Report("cross-stream event order", bad, 0);
    Report("event query before/after", (uint64_t)(early == hipErrorNotReady || early == hipSuccess) + 2 * (hipEventQuery(stop) == hipSuccess), 3);
    Report("elapsed time is positive", ms > 0.5f, 1);

    // ---- 5. null-stream work waits for blocking streams ---------------------------------------
    CHECK(hipMemsetD32Async((hipDeviceptr_t)a, 0, n, s1));
    Spin<<<1, 256, 0, s1>>>(spin, 1000000);
    AddInto<<<n / 256, 256, 0, s1>>>(a, b, 3, n);             // a = 0 + 117 + 3 = 120
    AddInto<<<n / 256, 256>>>(a, a, 0, n);                    // null stream: a = 240, after s1
    std::vector<uint32_t> a_host(n);
    CHECK(hipMemcpy(a_host.data(), a, n * 4, hipMemcpyDeviceToHost));
    bad = 0;
    for (size_t i = 0; i < n; ++i) bad += a_host[i] != 240;
    Report("null stream after stream", bad, 0);

    // ---- 6. host functions, stream queries, free behind queued work ----------------------------
    volatile uint32_t host_word = 0, callback_word = 0;
    Spin<<<1, 256, 0, s3>>>(spin, 1000000);
    CHECK(hipLaunchHostFunc(s3, HostFn, (void *)&host_word));
    CHECK(hipStreamAddCallback(s3, Callback, (void *)&callback_word, 0));
    while (hipStreamQuery(s3) == hipErrorNotReady) std::this_thread::yield();
    CHECK(hipStreamSynchronize(s3));
    Report("host function and callback", host_word + callback_word, 78);
    uint32_t *temp;
    CHECK(hipMalloc(&temp, n * 4));
    CHECK(hipMemsetD32Async((hipDeviceptr_t)temp, 9, n, s1));
    Spin<<<1, 256, 0, s1>>>(spin, 500000);
    AddInto<<<n / 256, 256, 0, s1>>>(a, temp, 0, n);          // a = 240 + 9 = 249
    CHECK(hipFree(temp));                                     // must not pull the memory from under the kernel
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(a_host.data(), a, n * 4, hipMemcpyDeviceToHost));
    bad = 0;
    for (size_t i = 0; i < n; ++i) bad += a_host[i] != 249;
    Report("free behind queued work", bad, 0);

    // ---- 7. two threads, each with its own stream ------------------------------------------------
    {
        uint32_t *acc[2], *ones;
        CHECK(hipMalloc(&ones, 1024 * 4));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)ones, 1, 1024, s1));
        CHECK(hipStreamSynchronize(s1));
        hipStream_t ts[2] = { s1, s2 };
        std::thread th[2];
        for (int t = 0; t < 2; ++t) {
            CHECK(hipMalloc(&acc[t], 1024 * 4));
            CHECK(hipMemset(acc[t], 0, 1024 * 4));
            th[t] = std::thread([&, t]() {
                for (uint32_t i = 0; i < 400; ++i) AddInto<<<4, 256, 0, ts[t]>>>(acc[t], ones, i * (t + 1), 1024);
                CHECK(hipStreamSynchronize(ts[t]));
            });
        }
        uint64_t sums = 0;
        for (int t = 0; t < 2; ++t) {
            th[t].join();
            uint32_t first = 0;
            CHECK(hipMemcpy(&first, acc[t] + 1023, 4, hipMemcpyDeviceToHost));
            sums = sums * 1000003u + first;
        }
        // thread t: sum over i of (1 + i * (t + 1)) = 400 + (t + 1) * 79800
        Report("two threads, two streams", sums, (uint64_t)(400 + 79800) * 1000003u + (400 + 2 * 79800));
        CHECK(hipFree(acc[0])); CHECK(hipFree(acc[1])); CHECK(hipFree(ones));
    }

    // ---- 7c. a kernel with the XSched guard compiled in, launched like any other ----------------
    {
        constexpr uint32_t gn = 100000;
        float *gy;
        std::vector<float> gy_host(gn), gy_want(gn);
        for (uint32_t i = 0; i < gn; ++i) gy_want[i] = gy_host[i] = (float)(i % 251) * 0.25f;
        CHECK(hipMalloc(&gy, gn * 4));
        CHECK(hipMemcpy(gy, gy_host.data(), gn * 4, hipMemcpyHostToDevice));
        for (int rep = 0; rep < 50; ++rep) {
            AffineGuarded<<<(gn + 1023) / 1024, 256, 0, s2>>>(gy, 1.0f + rep, gn, XGuardArgs {});
            for (uint32_t i = 0; i < gn; ++i) gy_want[i] = 0.5f * gy_want[i] + (1.0f + rep);
        }
        CHECK(hipStreamSynchronize(s2));
        CHECK(hipMemcpy(gy_host.data(), gy, gn * 4, hipMemcpyDeviceToHost));
        Report("guarded kernel, 50 launches", Fnv(gy_host.data(), gn * 4), Fnv(gy_want.data(), gn * 4));
        CHECK(hipFree(gy));
    }

    // ---- 7a. a launch the runtime refuses is refused the same way ------------------------------
    {
        void *args[] = { &spin, &zero };
        const hipError_t too_wide = hipLaunchKernel((const void *)Spin, dim3(1), dim3(2048), args, 0, s1);
        (void)hipGetLastError();
        const hipError_t no_grid = hipLaunchKernel((const void *)Spin, dim3(0), dim3(64), args, 0, s1);
        (void)hipGetLastError();
        CHECK(hipStreamSynchronize(s1));
        Report("refused launches", (uint64_t)too_wide * 1000 + (uint64_t)no_grid, (uint64_t)too_wide * 1000 + (uint64_t)no_grid);
        printf("    error codes %d %d\n", (int)too_wide, (int)no_grid);
    }

    // ---- 7b. a graph captured from a stream and launched between ordinary launches --------------
    {
        uint32_t *gbuf, *gone;
        CHECK(hipMalloc(&gbuf, 1024 * 4)); CHECK(hipMalloc(&gone, 1024 * 4));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)gbuf, 0, 1024, s1));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)gone, 1, 1024, s1));
        AddInto<<<4, 256, 0, s1>>>(gbuf, gone, 1, 1024);                  // 2, still queued when the capture begins
        hipGraph_t graph;
        hipGraphExec_t exec;
        // Another stream is busy during the capture: whoever waits for its work on the program's
        // behalf must not disturb a capture in the default (global) mode.
        for (int i = 0; i < 40; ++i) Spin<<<1, 256, 0, s3>>>(spin, 20000);
        CHECK(hipStreamBeginCapture(s1, hipStreamCaptureModeGlobal));
        for (int i = 0; i < 3; ++i) AddInto<<<4, 256, 0, s1>>>(gbuf, gone, 9, 1024);   // + 30 per launch of the graph
        std::this_thread::sleep_for(std::chrono::milliseconds(2));
        CHECK(hipStreamEndCapture(s1, &graph));
        CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        CHECK(hipGraphLaunch(exec, s1));                                  // 32
        AddInto<<<4, 256, 0, s1>>>(gbuf, gbuf, 0, 1024);                  // 64, must follow the graph
        CHECK(hipGraphLaunch(exec, s1));                                  // 94, must follow the kernel
        std::vector<uint32_t> g_host(1024);
        CHECK(hipMemcpyAsync(g_host.data(), gbuf, 1024 * 4, hipMemcpyDeviceToHost, s1));
        CHECK(hipStreamSynchronize(s1));
        bad = 0;
        for (int i = 0; i < 1024; ++i) bad += g_host[i] != 94;
        Report("captured graph in order", bad, 0);
        CHECK(hipGraphExecDestroy(exec)); CHECK(hipGraphDestroy(graph));
        CHECK(hipFree(gbuf)); CHECK(hipFree(gone));
    }

    // ---- 7d. the calls that are ordered but not deferred, between calls that are deferred ----------
    if (!skip_ordered_only) {
        constexpr uint32_t rows = 64, cols = 256;                      // a 64 x 256 matrix of uint32_t
        uint32_t *m0, *m1, *pool_buf = nullptr;
        CHECK(hipMalloc(&m0, rows * cols * 4)); CHECK(hipMalloc(&m1, rows * cols * 4));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)m0, 2, rows * cols, s1));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)m1, 0, rows * cols, s1));
        AddInto<<<rows * cols / 256, 256, 0, s1>>>(m0, m0, 1, rows * cols);                    // m0 = 5
        CHECK(hipMemcpy2DAsync(m1, cols * 4, m0, cols * 4, cols * 2, rows, hipMemcpyDeviceToDevice, s1)); // left half of m1 = 5
        AddInto<<<rows * cols / 256, 256, 0, s1>>>(m1, m0, 0, rows * cols);                    // m1 = 10 | 5
        CHECK(hipMallocAsync((void **)&pool_buf, rows * cols * 4, s1));
        CHECK(hipMemcpyAsync(pool_buf, m1, rows * cols * 4, hipMemcpyDeviceToDevice, s1));
        void *coop_args[] = { &pool_buf, &m0, &zero, &zero };
        uint32_t count = rows * cols;
        coop_args[3] = &count;
        CHECK(hipLaunchCooperativeKernel((const void *)AddInto, dim3(rows * cols / 256), dim3(256), coop_args, 0, s1)); // + 5
        CHECK(hipExtLaunchKernel((const void *)AddInto, dim3(rows * cols / 256), dim3(256), coop_args, 0, s1, nullptr, nullptr, 0)); // + 5
        AddInto<<<rows * cols / 256, 256, 0, s1>>>(m1, pool_buf, 0, rows * cols);              // m1 += pool_buf
        CHECK(hipFreeAsync(pool_buf, s1));
        std::vector<uint32_t> m_host(rows * cols);
        CHECK(hipMemcpyDtoH(m_host.data(), (hipDeviceptr_t)m1, rows * cols * 4));               // null stream, after s1
        bad = 0;
        for (uint32_t r = 0; r < rows; ++r) {
            for (uint32_t c = 0; c < cols; ++c) bad += m_host[r * cols + c] != (c < cols / 2 ? 10u + 20u : 5u + 15u);
        }
        Report("ordered, not deferred calls", bad, 0);
        CHECK(hipFree(m0)); CHECK(hipFree(m1));
    }

    // ---- 7e. hipStreamSynchronize covers work that reached the stream outside the XQueue ---------
    // A launch the shim only orders (it goes to the runtime after a drain) of a kernel that runs
    // for milliseconds and then writes pinned memory; the host reads that memory right after
    // hipStreamSynchronize, with no copy or other command in between.
    {
        uint32_t *word;
        CHECK(hipHostMalloc((void **)&word, 64, hipHostMallocDefault));
        bad = 0;
        for (uint32_t round = 1; round <= 3; ++round) {
            *(volatile uint32_t *)word = 0;
            uint32_t iters = 4000000, value = 1000 + round;
            void *spin_args[] = { &word, &iters, &value };
            CHECK(hipExtLaunchKernel((const void *)SpinThenStore, dim3(1), dim3(64), spin_args, 0, s1, nullptr, nullptr, 0));
            CHECK(hipStreamSynchronize(s1));
            bad += *(volatile uint32_t *)word != value;
        }
        Report("sync after direct launch", bad, 0);
        CHECK(hipHostFree(word));
    }

    // ---- 8. kernels of a loaded module ------------------------------------------------------------
    if (module_path != nullptr) {
        hipModule_t mod;
        hipFunction_t scale, shift;
        CHECK(hipModuleLoad(&mod, module_path));
        CHECK(hipModuleGetFunction(&scale, mod, "ModScale"));
        CHECK(hipModuleGetFunction(&shift, mod, "ModShift"));
        uint32_t *m;
        CHECK(hipMalloc(&m, 1024 * 4));
        CHECK(hipMemsetD32Async((hipDeviceptr_t)m, 3, 1024, s1));
        uint32_t factor = 7, count = 1024;
        unsigned short add = 11;
        void *params[] = { &m, &factor, &count };
        CHECK(hipModuleLaunchKernel(scale, 4, 1, 1, 256, 1, 1, 0, s1, params, nullptr));   // 3 * 7 = 21
        factor = 0;                                                                          // a copy was taken
        struct { uint32_t *ptr; unsigned short add; uint32_t count; } packed { m, add, count };
        size_t packed_bytes = sizeof packed;
        void *extra[] = { HIP_LAUNCH_PARAM_BUFFER_POINTER, &packed, HIP_LAUNCH_PARAM_BUFFER_SIZE, &packed_bytes, HIP_LAUNCH_PARAM_END };
        CHECK(hipModuleLaunchKernel(shift, 4, 1, 1, 256, 1, 1, 0, s1, nullptr, extra));     // 21 + 11 = 32
        factor = 2;
        void *params2[] = { &m, &factor, &count };
        CHECK(hipExtModuleLaunchKernel(scale, 1024, 1, 1, 256, 1, 1, 0, s1, params2, nullptr, nullptr, nullptr, 0)); // 64
        std::vector<uint32_t> m_host(1024);
        CHECK(hipMemcpyAsync(m_host.data(), m, 1024 * 4, hipMemcpyDeviceToHost, s1));
        CHECK(hipStreamSynchronize(s1));
        bad = 0;
        for (int i = 0; i < 1024; ++i) bad += m_host[i] != 64;
        Report("module kernels", bad, 0);
        CHECK(hipFree(m));
        CHECK(hipModuleUnload(mod));
    }

    CHECK(hipEventDestroy(start)); CHECK(hipEventDestroy(produced)); CHECK(hipEventDestroy(stop));
    CHECK(hipStreamDestroy(s1)); CHECK(hipStreamDestroy(s2)); CHECK(hipStreamDestroy(s3));
    CHECK(hipFree(x)); CHECK(hipFree(y)); CHECK(hipFree(fills)); CHECK(hipFree(mixed_out)); CHECK(hipFree(wide_out));
    CHECK(hipFree(counter_out)); CHECK(hipFree(a)); CHECK(hipFree(b)); CHECK(hipFree(spin));
    CHECK(hipHostFree(pinned)); CHECK(hipHostFree(pinned_out));
    printf("done\n");
    return 0;
}
