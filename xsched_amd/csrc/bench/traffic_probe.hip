// Small driver for hardware-counter runs: launches a plain copy kernel of known size
// (1 GiB read + 1 GiB written) and then a victim kernel through an XQueue, a few times:
//   traffic_probe [n] [reps]          AXPY of n elements in its three forms (plain, guarded at
//                                     level 1, guarded at level 2)
//   traffic_probe [n] [reps] hist     histogram of 2^26 Zipf keys, plain and guarded at level 2
//   traffic_probe [n] [reps] gemm     bf16 GEMM 8192^3, plain and guarded at level 2
//   traffic_probe [n] [reps] gemmk K  plain bf16 GEMM 8192 x 8192 x K (random bf16 inputs of about
//                                     unit variance): the same 1024 tiles with a loop K / 64 steps
//                                     long, prints the time per launch (how much of a launch is
//                                     per-tile fixed cost)
// Run it under `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`: the copy kernel's
// counters give the scale factor of the counter, the other rows the kernels' real HBM
// traffic per launch.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <hip/hip_runtime.h>

#include "xsched/hip/bench.h"
#include "xsched/hip/hal.h"
#include "xsched/xsched.h"

#define CHECK_HIP(e) do { hipError_t r_ = (e); if (r_ != hipSuccess) { \
    fprintf(stderr, "HIP error %s at %s\n", hipGetErrorString(r_), #e); exit(1); } } while (0)
#define CHECK_X(e) do { XResult r_ = (e); if (r_ != kXSchedSuccess) { \
    fprintf(stderr, "XSched error %d at %s\n", (int)r_, #e); exit(1); } } while (0)

typedef float f4 __attribute__((ext_vector_type(4)));

__global__ void PlainCopyKernel(const f4 *src, f4 *dst, size_t n4)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        dst[i] = src[i];
    }
}

// bf16 bits of a value in [-2, 2) from a hash of the index: cheap, and the matrix cores' power
// draw depends on the data (all-zero inputs run at a higher clock than real ones).
__global__ void FillRandomBf16(uint16_t *dst, size_t n, uint32_t seed)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t h = (uint32_t)i * 2654435761u + seed;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        dst[i] = (uint16_t)((h & 0x8000u) | (0x3F00u + (h & 0xFFu)));   // sign, exponent 126..127, 7 mantissa bits
    }
}

static int GemmOfDepth(int k, int reps, hipStream_t stream)
{
    const int mn = 8192;
    uint16_t *a = nullptr, *b = nullptr, *c = nullptr;
    CHECK_HIP(hipMalloc((void **)&a, (size_t)mn * k * 2));
    CHECK_HIP(hipMalloc((void **)&b, (size_t)k * mn * 2));
    CHECK_HIP(hipMalloc((void **)&c, (size_t)mn * mn * 2));
    hipLaunchKernelGGL(FillRandomBf16, dim3(4096), dim3(256), 0, stream, a, (size_t)mn * k, 1u);
    hipLaunchKernelGGL(FillRandomBf16, dim3(4096), dim3(256), 0, stream, b, (size_t)k * mn, 2u);
    CHECK_HIP(hipStreamSynchronize(stream));
    HwQueueHandle hwq;
    XQueueHandle xq;
    CHECK_X(HipQueueCreate(&hwq, stream));
    CHECK_X(XQueueCreate(&xq, hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    CHECK_X(XQueueSetLaunchConfig(xq, 2, 1));
    auto run = [&](int count) {
        for (int i = 0; i < count; ++i) {
            HwCommandHandle cmd;
            CHECK_X(HipGemmBf16CommandCreate(&cmd, a, b, c, mn, mn, k, 0));
            CHECK_X(XQueueSubmit(xq, cmd));
        }
        CHECK_X(XQueueWaitAll(xq));
    };
    run(reps);   // the clock settles
    hipEvent_t e0, e1;
    CHECK_HIP(hipEventCreate(&e0)); CHECK_HIP(hipEventCreate(&e1));
    CHECK_HIP(hipEventRecord(e0, stream));
    run(reps);
    CHECK_HIP(hipEventRecord(e1, stream));
    CHECK_HIP(hipEventSynchronize(e1));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
    printf("traffic_probe: gemmk 8192x8192x%d reps=%d ms_per_launch=%.4f TFLOPs=%.1f\n", k, reps, ms / reps,
           2.0 * mn * mn * k / (ms / reps * 1e-3) / 1e12);
    CHECK_X(XQueueDestroy(xq));
    CHECK_X(HwQueueDestroy(hwq));
    return 0;
}

int main(int argc, char **argv)
{
    const size_t n = argc > 1 ? (size_t)atoll(argv[1]) : (size_t)1 << 28;
    const int reps = argc > 2 ? atoi(argv[2]) : 5;
    float *x = nullptr, *y = nullptr;
    CHECK_HIP(hipMalloc((void **)&x, n * 4));
    CHECK_HIP(hipMalloc((void **)&y, n * 4));
    CHECK_HIP(hipMemset(x, 0, n * 4));
    CHECK_HIP(hipMemset(y, 0, n * 4));
    CHECK_HIP(hipDeviceSynchronize()); // hipMemset returns before the fill has run; the stream below would not wait for it
    hipStream_t stream;
    CHECK_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));

    for (int i = 0; i < reps; ++i) {
        hipLaunchKernelGGL(PlainCopyKernel, dim3(8192), dim3(256), 0, stream, (const f4 *)x, (f4 *)y, n / 4);
    }
    CHECK_HIP(hipStreamSynchronize(stream));

    CHECK_X(XHintSetScheduler(kSchedulerAppManaged, kPolicyUnknown));
    if (argc > 4 && strcmp(argv[3], "gemmk") == 0) return GemmOfDepth(atoi(argv[4]), reps, stream);
    if (argc > 3) {
        // The harness of bench.py fills the seeded inputs and streams `reps` background commands.
        const bool hist = strcmp(argv[3], "hist") == 0;
        for (int pass = 0; pass < 2; ++pass) {
            XBenchConfig cfg;
            memset(&cfg, 0, sizeof cfg);
            cfg.n_bg = 1;
            cfg.bg.kind = hist ? kXBenchHist : kXBenchGemm;
            cfg.bg.guard = pass;                         // 0 plain, 1 guarded at level 2
            cfg.bg.n = hist ? (uint64_t)1 << 26 : 8192;
            cfg.bg.level = pass ? kPreemptLevelDeactivate : kPreemptLevelBlock;
            cfg.bg.threshold = 2; cfg.bg.batch = 1;
            cfg.fg = cfg.bg; cfg.fg.n = hist ? (uint64_t)1 << 20 : 1024; cfg.fg.period_us = 1000;
            cfg.bg_burst = reps;
            cfg.seed = 7;
            XBench *b = XBenchCreate(&cfg);
            if (b == nullptr) { fprintf(stderr, "XBenchCreate failed\n"); return 1; }
            XBenchPhaseResult res;
            CHECK_X(XBenchRunBackgroundAlone(b, reps, &res));
            XBenchDestroy(b);
        }
        printf("traffic_probe: %s reps=%d copy_bytes_read=%zu copy_bytes_written=%zu\n", argv[3], reps, n * 4, n * 4);
        return 0;
    }
    HwQueueHandle hwq;
    XQueueHandle xq;
    CHECK_X(HipQueueCreate(&hwq, stream));
    CHECK_X(XQueueCreate(&xq, hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    CHECK_X(XQueueSetLaunchConfig(xq, 2, 1));
    auto run = [&](int guard) {
        for (int i = 0; i < reps; ++i) {
            HwCommandHandle cmd;
            CHECK_X(HipAxpyCommandCreate(&cmd, 0.5f, x, y, n, guard));
            CHECK_X(XQueueSubmit(xq, cmd));
        }
        CHECK_X(XQueueWaitAll(xq));
    };
    run(0);                                                   // plain: AxpyPersistentKernel<3, false> from 2^23 elements on
    run(2);                                                   // AxpyPersistentKernel, no progress map
    CHECK_X(XQueueSetPreemptLevel(xq, kPreemptLevelDeactivate));
    run(1);                                                   // AxpyPersistentKernel with progress map
    CHECK_X(XQueueDestroy(xq));
    CHECK_X(HwQueueDestroy(hwq));
    printf("traffic_probe: n=%zu reps=%d copy_bytes_read=%zu copy_bytes_written=%zu axpy_algorithmic_bytes=%zu\n",
           n, reps, n * 4, n * 4, n * 12);
    return 0;
}
