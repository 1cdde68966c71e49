// Where the slow samples of a "launch, record an event, wait" loop come from: plain HIP, no
// library of this repository involved. A short kernel every PERIOD_US on one non-blocking
// stream, launch-to-completion time per sample, the wait done by polling hipEventQuery or by
// hipEventSynchronize. Prints the median, the p99 and the numbers of the samples that took
// more than 20 us longer than the median: with the runtime's own pool of completion signals
// they come at a fixed period (every 256 packets of the queue; a launch is one packet, an
// event record two), with ROC_SIGNAL_POOL_SIZE=512 in the environment they do not.
//
//   launch_tail_probe [SAMPLES] [PERIOD_US]
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { \
    fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); exit(2); } } while (0)

__global__ void Touch(float *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] += 1.0f;
}

using Clock = std::chrono::steady_clock;

static void Run(const char *name, bool poll, int samples, int period_us, hipStream_t stream, float *buf, int n)
{
    hipEvent_t ev;
    CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    std::vector<double> lat;
    auto next = Clock::now();
    for (int i = 0; i < samples; ++i) {
        while (Clock::now() < next) {}
        const auto t0 = Clock::now();
        Touch<<<n / 256, 256, 0, stream>>>(buf, n);
        CHECK(hipEventRecord(ev, stream));
        if (poll) { while (hipEventQuery(ev) == hipErrorNotReady) {} }
        else CHECK(hipEventSynchronize(ev));
        lat.push_back(std::chrono::duration<double, std::micro>(Clock::now() - t0).count());
        next += std::chrono::microseconds(period_us);
    }
    std::vector<double> sorted = lat;
    std::sort(sorted.begin(), sorted.end());
    const double p50 = sorted[sorted.size() / 2], p99 = sorted[sorted.size() * 99 / 100];
    printf("%-24s n=%d p50_us=%.1f p99_us=%.1f long samples:", name, samples, p50, p99);
    int shown = 0;
    for (int i = 1; i < samples && shown < 16; ++i) {
        if (lat[(size_t)i] > p50 + 20) { printf(" %d(%.0f)", i, lat[(size_t)i]); shown++; }
    }
    printf("\n");
    CHECK(hipEventDestroy(ev));
}

int main(int argc, char **argv)
{
    const int samples = argc > 1 ? atoi(argv[1]) : 800;
    const int period_us = argc > 2 ? atoi(argv[2]) : 3000;
    if (samples < 10 || period_us < 0) { fprintf(stderr, "usage: launch_tail_probe [SAMPLES >= 10] [PERIOD_US]\n"); return 2; }
    const int n = 1 << 22;
    float *buf;
    CHECK(hipMalloc((void **)&buf, (size_t)n * 4));
    CHECK(hipMemset(buf, 0, (size_t)n * 4));
    CHECK(hipDeviceSynchronize());
    hipStream_t stream;
    CHECK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    const char *pool = getenv("ROC_SIGNAL_POOL_SIZE");
    printf("ROC_SIGNAL_POOL_SIZE=%s\n", pool ? pool : "(unset)");
    Run("hipEventQuery polled", true, samples, period_us, stream, buf, n);
    Run("hipEventSynchronize", false, samples, period_us, stream, buf, n);
    CHECK(hipStreamDestroy(stream));
    CHECK(hipFree(buf));
    return 0;
}
