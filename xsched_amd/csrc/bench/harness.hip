// Contention benchmark harness; see include/xsched/hip/bench.h.
#include <atomic>
#include <chrono>
#include <cmath>
#include <memory>
#include <thread>
#include <vector>

#include <hip/hip_runtime.h>

#include "synth.h"
#include "xsched/hip/bench.h"
#include "xsched/hip/hal.h"
#include "xsched/xsched.h"
#include "xsched/utils/common.h"
#include "xsched/utils/log.h"

using Clock = std::chrono::steady_clock;

#define BENCH_HIP(expr) \
    do { hipError_t e_ = (expr); if (e_ != hipSuccess) { \
        XERRO("HIP error %d (%s) at %s", (int)e_, hipGetErrorString(e_), #expr); } } while (0)
#define BENCH_X(expr) \
    do { XResult r_ = (expr); if (r_ != kXSchedSuccess) { XERRO("XSched error %d at %s", (int)r_, #expr); } } while (0)

namespace
{

// ---- device fill kernels -------------------------------------------------------

__global__ void FillUniform(float *dst, uint64_t n, uint64_t key)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (uint64_t)gridDim.x * blockDim.x) dst[i] = synth_uniform_pm1(key, i);
}

__global__ void FillNormalBf16(uint16_t *dst, uint64_t n, uint64_t key)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (uint64_t)gridDim.x * blockDim.x) dst[i] = synth_normal_bf16(key, i);
}

__global__ void FillZipf(int32_t *dst, uint64_t n, uint64_t key, const uint32_t *table, uint32_t n_bins)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (uint64_t)gridDim.x * blockDim.x) dst[i] = (int32_t)synth_zipf_key(table, n_bins, key, i);
}

// y = 0.5 * x + y with 128-bit accesses, one work-group per 1024 elements: the plain-HIP
// stand-in of the foreground AXPY for the latency floor (n a multiple of 4).
__global__ void FloorAxpy(const float4 *x, float4 *y, uint64_t n4)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n4) {
        const float4 a = x[i];
        float4 b = y[i];
        b.x = fmaf(0.5f, a.x, b.x); b.y = fmaf(0.5f, a.y, b.y);
        b.z = fmaf(0.5f, a.z, b.z); b.w = fmaf(0.5f, a.w, b.w);
        y[i] = b;
    }
}

constexpr uint32_t kHistBins = 65536;
constexpr double kZipfS = 1.1;

std::vector<uint32_t> ZipfTable(uint32_t n_bins, double s)
{
    std::vector<long double> h(n_bins);
    long double acc = 0;
    for (uint32_t k = 0; k < n_bins; ++k) { acc += powl((long double)(k + 1), -(long double)s); h[k] = acc; }
    std::vector<uint32_t> t(n_bins);
    for (uint32_t k = 0; k < n_bins; ++k) {
        long double v = floorl(4294967296.0L * (h[k] / acc));
        t[k] = v >= 4294967295.0L ? 0xFFFFFFFFu : (uint32_t)v;
    }
    t[n_bins - 1] = 0xFFFFFFFFu;
    return t;
}

// ---- one queue with its buffers ------------------------------------------------

struct Lane
{
    XBenchQueueSpec spec {};
    hipStream_t stream = nullptr;
    HwQueueHandle hwq = 0;
    XQueueHandle xq = 0;
    void *in0 = nullptr, *in1 = nullptr, *out = nullptr; // axpy: x,-,y  gemm: A,B,C  hist: keys,-,bins
    std::atomic<uint64_t> applied { 0 };

    HwCommandHandle MakeCommand() const
    {
        HwCommandHandle cmd = 0;
        switch (spec.kind) {
        case kXBenchAxpy:
            BENCH_X(HipAxpyCommandCreate(&cmd, 0.5f, in0, out, spec.n, spec.guard));
            break;
        case kXBenchGemm:
            BENCH_X(HipGemmBf16CommandCreate(&cmd, in0, in1, out, (int)spec.n, (int)spec.n, (int)spec.n, spec.guard));
            break;
        case kXBenchHist:
            BENCH_X(HipHistogramCommandCreate(&cmd, in0, spec.n, out, kHistBins, spec.guard));
            break;
        default:
            XERRO("unknown workload kind %d", spec.kind);
        }
        return cmd;
    }

    void Submit() { BENCH_X(XQueueSubmit(xq, MakeCommand())); applied.fetch_add(1, std::memory_order_relaxed); }

    size_t OutElemSize() const { return spec.kind == kXBenchGemm ? 2 : 4; }
    uint64_t OutElems() const
    {
        if (spec.kind == kXBenchAxpy) return spec.n;
        if (spec.kind == kXBenchGemm) return spec.n * spec.n;
        return kHistBins;
    }
};

} // namespace

struct XBench
{
    XBenchConfig cfg {};
    XBenchStressConfig stress {};
    std::vector<std::unique_ptr<Lane>> bg;
    std::unique_ptr<Lane> fg;
    uint32_t *zipf_table_dev = nullptr;
};

namespace
{

void SetupLane(XBench &b, Lane &lane, const XBenchQueueSpec &spec, uint64_t seed, uint64_t lane_id)
{
    lane.spec = spec;
    BENCH_HIP(hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking));
    const uint64_t k0 = synth_stream_key(seed, lane_id * 4 + 0);
    const uint64_t k1 = synth_stream_key(seed, lane_id * 4 + 1);
    const dim3 grid(2048), block(256);

    switch (spec.kind) {
    case kXBenchAxpy:
        BENCH_HIP(hipMalloc(&lane.in0, spec.n * 4));
        BENCH_HIP(hipMalloc(&lane.out, spec.n * 4));
        hipLaunchKernelGGL(FillUniform, grid, block, 0, lane.stream, (float *)lane.in0, spec.n, k0);
        hipLaunchKernelGGL(FillUniform, grid, block, 0, lane.stream, (float *)lane.out, spec.n, k1);
        break;
    case kXBenchGemm:
        BENCH_HIP(hipMalloc(&lane.in0, spec.n * spec.n * 2));
        BENCH_HIP(hipMalloc(&lane.in1, spec.n * spec.n * 2));
        BENCH_HIP(hipMalloc(&lane.out, spec.n * spec.n * 2));
        hipLaunchKernelGGL(FillNormalBf16, grid, block, 0, lane.stream, (uint16_t *)lane.in0, spec.n * spec.n, k0);
        hipLaunchKernelGGL(FillNormalBf16, grid, block, 0, lane.stream, (uint16_t *)lane.in1, spec.n * spec.n, k1);
        BENCH_HIP(hipMemsetAsync(lane.out, 0, spec.n * spec.n * 2, lane.stream));
        break;
    case kXBenchHist:
        if (b.zipf_table_dev == nullptr) {
            const auto table = ZipfTable(kHistBins, kZipfS);
            BENCH_HIP(hipMalloc((void **)&b.zipf_table_dev, kHistBins * 4));
            BENCH_HIP(hipMemcpy(b.zipf_table_dev, table.data(), kHistBins * 4, hipMemcpyHostToDevice));
        }
        BENCH_HIP(hipMalloc(&lane.in0, spec.n * 4));
        BENCH_HIP(hipMalloc(&lane.out, kHistBins * 4));
        hipLaunchKernelGGL(FillZipf, grid, block, 0, lane.stream, (int32_t *)lane.in0, spec.n, k0,
                           b.zipf_table_dev, kHistBins);
        BENCH_HIP(hipMemsetAsync(lane.out, 0, kHistBins * 4, lane.stream));
        break;
    default:
        XERRO("unknown workload kind %d", spec.kind);
    }
    BENCH_HIP(hipGetLastError());
    BENCH_HIP(hipStreamSynchronize(lane.stream));

    BENCH_X(HipQueueCreate(&lane.hwq, lane.stream));
    BENCH_X(XQueueCreate(&lane.xq, lane.hwq, spec.level, kQueueCreateFlagNone));
    BENCH_X(XQueueSetLaunchConfig(lane.xq, spec.threshold, spec.batch));
    if (b.cfg.policy == kPolicyLaxity && spec.laxity_us >= 0) {
        BENCH_X(XHintLaxity(lane.xq, spec.laxity_us, spec.lax_priority, spec.priority));
    } else if (b.cfg.policy == kPolicyLaxity) {
        // No laxity: a constant priority (lax == crit).
        BENCH_X(XHintLaxity(lane.xq, 0, spec.priority, spec.priority));
    } else {
        BENCH_X(XHintPriority(lane.xq, spec.priority));
    }
}

void TeardownLane(Lane &lane)
{
    if (lane.xq) BENCH_X(XQueueDestroy(lane.xq));
    if (lane.hwq) BENCH_X(HwQueueDestroy(lane.hwq));
    if (lane.stream) { (void)hipStreamSynchronize(lane.stream); (void)hipStreamDestroy(lane.stream); }
    (void)hipFree(lane.in0); (void)hipFree(lane.in1); (void)hipFree(lane.out);
}

// Streams commands on one background queue until told to stop: bursts of
// `burst` commands with a drain after each (the drain of burst k overlaps nothing,
// so bursts are long: the bubble is one launch latency per burst).
struct BgDriver
{
    Lane *lane;
    int burst;
    std::atomic<bool> *stop;
    std::atomic<uint64_t> done { 0 };
    std::thread thread;
    // Optional timing events, recorded in stream order around everything submitted.
    hipEvent_t ev_first = nullptr, ev_last = nullptr;
    uint64_t submitted = 0;

    void Record(hipEvent_t ev)
    {
        HwCommandHandle rec = 0;
        BENCH_X(HipEventRecordCommandCreate(&rec, ev));
        BENCH_X(XQueueSubmit(lane->xq, rec));
    }

    void Start()
    {
        thread = std::thread([this]() {
            if (ev_first) Record(ev_first);
            while (!stop->load(std::memory_order_acquire)) {
                for (int i = 0; i < burst && !stop->load(std::memory_order_relaxed); ++i) {
                    lane->Submit();
                    submitted++;
                }
                BENCH_X(XQueueWaitAll(lane->xq));
                done.store(lane->applied.load(), std::memory_order_release);
            }
            if (ev_last) {
                Record(ev_last);
                BENCH_X(XQueueWaitAll(lane->xq));
            }
        });
    }
    void Join() { if (thread.joinable()) thread.join(); }
};

void FillStats(XBench *b, XBenchPhaseResult *res)
{
    if (res && !b->bg.empty()) (void)HipQueueGetStats(b->bg[0]->hwq, res->stats);
}

void SleepUntil(Clock::time_point tp)
{
    // Sleep most of the way, spin the rest: the period must not add wake-up jitter
    // to the measured latency.
    const auto coarse = tp - std::chrono::microseconds(200);
    if (Clock::now() < coarse) std::this_thread::sleep_until(coarse);
    while (Clock::now() < tp) __builtin_ia32_pause();
}

// One foreground sample: ready time, submit, wait, latency.
double ForegroundOnce(Lane &fg, bool *missed)
{
    const auto t0 = Clock::now();
    fg.Submit();
    BENCH_X(XQueueWaitAll(fg.xq));
    const double us = std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
    if (missed) *missed = fg.spec.deadline_us > 0 && us > (double)fg.spec.deadline_us;
    return us;
}

} // namespace

extern "C" {

EXPORT_C_FUNC XBench *XBenchCreate(const XBenchConfig *cfg)
{
    if (cfg == nullptr || cfg->n_bg < 0 || cfg->n_bg > 64) return nullptr;
    auto *b = new XBench();
    b->cfg = *cfg;
    if (cfg->policy != kPolicyUnknown) BENCH_X(XHintSetScheduler(kSchedulerLocal, (XPolicyType)cfg->policy));
    else BENCH_X(XHintSetScheduler(kSchedulerAppManaged, kPolicyUnknown));
    for (int i = 0; i < cfg->n_bg; ++i) {
        b->bg.emplace_back(std::make_unique<Lane>());
        SetupLane(*b, *b->bg.back(), cfg->bg, cfg->seed, (uint64_t)i + 1);
    }
    if (cfg->fg.n > 0) {
        b->fg = std::make_unique<Lane>();
        SetupLane(*b, *b->fg, cfg->fg, cfg->seed, 0);
    }
    return b;
}

EXPORT_C_FUNC void XBenchDestroy(XBench *b)
{
    if (b == nullptr) return;
    for (auto &lane : b->bg) TeardownLane(*lane);
    if (b->fg) TeardownLane(*b->fg);
    (void)hipFree(b->zipf_table_dev);
    delete b;
}

EXPORT_C_FUNC XResult XBenchRunForegroundAlone(XBench *b, int samples, double *latency_us,
                                               XBenchPhaseResult *res)
{
    if (b == nullptr || b->fg == nullptr || samples <= 0 || latency_us == nullptr) return kXSchedErrorInvalidValue;
    Lane &fg = *b->fg;
    const auto t_begin = Clock::now();
    auto next = t_begin;
    uint64_t missed = 0;
    for (int i = 0; i < samples; ++i) {
        SleepUntil(next);
        bool m = false;
        latency_us[i] = ForegroundOnce(fg, &m);
        missed += m;
        next += std::chrono::microseconds(fg.spec.period_us);
    }
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = std::chrono::duration<double>(Clock::now() - t_begin).count();
        res->fg_samples = (uint64_t)samples;
        res->fg_deadline_miss = missed;
        FillStats(b, res);
    }
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchRunBackgroundAlone(XBench *b, int commands, XBenchPhaseResult *res)
{
    if (b == nullptr || b->bg.empty() || commands <= 0) return kXSchedErrorInvalidValue;
    hipEvent_t ev0, ev1;
    BENCH_HIP(hipEventCreate(&ev0));
    BENCH_HIP(hipEventCreate(&ev1));
    Lane &q0 = *b->bg[0];

    // Timing events travel through the XQueue like any other command, so they sit
    // in stream order right before the first and right after the last kernel.
    HwCommandHandle rec = 0;
    BENCH_X(HipEventRecordCommandCreate(&rec, ev0));
    BENCH_X(XQueueSubmit(q0.xq, rec));
    const auto t0 = Clock::now();
    for (int i = 0; i < commands; ++i) for (auto &lane : b->bg) lane->Submit();
    BENCH_X(HipEventRecordCommandCreate(&rec, ev1));
    BENCH_X(XQueueSubmit(q0.xq, rec));
    for (auto &lane : b->bg) BENCH_X(XQueueWaitAll(lane->xq));
    const double elapsed = std::chrono::duration<double>(Clock::now() - t0).count();

    float ms = 0;
    BENCH_HIP(hipEventSynchronize(ev1));
    BENCH_HIP(hipEventElapsedTime(&ms, ev0, ev1));
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = elapsed;
        res->bg_commands = (uint64_t)commands * b->bg.size();
        res->bg_stream_ms = ms;
        res->bg_stream_cmds = (uint64_t)commands;
        FillStats(b, res);
    }
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchRunContended(XBench *b, int samples, double *latency_us,
                                         XBenchPhaseResult *res)
{
    if (b == nullptr || b->fg == nullptr || b->bg.empty() || samples <= 0 || latency_us == nullptr) {
        return kXSchedErrorInvalidValue;
    }
    Lane &fg = *b->fg;
    std::atomic<bool> stop { false };
    std::vector<std::unique_ptr<BgDriver>> drivers;
    uint64_t applied_before = 0;
    for (auto &lane : b->bg) {
        applied_before += lane->applied.load();
        auto d = std::make_unique<BgDriver>();
        d->lane = lane.get();
        d->burst = b->cfg.bg_burst > 0 ? b->cfg.bg_burst : 64;
        d->stop = &stop;
        drivers.emplace_back(std::move(d));
    }
    hipEvent_t ev0, ev1;
    BENCH_HIP(hipEventCreate(&ev0));
    BENCH_HIP(hipEventCreate(&ev1));
    drivers[0]->ev_first = ev0;
    drivers[0]->ev_last = ev1;
    const auto t_begin = Clock::now();
    for (auto &d : drivers) d->Start();
    // Let the background reach steady state before the first sample.
    std::this_thread::sleep_for(std::chrono::milliseconds(50));

    auto next = Clock::now();
    uint64_t missed = 0;
    for (int i = 0; i < samples; ++i) {
        SleepUntil(next);
        bool m = false;
        latency_us[i] = ForegroundOnce(fg, &m);
        missed += m;
        next += std::chrono::microseconds(fg.spec.period_us);
    }
    stop.store(true, std::memory_order_release);
    for (auto &d : drivers) d->Join();
    const double elapsed = std::chrono::duration<double>(Clock::now() - t_begin).count();

    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = elapsed;
        uint64_t applied_after = 0;
        for (auto &lane : b->bg) applied_after += lane->applied.load();
        res->bg_commands = applied_after - applied_before;
        res->fg_samples = (uint64_t)samples;
        res->fg_deadline_miss = missed;
        float ms = 0;
        if (hipEventSynchronize(ev1) == hipSuccess && hipEventElapsedTime(&ms, ev0, ev1) == hipSuccess) {
            res->bg_stream_ms = ms;
            res->bg_stream_cmds = drivers[0]->submitted;
        }
        FillStats(b, res);
    }
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchRunForegroundBreakdown(XBench *b, int samples, int mode, int contended, double *out,
                                                   XBenchPhaseResult *res)
{
    if (b == nullptr || b->fg == nullptr || samples <= 0 || out == nullptr || mode < 0 || mode > 2) {
        return kXSchedErrorInvalidValue;
    }
    if (contended && b->bg.empty()) return kXSchedErrorInvalidValue;
    Lane &fg = *b->fg;
    if (mode == 2 && (fg.spec.kind != kXBenchAxpy || fg.spec.n % 4 != 0)) return kXSchedErrorNotSupported;
    hipEvent_t ev_a, ev_b;
    BENCH_HIP(hipEventCreate(&ev_a));
    BENCH_HIP(hipEventCreate(&ev_b));
    // modes 1 and 2 use a stream of their own, with no XQueue on it
    hipStream_t raw = nullptr;
    HwQueueHandle raw_hwq = 0;
    if (mode != 0) {
        BENCH_X(XQueueWaitAll(fg.xq));
        BENCH_HIP(hipStreamCreateWithFlags(&raw, hipStreamNonBlocking));
        if (mode == 1) BENCH_X(HipQueueCreate(&raw_hwq, raw));
    }

    std::atomic<bool> stop { false };
    std::vector<std::unique_ptr<BgDriver>> drivers;
    if (contended) {
        for (auto &lane : b->bg) {
            auto d = std::make_unique<BgDriver>();
            d->lane = lane.get();
            d->burst = b->cfg.bg_burst > 0 ? b->cfg.bg_burst : 64;
            d->stop = &stop;
            drivers.emplace_back(std::move(d));
        }
        for (auto &d : drivers) d->Start();
        std::this_thread::sleep_for(std::chrono::milliseconds(50));
    }

    const auto t_begin = Clock::now();
    auto next = t_begin;
    auto us = [](Clock::duration d) { return std::chrono::duration<double, std::micro>(d).count(); };
    for (int i = 0; i < samples; ++i) {
        SleepUntil(next);
        Clock::time_point t0, t1, t2;
        if (mode == 0) {
            HwCommandHandle rec_a = 0, rec_b = 0;
            BENCH_X(HipEventRecordCommandCreate(&rec_a, ev_a));
            BENCH_X(HipEventRecordCommandCreate(&rec_b, ev_b));
            const HwCommandHandle cmd = fg.MakeCommand();
            t0 = Clock::now();
            BENCH_X(XQueueSubmit(fg.xq, rec_a));
            BENCH_X(XQueueSubmit(fg.xq, cmd));
            BENCH_X(XQueueSubmit(fg.xq, rec_b));
            t1 = Clock::now();
            BENCH_X(XQueueWaitAll(fg.xq));
            t2 = Clock::now();
            fg.applied.fetch_add(1, std::memory_order_relaxed);
        } else if (mode == 1) {
            const HwCommandHandle cmd = fg.MakeCommand();
            t0 = Clock::now();
            BENCH_HIP(hipEventRecord(ev_a, raw));
            BENCH_X(HwQueueLaunch(raw_hwq, cmd));
            BENCH_HIP(hipEventRecord(ev_b, raw));
            t1 = Clock::now();
            BENCH_X(HwQueueSynchronize(raw_hwq));
            t2 = Clock::now();
            fg.applied.fetch_add(1, std::memory_order_relaxed);
        } else {
            const uint64_t n4 = fg.spec.n / 4;
            t0 = Clock::now();
            BENCH_HIP(hipEventRecord(ev_a, raw));
            hipLaunchKernelGGL(FloorAxpy, dim3((uint32_t)((n4 + 255) / 256)), dim3(256), 0, raw,
                               (const float4 *)fg.in0, (float4 *)fg.out, n4);
            BENCH_HIP(hipEventRecord(ev_b, raw));
            t1 = Clock::now();
            while (hipStreamQuery(raw) == hipErrorNotReady) __builtin_ia32_pause();
            t2 = Clock::now();
            fg.applied.fetch_add(1, std::memory_order_relaxed);
        }
        float ms = 0;
        BENCH_HIP(hipEventSynchronize(ev_b));
        BENCH_HIP(hipEventElapsedTime(&ms, ev_a, ev_b));
        out[(size_t)i * 4 + 0] = us(t1 - t0);
        out[(size_t)i * 4 + 1] = (double)ms * 1e3;
        out[(size_t)i * 4 + 2] = us(t2 - t1);
        out[(size_t)i * 4 + 3] = us(t2 - t0);
        next += std::chrono::microseconds(fg.spec.period_us);
    }
    stop.store(true, std::memory_order_release);
    for (auto &d : drivers) d->Join();
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = std::chrono::duration<double>(Clock::now() - t_begin).count();
        res->fg_samples = (uint64_t)samples;
        FillStats(b, res);
    }
    if (raw_hwq) BENCH_X(HwQueueDestroy(raw_hwq));
    if (raw) { (void)hipStreamSynchronize(raw); (void)hipStreamDestroy(raw); }
    (void)hipEventDestroy(ev_a);
    (void)hipEventDestroy(ev_b);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchRunPreempt(XBench *b, int samples, double *suspend_us, double *resume_us,
                                       XBenchPhaseResult *res)
{
    if (b == nullptr || b->bg.empty() || samples <= 0 || suspend_us == nullptr || resume_us == nullptr) {
        return kXSchedErrorInvalidValue;
    }
    Lane &q0 = *b->bg[0];
    std::atomic<bool> stop { false };
    BgDriver driver;
    driver.lane = &q0;
    driver.burst = b->cfg.bg_burst > 0 ? b->cfg.bg_burst : 64;
    driver.stop = &stop;
    const auto t_begin = Clock::now();
    driver.Start();
    std::this_thread::sleep_for(std::chrono::milliseconds(50));

    uint64_t lcg = 0x2545F4914F6CDD1Dull ^ b->cfg.seed;
    for (int i = 0; i < samples; ++i) {
        lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
        std::this_thread::sleep_for(std::chrono::microseconds(200 + (lcg >> 33) % 800));
        auto t0 = Clock::now();
        BENCH_X(XQueueSuspend(q0.xq, kQueueSuspendFlagSyncHwQueue));
        auto t1 = Clock::now();
        std::this_thread::sleep_for(std::chrono::microseconds(300));
        auto t2 = Clock::now();
        BENCH_X(XQueueResume(q0.xq, kQueueResumeFlagNone));
        auto t3 = Clock::now();
        suspend_us[i] = std::chrono::duration<double, std::micro>(t1 - t0).count();
        resume_us[i] = std::chrono::duration<double, std::micro>(t3 - t2).count();
    }
    stop.store(true, std::memory_order_release);
    driver.Join();
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = std::chrono::duration<double>(Clock::now() - t_begin).count();
        res->bg_commands = q0.applied.load();
        FillStats(b, res);
    }
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchRunPreemptDeviceTimed(XBench *b, int samples, double *drain_us, XBenchPhaseResult *res)
{
    if (b == nullptr || b->bg.empty() || samples <= 0 || drain_us == nullptr) return kXSchedErrorInvalidValue;
    Lane &q0 = *b->bg[0];
    hipStream_t helper = nullptr;
    hipEvent_t ev_out = nullptr, ev_drained = nullptr;
    BENCH_HIP(hipStreamCreateWithFlags(&helper, hipStreamNonBlocking));
    BENCH_HIP(hipEventCreate(&ev_out));
    BENCH_HIP(hipEventCreate(&ev_drained));

    std::atomic<bool> stop { false };
    BgDriver driver;
    driver.lane = &q0;
    driver.burst = b->cfg.bg_burst > 0 ? b->cfg.bg_burst : 64;
    driver.stop = &stop;
    const auto t_begin = Clock::now();
    driver.Start();
    std::this_thread::sleep_for(std::chrono::milliseconds(50));

    uint64_t lcg = 0x9E3779B97F4A7C15ull ^ b->cfg.seed;
    for (int i = 0; i < samples; ++i) {
        lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
        std::this_thread::sleep_for(std::chrono::microseconds(200 + (lcg >> 33) % 800));
        BENCH_X(XQueueSuspend(q0.xq, kQueueSuspendFlagNone));
        // The launch thread is paused, so nothing else is enqueued on the stream now.
        BENCH_HIP(hipEventRecord(ev_out, helper));
        BENCH_HIP(hipEventRecord(ev_drained, q0.stream));
        BENCH_HIP(hipEventSynchronize(ev_drained));
        BENCH_HIP(hipEventSynchronize(ev_out));
        float ms = 0;
        BENCH_HIP(hipEventElapsedTime(&ms, ev_out, ev_drained));
        drain_us[i] = (double)ms * 1e3;
        std::this_thread::sleep_for(std::chrono::microseconds(300));
        BENCH_X(XQueueResume(q0.xq, kQueueResumeFlagNone));
    }
    stop.store(true, std::memory_order_release);
    driver.Join();
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = std::chrono::duration<double>(Clock::now() - t_begin).count();
        res->bg_commands = q0.applied.load();
        FillStats(b, res);
    }
    (void)hipEventDestroy(ev_out);
    (void)hipEventDestroy(ev_drained);
    (void)hipStreamDestroy(helper);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XBench *XBenchCreateStress(const XBenchStressConfig *cfg)
{
    if (cfg == nullptr || cfg->n_queues <= 0 || cfg->n_queues > 64 || cfg->mean_interarrival_us <= 0) return nullptr;
    auto *b = new XBench();
    b->stress = *cfg;
    b->cfg.policy = cfg->policy;
    b->cfg.seed = cfg->seed;
    if (cfg->policy != kPolicyUnknown) BENCH_X(XHintSetScheduler(kSchedulerLocal, (XPolicyType)cfg->policy));
    else BENCH_X(XHintSetScheduler(kSchedulerAppManaged, kPolicyUnknown));
    for (int i = 0; i < cfg->n_queues; ++i) {
        XBenchQueueSpec spec {};
        spec.kind = i % 3;
        spec.guard = cfg->guard;
        spec.n = spec.kind == kXBenchAxpy ? cfg->axpy_n : spec.kind == kXBenchGemm ? cfg->gemm_n : cfg->hist_n;
        spec.level = cfg->level;
        spec.threshold = cfg->threshold;
        spec.batch = cfg->batch;
        spec.priority = i;
        spec.laxity_us = -1;
        b->bg.emplace_back(std::make_unique<Lane>());
        SetupLane(*b, *b->bg.back(), spec, cfg->seed, (uint64_t)i + 1);
    }
    return b;
}

EXPORT_C_FUNC XResult XBenchRunStress(XBench *b, double duration_s, double *latency_us, uint64_t cap,
                                      uint64_t *counts, XBenchPhaseResult *res)
{
    return XBenchRunStressQueues(b, duration_s, ~0ull, latency_us, cap, counts, res);
}

EXPORT_C_FUNC XResult XBenchRunStressQueues(XBench *b, double duration_s, uint64_t queue_mask, double *latency_us,
                                            uint64_t cap, uint64_t *counts, XBenchPhaseResult *res)
{
    if (b == nullptr || b->stress.n_queues <= 0 || b->stress.n_queues > 64 || (size_t)b->stress.n_queues != b->bg.size() ||
        duration_s <= 0 || latency_us == nullptr || counts == nullptr || cap == 0) {
        return kXSchedErrorInvalidValue;
    }
    const int nq = b->stress.n_queues;
    const double mean = b->stress.mean_interarrival_us;
    uint64_t applied_before = 0;
    for (auto &lane : b->bg) applied_before += lane->applied.load();
    const auto t_begin = Clock::now() + std::chrono::milliseconds(5);
    std::vector<std::thread> threads;
    for (int i = 0; i < nq; ++i) {
        counts[i] = 0;
        if (!((queue_mask >> i) & 1)) continue;
        threads.emplace_back([&, i]() {
            Lane &lane = *b->bg[i];
            const uint64_t key = synth_stream_key(b->stress.seed, 1000 + (uint64_t)i);
            double t_us = 0; // arrival time since t_begin
            for (uint64_t k = 0;; ++k) {
                const double u = (double)(synth_bits(key, k) >> 11) * (1.0 / 9007199254740992.0);
                t_us += -mean * std::log1p(-u);
                if (t_us > duration_s * 1e6) break;
                const auto arrival = t_begin + std::chrono::nanoseconds((int64_t)(t_us * 1e3));
                SleepUntil(arrival);
                lane.Submit();
                BENCH_X(XQueueWaitAll(lane.xq));
                const double us = std::chrono::duration<double, std::micro>(Clock::now() - arrival).count();
                if (counts[i] < cap) latency_us[(uint64_t)i * cap + counts[i]++] = us;
            }
        });
    }
    for (auto &t : threads) t.join();
    if (res) {
        *res = XBenchPhaseResult {};
        res->elapsed_s = std::chrono::duration<double>(Clock::now() - t_begin).count();
        uint64_t applied_after = 0;
        for (auto &lane : b->bg) applied_after += lane->applied.load();
        res->bg_commands = applied_after - applied_before;
        FillStats(b, res);
    }
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XBenchReadOutput(XBench *b, int which, int q, uint64_t first, uint64_t count,
                                       void *dst, uint64_t *applied)
{
    if (b == nullptr || dst == nullptr) return kXSchedErrorInvalidValue;
    Lane *lane = nullptr;
    if (which == 1) lane = b->fg.get();
    else if (q >= 0 && (size_t)q < b->bg.size()) lane = b->bg[q].get();
    if (lane == nullptr) return kXSchedErrorNotFound;
    if (first + count > lane->OutElems()) return kXSchedErrorInvalidValue;
    BENCH_X(XQueueWaitAll(lane->xq));
    const size_t es = lane->OutElemSize();
    BENCH_HIP(hipMemcpy(dst, (const char *)lane->out + first * es, count * es, hipMemcpyDeviceToHost));
    if (applied) *applied = lane->applied.load();
    return kXSchedSuccess;
}

} // extern "C"
