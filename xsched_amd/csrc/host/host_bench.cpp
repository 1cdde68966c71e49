// The CPU-only configuration over the host adapter; see include/xsched/host/bench.h.
#include <atomic>
#include <chrono>
#include <thread>

#include "../bench/synth.h"
#include "xsched/hint.h"
#include "xsched/xqueue.h"
#include "xsched/host/bench.h"
#include "xsched/host/hal.h"
#include "xsched/utils/common.h"

namespace
{
using Clock = std::chrono::steady_clock;

#define HOSTBENCH_TRY(call) do { XResult r_ = (call); if (r_ != kXSchedSuccess) return r_; } while (0)

void SleepUntil(Clock::time_point tp)
{
    // most of the way asleep, the rest spinning: the period must not add the wake-up jitter
    // of this thread to what is measured
    const auto coarse = tp - std::chrono::microseconds(200);
    if (Clock::now() < coarse) std::this_thread::sleep_until(coarse);
    while (Clock::now() < tp) __builtin_ia32_pause();
}
} // namespace

EXPORT_C_FUNC void HostBenchFillUniform(float *dst, uint64_t first, uint64_t count, uint64_t seed, uint64_t stream)
{
    const uint64_t key = synth_stream_key(seed, stream);
    for (uint64_t i = 0; i < count; ++i) dst[i] = synth_uniform_pm1(key, first + i);
}

EXPORT_C_FUNC XResult HostBenchRunVecAdd(const HostBenchConfig *cfg, const float *bg_a, const float *bg_b, float *bg_c,
                                         const float *fg_a, const float *fg_b, float *fg_c,
                                         double *alone_us, double *contended_us, HostBenchResult *res)
{
    if (cfg == nullptr || bg_a == nullptr || bg_b == nullptr || bg_c == nullptr || fg_a == nullptr || fg_b == nullptr ||
        fg_c == nullptr || alone_us == nullptr || contended_us == nullptr || cfg->samples <= 0 || cfg->bg_burst <= 0 ||
        cfg->threshold < cfg->batch || cfg->batch <= 0) {
        return kXSchedErrorInvalidValue;
    }
    HOSTBENCH_TRY(XHintSetScheduler(kSchedulerLocal, kPolicyHighestPriorityFirst));
    HwQueueHandle bg_hwq = 0, fg_hwq = 0;
    XQueueHandle bg_xq = 0, fg_xq = 0;
    HOSTBENCH_TRY(HostQueueCreate(&bg_hwq));
    HOSTBENCH_TRY(HostQueueCreate(&fg_hwq));
    HOSTBENCH_TRY(XQueueCreate(&bg_xq, bg_hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    HOSTBENCH_TRY(XQueueCreate(&fg_xq, fg_hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    HOSTBENCH_TRY(XQueueSetLaunchConfig(bg_xq, cfg->threshold, cfg->batch));
    HOSTBENCH_TRY(XQueueSetLaunchConfig(fg_xq, cfg->threshold, cfg->batch));
    HOSTBENCH_TRY(XHintPriority(bg_xq, 1));
    HOSTBENCH_TRY(XHintPriority(fg_xq, 2));

    std::atomic<int> failed { 0 };
    uint64_t fg_done = 0;
    auto foreground = [&](double *out) {
        auto next = Clock::now();
        for (int i = 0; i < cfg->samples; ++i) {
            SleepUntil(next);
            const auto t0 = Clock::now();
            HwCommandHandle cmd = 0;
            if (HostVecAddCommandCreate(&cmd, fg_a, fg_b, fg_c, cfg->fg_n, 0) != kXSchedSuccess ||
                XQueueSubmit(fg_xq, cmd) != kXSchedSuccess || XQueueWaitAll(fg_xq) != kXSchedSuccess) failed.store(1);
            out[i] = std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
            fg_done++;
            next += std::chrono::microseconds(cfg->period_us);
        }
    };

    const auto t_alone = Clock::now();
    foreground(alone_us);
    const double alone_s = std::chrono::duration<double>(Clock::now() - t_alone).count();

    std::atomic<bool> stop { false };
    std::atomic<uint64_t> bg_done { 0 };
    std::thread background([&]() {
        while (!stop.load(std::memory_order_acquire)) {
            for (int i = 0; i < cfg->bg_burst; ++i) {
                HwCommandHandle cmd = 0;
                if (HostVecAddCommandCreate(&cmd, bg_a, bg_b, bg_c, cfg->bg_n, 0) != kXSchedSuccess ||
                    XQueueSubmit(bg_xq, cmd) != kXSchedSuccess) { failed.store(1); return; }
            }
            if (XQueueWaitAll(bg_xq) != kXSchedSuccess) { failed.store(1); return; }
            bg_done.fetch_add((uint64_t)cfg->bg_burst, std::memory_order_relaxed);
        }
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(20));
    const auto t_cont = Clock::now();
    foreground(contended_us);
    const double contended_s = std::chrono::duration<double>(Clock::now() - t_cont).count();
    stop.store(true, std::memory_order_release);
    background.join();

    if (res != nullptr) {
        res->alone_s = alone_s;
        res->contended_s = contended_s;
        res->bg_commands = bg_done.load();
        res->fg_commands = fg_done;
    }
    HOSTBENCH_TRY(XQueueDestroy(bg_xq));
    HOSTBENCH_TRY(XQueueDestroy(fg_xq));
    HOSTBENCH_TRY(HwQueueDestroy(bg_hwq));
    HOSTBENCH_TRY(HwQueueDestroy(fg_hwq));
    HOSTBENCH_TRY(XHintSetScheduler(kSchedulerAppManaged, kPolicyUnknown));
    return failed.load() ? kXSchedErrorUnknown : kXSchedSuccess;
}
