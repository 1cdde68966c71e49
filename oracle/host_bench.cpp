// ORACLE - test infrastructure only. The headline workload (background AXPY back to back
// at priority 1, foreground AXPY every period at priority 2, level 1, local scheduler with
// the highest-priority-first policy) run on CPU cores through the PUBLIC C API only:
// XQueueCreate / XQueueSetLaunchConfig / XHintSetScheduler / XHintPriority / XQueueSubmit /
// XQueueWaitAll over the host adapter. Because it touches nothing but that API it links
// against either XQueue core:
//   _ref/libxqueue_ref.so   the reference's own core, scheduler and policy sources (the
//                           CPU baseline of kind "reference": XSched's host-side loop as
//                           its authors wrote it, driving scalar CPU kernels)
//   libhostbench.so         the shipped libpreempt.so + libhalhost.so
// The reference ships no CPU adapter, so both builds use this repository's host adapter
// (xsched_amd/csrc/host/host_queue.cpp) compiled against the respective headers.
#include <atomic>
#include <chrono>
#include <cstring>
#include <thread>
#include <vector>

#include "xsched/hint.h"
#include "xsched/xqueue.h"
#include "xsched/host/hal.h"

extern "C" {
// oracle/kernels.c
uint64_t oracle_stream_key(uint64_t seed, uint64_t stream);
void oracle_fill_uniform(float *out, uint64_t first, uint64_t n, uint64_t key);
}

namespace
{
using Clock = std::chrono::steady_clock;

#define HB_CHECK(call) do { XResult r_ = (call); if (r_ != kXSchedSuccess) return (int)r_; } while (0)
} // namespace

// bg_n / fg_n: elements of the background / foreground AXPY; one foreground command every
// period_us, `samples` of them alone and `samples` beside the background stream; the
// background window is bg_threshold / bg_batch (foreground 8 / 4). Outputs: the two latency
// arrays (microseconds), background commands completed and seconds of the contended phase,
// and a checksum over every 97th element of the foreground result.
namespace
{
enum class Op { kAxpy, kVecAdd };

// kAxpy: y = fma(0.5, x, y) in place (the GPU headline workload scaled down);
// kVecAdd: c = a + b into a third array (the CPU-only configuration: 1000 x 2^20 additions
// in the background, 2^16 every 10 ms in the foreground, window 8 / 4 on both queues).
int Run(Op op, uint64_t bg_n, uint64_t fg_n, int64_t period_us, int samples,
        int bg_threshold, int bg_batch, int fg_threshold, int fg_batch, int bg_burst,
        double *alone_us, double *contended_us,
        uint64_t *bg_commands, double *contended_seconds, uint64_t *checksum)
{
    std::vector<float> bx(bg_n), by(bg_n), fx(fg_n), fy(fg_n);
    std::vector<float> bc(op == Op::kVecAdd ? bg_n : 0), fc(op == Op::kVecAdd ? fg_n : 0);
    oracle_fill_uniform(bx.data(), 0, bg_n, oracle_stream_key(0, 4));
    oracle_fill_uniform(by.data(), 0, bg_n, oracle_stream_key(0, 5));
    oracle_fill_uniform(fx.data(), 0, fg_n, oracle_stream_key(0, 0));
    oracle_fill_uniform(fy.data(), 0, fg_n, oracle_stream_key(0, 1));

    HB_CHECK(XHintSetScheduler(kSchedulerLocal, kPolicyHighestPriorityFirst));
    HwQueueHandle bg_hwq = 0, fg_hwq = 0;
    XQueueHandle bg_xq = 0, fg_xq = 0;
    HB_CHECK(HostQueueCreate(&bg_hwq));
    HB_CHECK(HostQueueCreate(&fg_hwq));
    HB_CHECK(XQueueCreate(&bg_xq, bg_hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    HB_CHECK(XQueueCreate(&fg_xq, fg_hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    HB_CHECK(XQueueSetLaunchConfig(bg_xq, bg_threshold, bg_batch));
    HB_CHECK(XQueueSetLaunchConfig(fg_xq, fg_threshold, fg_batch));
    HB_CHECK(XHintPriority(bg_xq, 1));
    HB_CHECK(XHintPriority(fg_xq, 2));

    auto fg_once = [&]() -> double {
        HwCommandHandle cmd = 0;
        const auto t0 = Clock::now();
        const XResult made = op == Op::kAxpy ? HostAxpyCommandCreate(&cmd, 0.5f, fx.data(), fy.data(), fg_n, 0)
                                             : HostVecAddCommandCreate(&cmd, fx.data(), fy.data(), fc.data(), fg_n, 0);
        if (made != kXSchedSuccess) return -1;
        if (XQueueSubmit(fg_xq, cmd) != kXSchedSuccess) return -1;
        if (XQueueWaitAll(fg_xq) != kXSchedSuccess) return -1;
        return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
    };
    auto run_fg = [&](double *out) {
        auto next = Clock::now();
        for (int i = 0; i < samples; ++i) {
            std::this_thread::sleep_until(next);
            out[i] = fg_once();
            next += std::chrono::microseconds(period_us);
        }
    };

    run_fg(alone_us);

    std::atomic<bool> stop { false };
    std::thread bg_thread([&] {
        while (!stop.load()) {
            for (int n = 0; n < bg_burst && !stop.load(); ++n) {
                HwCommandHandle cmd = 0;
                const XResult made = op == Op::kAxpy ? HostAxpyCommandCreate(&cmd, 0.5f, bx.data(), by.data(), bg_n, 0)
                                                     : HostVecAddCommandCreate(&cmd, bx.data(), by.data(), bc.data(), bg_n, 0);
                if (made != kXSchedSuccess) return;
                if (XQueueSubmit(bg_xq, cmd) != kXSchedSuccess) return;
            }
            XQueueWaitAll(bg_xq);
        }
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(50));
    const auto t0 = Clock::now();
    uint64_t wg0 = 0, wg1 = 0, skipped = 0, replays = 0;
    HostQueueGetStats(bg_hwq, &wg0, &skipped, &replays);
    run_fg(contended_us);
    HostQueueGetStats(bg_hwq, &wg1, &skipped, &replays);
    *contended_seconds = std::chrono::duration<double>(Clock::now() - t0).count();
    // work-groups of 16384 elements (host adapter): commands = work-groups / per-command count
    const uint64_t wg_per_cmd = (bg_n + 16383) / 16384;
    *bg_commands = (wg1 - wg0) / (wg_per_cmd ? wg_per_cmd : 1);
    stop.store(true);
    bg_thread.join();

    uint64_t sum = 0;
    const std::vector<float> &result = op == Op::kAxpy ? fy : fc;
    for (uint64_t i = 0; i < fg_n; i += 97) { uint32_t u; memcpy(&u, &result[i], 4); sum += u; }
    *checksum = sum;

    HB_CHECK(XQueueDestroy(bg_xq));
    HB_CHECK(XQueueDestroy(fg_xq));
    HB_CHECK(HwQueueDestroy(bg_hwq));
    HB_CHECK(HwQueueDestroy(fg_hwq));
    return 0;
}
} // namespace

extern "C" __attribute__((visibility("default")))
int hostbench_run_fg_bg_axpy(uint64_t bg_n, uint64_t fg_n, int64_t period_us, int samples,
                             int bg_threshold, int bg_batch, double *alone_us, double *contended_us,
                             uint64_t *bg_commands, double *contended_seconds, uint64_t *checksum)
{
    return Run(Op::kAxpy, bg_n, fg_n, period_us, samples, bg_threshold, bg_batch, 8, 4, 8, alone_us, contended_us,
               bg_commands, contended_seconds, checksum);
}

// The CPU-only configuration: both queues with the window `threshold` / `batch`, the
// background in streams of `bg_burst` commands. The checksum covers every 97th element of
// the foreground sum a + b.
extern "C" __attribute__((visibility("default")))
int hostbench_run_fg_bg_vecadd(uint64_t bg_n, uint64_t fg_n, int64_t period_us, int samples,
                               int threshold, int batch, int bg_burst, double *alone_us, double *contended_us,
                               uint64_t *bg_commands, double *contended_seconds, uint64_t *checksum)
{
    return Run(Op::kVecAdd, bg_n, fg_n, period_us, samples, threshold, batch, threshold, batch, bg_burst, alone_us,
               contended_us, bg_commands, contended_seconds, checksum);
}
