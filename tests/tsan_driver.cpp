// Host-side concurrency under ThreadSanitizer. This program is compiled TOGETHER with the
// XQueue core, the scheduler and the host adapter (their sources, not the shared libraries)
// with -fsanitize=thread by tests/test_tsan.py, and drives them through the public C API
// from several threads at once:
//   1. sparse submissions that are launched on the submitting thread and waited for on it,
//      while another thread suspends and resumes the level-2 queue at random;
//   2. two threads submitting bursts into one queue, a third one waiting;
//   3. the CPU-only configuration in small: background and foreground queues under the local
//      scheduler with the highest-priority-first policy (scheduler thread, two launcher
//      threads, two executor threads, two submitters);
//   4. launch-configuration and level changes between bursts, and destroying a queue that is
//      suspended with work queued;
//   5. a LocalScheduler of its own whose rounds run on the threads that bring the events (the
//      daemon's arrangement): four threads report queues ready and idle, a fifth one switches
//      the policy back and forth, the round thread keeps the laxity policy's alarms.
// Every guarded work-group must have taken effect exactly once. The sanitizer's verdict is
// its exit code and stderr; this program only checks the counts.
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "xsched/hint.h"
#include "xsched/xqueue.h"
#include "xsched/sched/protocol/event.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/scheduler/local.h"
#include "xsched/host/bench.h"
#include "xsched/host/hal.h"

#define CHECK_X(call) do { XResult r_ = (call); if (r_ != kXSchedSuccess) { \
    fprintf(stderr, "%s:%d: %s -> %d\n", __FILE__, __LINE__, #call, (int)r_); exit(3); } } while (0)

namespace
{

struct Counters { std::vector<std::atomic<uint32_t>> hits; explicit Counters(size_t n): hits(n) {} };

void CountWorkGroup(void *arg, uint32_t wg, uint32_t)
{
    auto *c = (Counters *)arg;
    c->hits[wg].fetch_add(1, std::memory_order_relaxed);
    for (int spin = 0; spin < 200; ++spin) asm volatile("" ::: "memory");
}

void Submit(XQueueHandle xq, Counters &c, uint32_t n_wg, int guarded)
{
    HwCommandHandle cmd = 0;
    CHECK_X(HostKernelCommandCreate(&cmd, CountWorkGroup, &c, n_wg, guarded));
    CHECK_X(XQueueSubmit(xq, cmd));
}

bool AllEqual(const Counters &c, uint32_t want)
{
    for (auto &h : c.hits) if (h.load() != want) return false;
    return true;
}

int SparseSubmissionsUnderChurn()
{
    CHECK_X(XHintSetScheduler(kSchedulerAppManaged, kPolicyUnknown));
    HwQueueHandle hwq = 0; XQueueHandle xq = 0;
    CHECK_X(HostQueueCreate(&hwq));
    CHECK_X(XQueueCreate(&xq, hwq, kPreemptLevelDeactivate, kQueueCreateFlagNone));
    CHECK_X(XQueueSetLaunchConfig(xq, 4, 2));
    Counters c(64);
    std::atomic<bool> stop { false };
    std::thread churn([&]() {
        uint64_t lcg = 12345;
        while (!stop.load()) {
            lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
            std::this_thread::sleep_for(std::chrono::microseconds(50 + (lcg >> 33) % 300));
            CHECK_X(XQueueSuspend(xq, (lcg >> 20) & 1 ? kQueueSuspendFlagSyncHwQueue : kQueueSuspendFlagNone));
            std::this_thread::sleep_for(std::chrono::microseconds(20 + (lcg >> 40) % 100));
            CHECK_X(XQueueResume(xq, kQueueResumeFlagNone));
        }
    });
    const uint32_t rounds = 400;
    for (uint32_t i = 0; i < rounds; ++i) {
        Submit(xq, c, 64, 1);
        if (i % 3 == 0) Submit(xq, c, 64, 1);
        CHECK_X(XQueueWaitAll(xq));
        if (i % 16 == 0) std::this_thread::sleep_for(std::chrono::microseconds(300));
    }
    stop.store(true);
    churn.join();
    CHECK_X(XQueueWaitAll(xq));
    const uint32_t want = rounds + (rounds + 2) / 3;
    const bool ok = AllEqual(c, want);
    CHECK_X(XQueueDestroy(xq));
    CHECK_X(HwQueueDestroy(hwq));
    printf("sparse submissions under churn: %s (want %u per work-group)\n", ok ? "ok" : "WRONG COUNTS", want);
    return ok ? 0 : 1;
}

int TwoSubmittersOneWaiter()
{
    HwQueueHandle hwq = 0; XQueueHandle xq = 0;
    CHECK_X(HostQueueCreate(&hwq));
    CHECK_X(XQueueCreate(&xq, hwq, kPreemptLevelBlock, kQueueCreateFlagNone));
    CHECK_X(XQueueSetLaunchConfig(xq, 8, 4));
    Counters c(16);
    std::atomic<int> live { 2 };
    auto submitter = [&]() {
        for (int burst = 0; burst < 60; ++burst) {
            for (int i = 0; i < 5; ++i) Submit(xq, c, 16, 0);
            std::this_thread::sleep_for(std::chrono::microseconds(100));
        }
        live.fetch_sub(1);
    };
    std::thread a(submitter), b(submitter);
    std::thread waiter([&]() { while (live.load() > 0) { CHECK_X(XQueueWaitAll(xq)); XQueueState st; CHECK_X(XQueueQuery(xq, &st)); } });
    a.join(); b.join(); waiter.join();
    CHECK_X(XQueueWaitAll(xq));
    const bool ok = AllEqual(c, 2 * 60 * 5);
    // configuration changes between bursts, then destruction while suspended with work queued
    CHECK_X(XQueueSetLaunchConfig(xq, 2, 1));
    CHECK_X(XQueueSetPreemptLevel(xq, kPreemptLevelDeactivate));
    for (int i = 0; i < 10; ++i) Submit(xq, c, 16, 1);
    CHECK_X(XQueueSuspend(xq, kQueueSuspendFlagNone));
    for (int i = 0; i < 10; ++i) Submit(xq, c, 16, 1);
    CHECK_X(XQueueDestroy(xq));          // resumes, waits, stops the launcher
    CHECK_X(HwQueueDestroy(hwq));
    const bool ok2 = AllEqual(c, 2 * 60 * 5 + 20);
    printf("two submitters, one waiter: %s; destroyed while suspended: %s\n", ok ? "ok" : "WRONG COUNTS", ok2 ? "ok" : "WRONG COUNTS");
    return ok && ok2 ? 0 : 1;
}

int SchedulerWithTwoQueues()
{
    const uint64_t bg_n = 1 << 14, fg_n = 1 << 10;
    std::vector<float> ba(bg_n), bb(bg_n), bc(bg_n), fa(fg_n), fb(fg_n), fc(fg_n);
    HostBenchFillUniform(ba.data(), 0, bg_n, 0, 4); HostBenchFillUniform(bb.data(), 0, bg_n, 0, 5);
    HostBenchFillUniform(fa.data(), 0, fg_n, 0, 0); HostBenchFillUniform(fb.data(), 0, fg_n, 0, 1);
    HostBenchConfig cfg { bg_n, fg_n, 50, 8, 4, 80, 500 };
    std::vector<double> alone(80), cont(80);
    HostBenchResult res {};
    CHECK_X(HostBenchRunVecAdd(&cfg, ba.data(), bb.data(), bc.data(), fa.data(), fb.data(), fc.data(), alone.data(), cont.data(), &res));
    bool ok = res.bg_commands > 0;
    for (uint64_t i = 0; i < fg_n; ++i) ok = ok && fc[i] == fa[i] + fb[i];
    for (uint64_t i = 0; i < bg_n; ++i) ok = ok && bc[i] == ba[i] + bb[i];
    printf("local scheduler, two queues: %s (%llu background commands)\n", ok ? "ok" : "WRONG", (unsigned long long)res.bg_commands);
    return ok ? 0 : 1;
}

int RoundsOnTheCallersThreads()
{
    using namespace xsched::sched;
    LocalScheduler sched(kPolicyHighestPriorityFirst);
    std::atomic<uint64_t> operations { 0 }, suspended_seen { 0 };
    sched.SetExecutor([&](std::shared_ptr<const Operation> op) {
        operations.fetch_add(1);
        if (op->Type() == kOperationSched) {
            auto *so = static_cast<const SchedOperation *>(op.get());
            suspended_seen.fetch_add(so->SuspendedCnt());
        }
    });
    sched.RunRoundsOnCallers(LocalScheduler::kRoundsOnCallersAll);
    sched.Run();
    const PID pid = GetProcessId();
    sched.RecvEvent(std::make_shared<ProcessCreateEvent>("tsan_driver"));
    constexpr int kQueues = 4, kTurns = 600;
    for (int q = 0; q < kQueues; ++q) {
        const XQueueHandle h = 0x1000 + (XQueueHandle)q;
        sched.RecvEvent(std::make_shared<XQueueCreateEvent>(h, (XDevice)1, kPreemptLevelBlock, 16, 8));
        sched.RecvEvent(std::make_shared<HintEvent>(std::make_shared<PriorityHint>(h, (Priority)q)));
        sched.RecvEvent(std::make_shared<HintEvent>(std::make_shared<LaxityHint>(h, (Laxity)200, (Priority)0, (Priority)(q + 1))));
    }
    std::vector<std::thread> reporters;
    for (int q = 0; q < kQueues; ++q) {
        reporters.emplace_back([&, q]() {
            const XQueueHandle h = 0x1000 + (XQueueHandle)q;
            for (int i = 0; i < kTurns; ++i) {
                sched.RecvEvent(std::make_shared<XQueueReadyEvent>(h, std::chrono::system_clock::now()));
                std::this_thread::sleep_for(std::chrono::microseconds(20 + 13 * q));
                sched.RecvEvent(std::make_shared<XQueueIdleEvent>(h));
            }
        });
    }
    std::thread switcher([&]() {
        for (int i = 0; i < 12; ++i) {
            std::this_thread::sleep_for(std::chrono::milliseconds(3));
            sched.SetPolicy(i % 2 ? kPolicyHighestPriorityFirst : kPolicyLaxity);
        }
    });
    for (auto &t : reporters) t.join();
    switcher.join();
    for (int q = 0; q < kQueues; ++q) sched.RecvEvent(std::make_shared<XQueueDestroyEvent>(0x1000 + (XQueueHandle)q));
    sched.Stop();
    (void)pid;
    const bool ok = operations.load() >= (uint64_t)kQueues * kTurns && suspended_seen.load() > 0;
    printf("rounds on the callers' threads: %s (%llu operations)\n", ok ? "ok" : "TOO FEW OPERATIONS",
           (unsigned long long)operations.load());
    return ok ? 0 : 1;
}

} // namespace

int main()
{
    setenv("XLOG_LEVEL", "ERRO", 0);
    int bad = 0;
    bad += SparseSubmissionsUnderChurn();
    bad += TwoSubmittersOneWaiter();
    bad += SchedulerWithTwoQueues();
    bad += RoundsOnTheCallersThreads();
    printf("%s\n", bad ? "FAILED" : "done");
    return bad ? 1 : 0;
}
