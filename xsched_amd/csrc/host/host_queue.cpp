// Host (CPU) hardware-queue adapter; see include/xsched/host/hal.h.
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

#include "xsched/host/hal.h"
#include "xsched/xqueue.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/device.h"
#include "xsched/preempt/hal/extensions.h"
#include "xsched/preempt/hal/hw_command.h"
#include "xsched/preempt/hal/hw_queue.h"

using namespace xsched::preempt;
using namespace xsched::protocol;

namespace xsched::host
{

class HostQueue;

/// One launch of a kernel as the executor sees it.
struct Ticket
{
    std::shared_ptr<class HostKernelCommand> cmd;
    uint32_t epoch;   // deactivation count at launch time
    uint64_t seq;     // position in this queue's launch order
};

class HostKernelCommand : public HwCommand, public HwCommandExtension
{
public:
    HostKernelCommand(HostKernelFn fn, void *arg, uint32_t n_wg, bool guarded)
        : HwCommand(guarded ? kCommandPropertyDeactivatable : kCommandPropertyNone)
        , fn_(fn), arg_(arg), n_wg_(n_wg), done_((n_wg + 31) / 32) {}

    virtual void Synchronize() override
    {
        XASSERT(marked_, "Synchronize() needs EnableSynchronization() before launch");
        std::unique_lock<std::mutex> lock(mtx_);
        // Returns when the latest launch of this command has been retired by the
        // executor - fully executed or flushed.
        cv_.wait(lock, [this]() { return retired_launches_ == launches_; });
    }
    virtual bool Synchronizable() override { return marked_; }
    virtual bool EnableSynchronization() override { marked_ = true; return true; }
    // Launching is handing a ticket to the executor thread: any thread may do it.
    virtual bool DirectLaunchable() override { return true; }
    virtual bool CompletedWithoutWaiting() override
    {
        std::lock_guard<std::mutex> lock(mtx_);
        return marked_ && launches_ != 0 && retired_launches_ == launches_;
    }

    bool Finished() const
    {
        return n_done_.load(std::memory_order_acquire) == n_wg_;
    }

private:
    friend class HostQueue;
    const HostKernelFn fn_;
    void * const arg_;
    const uint32_t n_wg_;
    std::vector<uint32_t> done_;           // 1 bit per work-group, executor-owned
    std::atomic<uint32_t> n_done_ { 0 };
    bool marked_ = false;

    std::mutex mtx_;
    std::condition_variable cv_;
    uint64_t launches_ = 0;
    uint64_t retired_launches_ = 0;
};

class HostQueue : public HwQueue, public HwQueueExtension
{
public:
    HostQueue(): handle_(NextHandle())
    {
        thread_ = std::thread([this]() { this->Executor(); });
    }

    virtual ~HostQueue()
    {
        { std::lock_guard<std::mutex> lock(mtx_); stop_ = true; }
        cv_.notify_all();
        thread_.join();
    }

    virtual void Launch(std::shared_ptr<HwCommand> hw_cmd) override
    {
        auto cmd = std::dynamic_pointer_cast<HostKernelCommand>(hw_cmd);
        XASSERT(cmd != nullptr, "hw_cmd is not a HostKernelCommand");
        Enqueue(std::move(cmd));
    }

    virtual void Synchronize() override
    {
        std::unique_lock<std::mutex> lock(mtx_);
        const uint64_t target = launched_;
        drained_cv_.wait(lock, [&]() { return retired_ >= target; });
    }

    // Level 2: bump the preempt word. Tickets launched under an older epoch are
    // skipped work-group by work-group from now on.
    virtual void Deactivate() override { epoch_.fetch_add(1, std::memory_order_acq_rel); }

    // Replay, in order, every logged kernel that is deactivatable and unfinished.
    // Commands without the property ran to completion (the launch thread never
    // puts one behind an in-flight deactivatable command) and are left alone.
    virtual void Reactivate(const CommandLog &log) override
    {
        for (auto &hw_cmd : log) {
            auto cmd = std::dynamic_pointer_cast<HostKernelCommand>(hw_cmd);
            if (cmd == nullptr || !cmd->GetProps(kCommandPropertyDeactivatable)) continue;
            if (cmd->Finished()) continue;
            replays_.fetch_add(1, std::memory_order_relaxed);
            Enqueue(std::move(cmd));
        }
    }

    virtual XDevice GetDevice() override { return MakeDevice(kDeviceTypeCPU, 0); }
    virtual HwQueueHandle GetHandle() override { return handle_; }
    virtual bool SupportDynamicLevel() override { return true; }
    virtual XPreemptLevel GetMaxSupportedLevel() override { return kPreemptLevelDeactivate; }
    virtual void OnPreemptLevelChange(XPreemptLevel level) override { level_ = level; }
    virtual bool SupportDirectLaunch() override { return true; }
    virtual bool DeactivationConcernsInFlightWorkOnly() override { return true; }

    void GetStats(uint64_t *executed, uint64_t *skipped, uint64_t *replays) const
    {
        if (executed) *executed = wg_executed_.load();
        if (skipped)  *skipped = wg_skipped_.load();
        if (replays)  *replays = replays_.load();
    }

private:
    static HwQueueHandle NextHandle()
    {
        static std::atomic<uint64_t> next { 1 };
        return (0x484F5354ull << 32) | next.fetch_add(1); // "HOST" | serial
    }

    void Enqueue(std::shared_ptr<HostKernelCommand> cmd)
    {
        {
            std::lock_guard<std::mutex> cl(cmd->mtx_);
            cmd->launches_ += 1;
        }
        {
            std::lock_guard<std::mutex> lock(mtx_);
            const uint32_t epoch = epoch_.load(std::memory_order_acquire);
            tickets_.push_back(Ticket { std::move(cmd), epoch, ++launched_ });
        }
        cv_.notify_one();
    }

    void Executor()
    {
        while (true) {
            Ticket t;
            {
                std::unique_lock<std::mutex> lock(mtx_);
                cv_.wait(lock, [this]() { return stop_ || !tickets_.empty(); });
                if (tickets_.empty()) return; // stop_ and drained
                t = std::move(tickets_.front());
                tickets_.pop_front();
            }
            Run(t);
            {
                std::lock_guard<std::mutex> cl(t.cmd->mtx_);
                t.cmd->retired_launches_ += 1;
            }
            t.cmd->cv_.notify_all();
            {
                std::lock_guard<std::mutex> lock(mtx_);
                retired_ = t.seq;
            }
            drained_cv_.notify_all();
        }
    }

    // The guard: a deactivatable kernel looks at the preempt word before each
    // work-group; a work-group that has started always finishes and records
    // itself in the bitmap, so a replay runs exactly the missing ones.
    void Run(const Ticket &t)
    {
        HostKernelCommand &k = *t.cmd;
        const bool guarded = k.GetProps(kCommandPropertyDeactivatable) != 0;
        for (uint32_t wg = 0; wg < k.n_wg_; ++wg) {
            const uint32_t word = wg >> 5, bit = 1u << (wg & 31);
            if (k.done_[word] & bit) continue; // finished by an earlier launch
            if (guarded && epoch_.load(std::memory_order_acquire) != t.epoch) {
                wg_skipped_.fetch_add(1, std::memory_order_relaxed);
                continue;
            }
            k.fn_(k.arg_, wg, k.n_wg_);
            k.done_[word] |= bit;
            k.n_done_.fetch_add(1, std::memory_order_release);
            wg_executed_.fetch_add(1, std::memory_order_relaxed);
        }
    }

    const HwQueueHandle handle_;
    XPreemptLevel level_ = kPreemptLevelUnknown;

    std::mutex mtx_;
    std::condition_variable cv_, drained_cv_;
    std::deque<Ticket> tickets_;
    uint64_t launched_ = 0, retired_ = 0;
    bool stop_ = false;
    std::thread thread_;

    std::atomic<uint32_t> epoch_ { 0 };
    std::atomic<uint64_t> wg_executed_ { 0 }, wg_skipped_ { 0 }, replays_ { 0 };
};

// ---- built-in host kernels ---------------------------------------------------

constexpr size_t kWgElems = 16384;

struct VecArgs
{
    float alpha;
    const float *a;
    const float *b;
    float *c;
    size_t n;
};

/// Owns its argument block.
class OwningKernelCommand : public HostKernelCommand
{
public:
    OwningKernelCommand(HostKernelFn fn, std::unique_ptr<VecArgs> args, uint32_t n_wg, bool guarded)
        : HostKernelCommand(fn, args.get(), n_wg, guarded), args_(std::move(args)) {}
private:
    std::unique_ptr<VecArgs> args_;
};

static void VecAddWg(void *p, uint32_t wg, uint32_t)
{
    const VecArgs &v = *(const VecArgs *)p;
    const size_t lo = (size_t)wg * kWgElems, hi = std::min(v.n, lo + kWgElems);
    for (size_t i = lo; i < hi; ++i) v.c[i] = v.a[i] + v.b[i];
}

static void AxpyWg(void *p, uint32_t wg, uint32_t)
{
    const VecArgs &v = *(const VecArgs *)p;
    const size_t lo = (size_t)wg * kWgElems, hi = std::min(v.n, lo + kWgElems);
    // One rounding per element (fused multiply-add), like the device kernel.
    for (size_t i = lo; i < hi; ++i) v.c[i] = std::fmaf(v.alpha, v.a[i], v.c[i]);
}

} // namespace xsched::host

using namespace xsched::host;

EXPORT_C_FUNC XResult HostQueueCreate(HwQueueHandle *hwq)
{
    if (hwq == nullptr) return kXSchedErrorInvalidValue;
    auto q = std::make_shared<HostQueue>();
    const HwQueueHandle h = q->GetHandle();
    XResult res = HwQueueManager::Add(h, [&]() { return q; });
    if (res == kXSchedSuccess) *hwq = h;
    return res;
}

EXPORT_C_FUNC XResult HostKernelCommandCreate(HwCommandHandle *cmd, HostKernelFn fn, void *arg,
                                              uint32_t n_wg, int guarded)
{
    if (cmd == nullptr || fn == nullptr) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HostKernelCommand>(fn, arg, n_wg, guarded != 0));
    return kXSchedSuccess;
}

static XResult MakeVecCommand(HwCommandHandle *cmd, HostKernelFn fn, float alpha, const float *a,
                              const float *b, float *c, size_t n, int guarded)
{
    if (cmd == nullptr || a == nullptr || c == nullptr) return kXSchedErrorInvalidValue;
    auto args = std::make_unique<VecArgs>(VecArgs { alpha, a, b, c, n });
    const uint32_t n_wg = (uint32_t)((n + kWgElems - 1) / kWgElems);
    *cmd = HwCommandManager::Add(
        std::make_shared<OwningKernelCommand>(fn, std::move(args), n_wg, guarded != 0));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HostVecAddCommandCreate(HwCommandHandle *cmd, const float *a, const float *b,
                                              float *c, size_t n, int guarded)
{
    if (b == nullptr) return kXSchedErrorInvalidValue;
    return MakeVecCommand(cmd, VecAddWg, 0.f, a, b, c, n, guarded);
}

EXPORT_C_FUNC XResult HostAxpyCommandCreate(HwCommandHandle *cmd, float alpha, const float *x,
                                            float *y, size_t n, int guarded)
{
    return MakeVecCommand(cmd, AxpyWg, alpha, x, nullptr, y, n, guarded);
}

EXPORT_C_FUNC XResult HostQueueGetStats(HwQueueHandle hwq, uint64_t *wg_executed,
                                        uint64_t *wg_skipped, uint64_t *replays)
{
    auto q = std::dynamic_pointer_cast<HostQueue>(HwQueueManager::Get(hwq));
    if (q == nullptr) return kXSchedErrorNotFound;
    q->GetStats(wg_executed, wg_skipped, replays);
    return kXSchedSuccess;
}
