// RingXQueue: the preemptible command queue between XQueueSubmit() and a hardware adapter.
//
// One object, two rings, one launcher thread:
//
//   submitters --> [submission ring] --> launcher thread --> HwQueue::Launch()
//                                              |
//                                       [in-flight window]  <-- waiters retire from here
//
// The submission ring is a preallocated circular array of shared_ptr slots (it doubles when
// it runs full, so a suspended queue never blocks a submitter); nothing is allocated per
// command. The in-flight window is a second circular array, never longer than `threshold`:
// the commands handed to the adapter and not yet known complete. Every `batch`-th command
// carries a completion marker; when the window is full the launcher waits for the oldest
// marker, so a suspended queue leaves at most `threshold` commands behind on the device.
//
// Completion is tracked by ONE monotonic number, the index of the newest command known
// complete (`retired_`). XQueueWaitAll takes the index of the last submission as its ticket
// and waits for that number to reach it; no marker object is built for it. With an adapter
// that lets any thread launch and synchronise (HwQueueExtension::SupportDirectLaunch) the submitter
// launches a command itself when the launcher is parked on an empty ring, and a waiter whose
// commands have all been launched waits for the device itself; the launcher is only woken,
// off the caller's path, to run the drain sequence that ends in the Idle event.
//
// What the adapter and the scheduler observe (which command carries a marker, what is
// synchronised when, what Reactivate() is handed, when Ready / Idle are reported) is that of
// reference preempt/src/xqueue/{async_xqueue,command_buffer,launch_worker}.cpp; the traces of
// that code over a recording adapter are the specification this class is tested against.
#pragma once

#include <atomic>
#include <condition_variable>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "xsched/protocol/def.h"
#include "xsched/preempt/hal/extensions.h"
#include "xsched/preempt/xqueue/xqueue.h"

namespace xsched::preempt
{

class RingXQueue final : public XQueue
{
public:
    RingXQueue(std::shared_ptr<HwQueue> hwq, XPreemptLevel level,
               int64_t threshold = XSCHED_DEFAULT_COMMAND_THRESHOLD,
               int64_t batch = XSCHED_DEFAULT_COMMAND_BATCH_SIZE);
    ~RingXQueue() override;

    void Submit(std::shared_ptr<HwCommand> hw_cmd) override;
    std::shared_ptr<XQueueWaitAllCommand> SubmitWaitAll() override;
    void WaitAll() override;
    void Wait(std::shared_ptr<HwCommand> hw_cmd) override;
    XQueueState Query() override;
    int64_t GetHwCommandCount() override { return next_idx_.load(std::memory_order_acquire) - 1; }
    /// Commands launched on a submitting thread so far (not part of the XQueue interface).
    int64_t GetDirectLaunchCount() const { return direct_launches_.load(std::memory_order_relaxed); }

    void Suspend(int64_t flags) override;
    void Resume(int64_t flags) override;
    void SetPreemptLevel(XPreemptLevel level) override;
    void SetLaunchConfig(int64_t threshold, int64_t batch) override;

private:
    using Guard = std::unique_lock<std::mutex>;

    // ---- submission ring (ring_mu_) ---------------------------------------------------
    enum class Slot : uint8_t { kCommand, kDrain, kStop };
    struct Pending
    {
        Slot kind = Slot::kCommand;
        std::shared_ptr<XCommand> cmd; // kCommand: the HwCommand; kDrain: an optional marker object
    };
    /// What the launcher still owes once the ring is empty: after work, a wait for the oldest
    /// marked batch; after that, a wait for the whole hardware queue; after that, nothing.
    enum class Owed : uint8_t { kBatchThenDrain, kDrain, kNothing };
    enum class Step : uint8_t { kLaunch, kDrain, kBatch, kStop };

    void PushLocked(Slot kind, std::shared_ptr<XCommand> cmd);
    Step NextStep(Pending *out);
    void DiscardPending();
    void WaitForIdle();
    /// Pushes a drain slot unless one already closes the ring; returns the ticket (index of
    /// the last submission) or -1 when the queue is idle.
    int64_t RequestDrain(std::shared_ptr<XCommand> marker);

    std::mutex ring_mu_;
    std::condition_variable ring_cv_;   // the launcher parks here
    std::condition_variable idle_cv_;
    std::vector<Pending> ring_;         // capacity is a power of two
    size_t ring_head_ = 0, ring_count_ = 0;
    Owed owed_ = Owed::kNothing;
    bool parked_ = false;
    bool caller_launched_ = false;      // a submitter has launched since the launcher last stood by
    int64_t unwaited_submits_ = 0;      // submissions since anybody last asked for a drain
    XQueueState reported_ = kQueueStateIdle;
    bool ready_unsent_ = false;         // reported_ turned Ready, the event is still with the submitter
    bool idle_held_back_ = false;       // the launcher found the queue idle meanwhile and waits for that event to be out
    uint64_t idle_round_ = 0;

    // ---- in-flight window (win_mu_) ---------------------------------------------------
    struct Flight
    {
        std::shared_ptr<HwCommand> cmd;
        int64_t idx = 0;
        bool marked = false;     // carries a completion marker
        bool flushable = false;  // a deactivation may flush it
    };
    enum class Run : uint8_t { kRunning, kPaused, kStopped };

    Flight &At(size_t i) { return window_[(win_head_ + i) & (window_.size() - 1)]; }
    void ResizeWindow(int64_t threshold);
    void LauncherMain();
    void LaunchFromRing(std::shared_ptr<HwCommand> cmd);
    bool TryLaunchOnCaller(const std::shared_ptr<HwCommand> &cmd, bool mark);
    void HandOver(const std::shared_ptr<HwCommand> &cmd, bool mark = false);   // win_mu_ held
    bool MustDrainFlushablesFirst(const HwCommand &cmd, std::shared_ptr<HwCommand> *marker);
    std::shared_ptr<HwCommand> OldestMarker();
    bool HoldWhilePaused(Guard &g);                                // false: stopped
    void AwaitQueue(Guard &g);                                     // whole hardware queue
    void AwaitMarker(Guard &g, const std::shared_ptr<HwCommand> &marker);
    void RetireThrough(int64_t idx);
    void RetireEverything();
    void PublishRetired(int64_t idx);
    void AwaitRetired(int64_t ticket);
    CommandLog InFlightLog();

    std::mutex win_mu_;
    std::condition_variable win_cv_;
    std::vector<Flight> window_;        // capacity is a power of two >= threshold_
    size_t win_head_ = 0, win_count_ = 0;
    Run run_ = Run::kRunning;
    int64_t pauses_ = 0;                // grows with every Pause: a device wait that spans one proves nothing
    int64_t threshold_, batch_;
    int64_t last_marked_idx_ = -1;
    int64_t drop_through_ = -1;         // commands up to this index complete without launching
    bool queue_wait_active_ = false;    // some thread is waiting for the whole hardware queue

    bool lazy_deactivation_ = false;           // the adapter's Deactivate() concerns in-flight launches only
    std::atomic<bool> deactivated_ { false };  // the current suspension did call Deactivate()

    std::atomic<int64_t> next_idx_ { 1 };
    std::atomic<int64_t> handed_over_ { 0 };   // newest index launched or dropped
    std::atomic<int64_t> retired_ { 0 };       // newest index known complete
    std::atomic<int64_t> direct_launches_ { 0 };

    XPreemptLevel level_;
    bool caller_may_launch_ = false;
    std::atomic_bool suspended_ { false };
    std::atomic_bool closing_ { false };
    std::thread launcher_;
};

} // namespace xsched::preempt
