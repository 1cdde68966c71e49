// RingXQueue, see ring_queue.h. Behaviour pinned by the adapter traces of reference
// preempt/src/xqueue/{async_xqueue,command_buffer,launch_worker}.cpp (citations below name
// the rule each block keeps).
#include <chrono>
#include <typeinfo>

#include <sys/prctl.h>

#include "ring_queue.h"
#include "xsched/utils/env.h"
#include "xsched/utils/xassert.h"
#include "agent.h"

using namespace xsched::sched;

namespace xsched::preempt
{

namespace
{
constexpr size_t kInitialRingSlots = 256;
constexpr int64_t kSpinMicros = 150; // a waiter polls this long before it sleeps
constexpr int64_t kDirectBurst = 8;           // submissions in a row without a wait that are still launched by the submitter
constexpr int64_t kStandByMicros = 500;      // how long the launcher leaves the device to callers that launch themselves
constexpr int64_t kStandBySliceMicros = 25;  // how often it looks whether their commands have retired
constexpr unsigned long kLauncherTimerSlackNanos = 1000; // timed waits of the launcher end on time (the default slack is 50 us)

size_t PowerOfTwoAtLeast(size_t n)
{
    size_t p = 1;
    while (p < n) p <<= 1;
    return p;
}
} // namespace

RingXQueue::RingXQueue(std::shared_ptr<HwQueue> hwq, XPreemptLevel level, int64_t threshold, int64_t batch)
    : XQueue(kXQueueImplTypeAsync,
             kQueueFeatureAsyncSubmit | kQueueFeatureDynamicThreshold | kQueueFeatureDynamicBatchSize |
             kQueueFeatureSyncSuspend | kQueueFeatureResumeDropCommands |
             (hwq->SupportDynamicLevel() ? kQueueFeatureDynamicLevel : 0),
             hwq)
    , ring_(kInitialRingSlots), threshold_(threshold), batch_(batch), level_(level)
{
    XASSERT(level_ > kPreemptLevelUnknown && level_ < kPreemptLevelMax, "invalid preempt level: %d", level_);
    // With fewer window slots than the marker period the window could fill up without a
    // single marker in it to wait for.
    XASSERT(threshold_ >= batch_, "threshold must not be smaller than command batch size");
    ResizeWindow(threshold_);
    // What the adapter offers beyond the reference's contract, if anything.
    auto *ext = dynamic_cast<HwQueueExtension *>(hwq.get());
    caller_may_launch_ = ext != nullptr && ext->SupportDirectLaunch() && GetEnvOption(XSCHED_DIRECT_LAUNCH_ENV_NAME, true);
    lazy_deactivation_ = ext != nullptr && ext->DeactivationConcernsInFlightWorkOnly();

    // The adapter binds its device to the launcher thread before anything else runs there;
    // the constructor returns once that has happened (async_xqueue.cpp:25-29).
    std::atomic<bool> up { false };
    launcher_ = std::thread([this, &up]() {
        (void)prctl(PR_SET_TIMERSLACK, kLauncherTimerSlackNanos, 0, 0, 0);
        kHwQueue->OnXQueueCreate();
        up.store(true, std::memory_order_release);
        up.notify_all();
        LauncherMain();
    });
    up.wait(false, std::memory_order_acquire);
    kHwQueue->OnPreemptLevelChange(level_);
    SchedAgent::SendEvent(std::make_shared<XQueueCreateEvent>(kHandle, kDevice, level_, threshold_, batch_));
}

RingXQueue::~RingXQueue()
{
    // From here on Suspend() does nothing; what is still queued is dropped, what is in flight
    // is waited for by the launcher before it leaves (async_xqueue.cpp:32-42).
    closing_.store(true);
    Resume(kQueueResumeFlagDropCommands);
    {
        Guard g(ring_mu_);
        PushLocked(Slot::kStop, nullptr);
    }
    ring_cv_.notify_one();
    launcher_.join();
    SchedAgent::SendEvent(std::make_shared<XQueueDestroyEvent>(kHandle));
}

// ---- submission ring ---------------------------------------------------------------------

void RingXQueue::PushLocked(Slot kind, std::shared_ptr<XCommand> cmd)
{
    if (ring_count_ == ring_.size()) {
        // Full: double it, oldest entry first. Submitters never block on a queue that is
        // suspended or slow.
        std::vector<Pending> bigger(ring_.size() * 2);
        for (size_t i = 0; i < ring_count_; ++i) bigger[i] = std::move(ring_[(ring_head_ + i) & (ring_.size() - 1)]);
        ring_.swap(bigger);
        ring_head_ = 0;
    }
    Pending &slot = ring_[(ring_head_ + ring_count_) & (ring_.size() - 1)];
    slot.kind = kind;
    slot.cmd = std::move(cmd);
    ring_count_++;
}

void RingXQueue::Submit(std::shared_ptr<HwCommand> hw_cmd)
{
    XASSERT(hw_cmd != nullptr, "hw_cmd should not be nullptr");
    hw_cmd->OnSubmit(shared_from_this());
    hw_cmd->SetIdx(next_idx_.fetch_add(1, std::memory_order_acq_rel));
    kHwQueue->OnHwCommandSubmit(hw_cmd);
    const bool wait_for_launch = hw_cmd->GetProps(kCommandPropertyBlockingSubmit) != 0;
    hw_cmd->SetState(kCommandStatePending);

    // The Ready event either goes out first, under the ring lock (daemon client: one
    // datagram), or after the launch and with no lock of this queue held (in-process: it may
    // run a scheduling round on this thread, which suspends, deactivates and replays other
    // queues; meanwhile this queue's launcher, its other submitters and waiters go on).
    // (command_buffer.cpp:107-110 sends it under its lock, the scheduler there is always
    // another thread.)
    const bool event_first = SchedAgent::ReadyEventGoesFirst();
    std::shared_ptr<XQueueReadyEvent> ready_event;
    bool wake, launched;
    {
        Guard g(ring_mu_);
        if (reported_ == kQueueStateIdle) {
            reported_ = kQueueStateReady;
            ready_event = std::make_shared<XQueueReadyEvent>(kHandle, std::chrono::system_clock::now());
            if (event_first) {
                SchedAgent::SendEvent(ready_event);
                ready_event = nullptr;
            } else {
                // Ready and Idle reach the scheduler in the order in which they happened:
                // the launcher reports no Idle while this Ready is still to be sent.
                ready_unsent_ = true;
            }
        }
        const bool launcher_owed_nothing = owed_ == Owed::kNothing;
        owed_ = Owed::kBatchThenDrain;
        // The launcher is parked and nothing waits in the ring: launching here keeps
        // submission order, and the ring lock keeps it so against other submitters.
        // A submitter that waits for what it submits wants the launch at once, on its own
        // thread. One that keeps submitting without waiting (a framework issuing kernel after
        // kernel) is better off handing the launches to the launcher, which makes them on
        // another core while the submitter goes on: after kDirectBurst submissions with no
        // wait in between, the ring it is.
        const bool streaming = ++unwaited_submits_ > kDirectBurst;
        // The first submission after a wait (or a query) is most likely waited for in its turn:
        // launched here it gets a marker whatever the batch count says, recorded right behind
        // it, and the wait that follows needs no marker of its own.
        launched = caller_may_launch_ && !streaming && parked_ && ring_count_ == 0 &&
                   TryLaunchOnCaller(hw_cmd, unwaited_submits_ == 1);
        if (launched) caller_launched_ = true;
        else PushLocked(Slot::kCommand, wait_for_launch ? hw_cmd : std::move(hw_cmd));
        // A launcher that already stands by for callers (see NextStep) needs no wake-up for a
        // command that is on the device already; it looks again by itself.
        wake = parked_ && (!launched || launcher_owed_nothing);
    }
    // A command in the ring needs the launcher now; one that is on the device already needs
    // it only for the drain that ends in the Idle event, so the scheduler hears first.
    if (wake && !launched) ring_cv_.notify_one();
    if (ready_event != nullptr) {
        SchedAgent::SendEvent(ready_event);
        bool idle_waits;
        {
            Guard g(ring_mu_);
            ready_unsent_ = false;
            idle_waits = idle_held_back_;
        }
        if (idle_waits && !(wake && launched)) ring_cv_.notify_one();
    }
    if (wake && launched) ring_cv_.notify_one();
    if (wait_for_launch) hw_cmd->WaitUntil(kCommandStateInFlight);
}

// What the launcher does next. With an empty ring it first owes a wait for the oldest marked
// batch, then a wait for the whole hardware queue, and only when that has returned with the
// ring still empty does the queue count as idle (command_buffer.cpp:39-97).
RingXQueue::Step RingXQueue::NextStep(Pending *out)
{
    Guard g(ring_mu_);
    while (true) {
        if (ring_count_ != 0) {
            Pending &slot = ring_[ring_head_];
            out->kind = slot.kind;
            out->cmd = std::move(slot.cmd);
            ring_head_ = (ring_head_ + 1) & (ring_.size() - 1);
            ring_count_--;
            switch (out->kind) {
            case Slot::kCommand: return Step::kLaunch;
            case Slot::kDrain:   return Step::kDrain;
            case Slot::kStop:    return Step::kStop;
            }
        }
        out->cmd = nullptr;
        if (owed_ != Owed::kNothing && caller_launched_) {
            // Callers launch and wait for themselves: the launcher stands by, still parked as
            // far as submitters are concerned, until what they launched has retired (then the
            // waits it owes return at once), something is queued for it, or the stand-by has
            // lasted long enough that nobody seems to be waiting. It does not ask the device
            // meanwhile: a second thread polling the runtime slows the callers' launches.
            // Only for launches of callers: after a launch of its own the launcher is the one
            // who has to wait for the device, a submitter that waits for that command sleeps
            // on the completion number until the launcher has done so.
            // The stand-by is counted from the callers' latest launch: while they keep
            // launching, the queue is busy and theirs.
            auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(kStandByMicros);
            int64_t seen = handed_over_.load(std::memory_order_acquire);
            parked_ = true;
            while (ring_count_ == 0 && retired_.load(std::memory_order_acquire) < handed_over_.load(std::memory_order_acquire)) {
                const auto now = std::chrono::steady_clock::now();
                const int64_t newest = handed_over_.load(std::memory_order_acquire);
                if (newest != seen) { seen = newest; until = now + std::chrono::microseconds(kStandByMicros); }
                if (now >= until) break;
                // (a wait on the system clock: the sanitizer build's runtime does not know the
                // steady-clock wait of newer C libraries and would lose track of the lock)
                ring_cv_.wait_until(g, std::chrono::system_clock::now() + std::chrono::microseconds(kStandBySliceMicros));
            }
            parked_ = false;
            caller_launched_ = false;
            if (ring_count_ != 0) continue;
        }
        if (owed_ == Owed::kBatchThenDrain) { owed_ = Owed::kDrain; return Step::kBatch; }
        if (owed_ == Owed::kDrain) { owed_ = Owed::kNothing; return Step::kDrain; }
        idle_held_back_ = false;
        if (reported_ == kQueueStateReady) {
            if (ready_unsent_) {
                // The Ready of this busy period is still with the submitter that caused it:
                // Idle must not overtake it. That submitter wakes the launcher when it is out.
                idle_held_back_ = true;
            } else {
                reported_ = kQueueStateIdle;
                idle_round_++;
                idle_cv_.notify_all();
                SchedAgent::SendEvent(std::make_shared<XQueueIdleEvent>(kHandle));
            }
        }
        parked_ = true;
        ring_cv_.wait(g, [this]() { return ring_count_ != 0 || owed_ != Owed::kNothing || (idle_held_back_ && !ready_unsent_); });
        parked_ = false;
    }
}

void RingXQueue::DiscardPending()
{
    Guard g(ring_mu_);
    for (size_t i = 0; i < ring_count_; ++i) {
        Pending &slot = ring_[(ring_head_ + i) & (ring_.size() - 1)];
        if (slot.cmd) slot.cmd->SetState(kCommandStateCompleted);
        slot.cmd = nullptr;
    }
    ring_head_ = 0;
    ring_count_ = 0;
}

void RingXQueue::WaitForIdle()
{
    Guard g(ring_mu_);
    if (reported_ == kQueueStateIdle) return;
    const uint64_t round = idle_round_;
    idle_cv_.wait(g, [&]() { return idle_round_ != round; });
}

XQueueState RingXQueue::Query()
{
    Guard g(ring_mu_);
    unwaited_submits_ = 0;   // somebody follows this queue's progress: as good as a wait
    return reported_;
}

int64_t RingXQueue::RequestDrain(std::shared_ptr<XCommand> marker)
{
    bool wake = false;
    int64_t ticket;
    {
        Guard g(ring_mu_);
        unwaited_submits_ = 0;
        if (reported_ == kQueueStateIdle) return -1;
        ticket = next_idx_.load(std::memory_order_acquire) - 1;
        // With everything launched already and a caller that may wait for the device itself,
        // nothing is queued and nobody is woken: the launcher's own drain (owed since the
        // last submission) reports Idle afterwards.
        const bool caller_drains = marker == nullptr && caller_may_launch_ && ring_count_ == 0 &&
                                   handed_over_.load(std::memory_order_acquire) >= ticket;
        // A drain that already closes the ring (queued, or the launcher's own) covers
        // everything submitted so far (command_buffer.cpp:127-155); a marker object always
        // gets a slot of its own, it has to be completed by somebody.
        if (!caller_drains && (marker != nullptr || owed_ != Owed::kNothing)) {
            PushLocked(Slot::kDrain, std::move(marker));
            owed_ = Owed::kNothing;
            wake = parked_;
        }
    }
    if (wake) ring_cv_.notify_one();
    return ticket;
}

std::shared_ptr<XQueueWaitAllCommand> RingXQueue::SubmitWaitAll()
{
    auto marker = std::make_shared<XQueueWaitAllCommand>();
    marker->SetState(kCommandStatePending);
    if (RequestDrain(marker) < 0) marker->SetState(kCommandStateCompleted);
    return marker;
}

void RingXQueue::AwaitRetired(int64_t ticket)
{
    int64_t seen = retired_.load(std::memory_order_acquire);
    if (seen >= ticket) return;
    const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(kSpinMicros);
    for (int probes = 1; ; ++probes) {
        seen = retired_.load(std::memory_order_acquire);
        if (seen >= ticket) return;
        if ((probes & 63) == 0 && std::chrono::steady_clock::now() >= give_up) break;
        __builtin_ia32_pause();
    }
    while (seen < ticket) {
        retired_.wait(seen, std::memory_order_acquire);
        seen = retired_.load(std::memory_order_acquire);
    }
}

void RingXQueue::WaitAll()
{
    const int64_t ticket = RequestDrain(nullptr);
    if (ticket < 0 || retired_.load(std::memory_order_acquire) >= ticket) return;
    if (caller_may_launch_ && handed_over_.load(std::memory_order_acquire) >= ticket) {
        // Everything is on the device already: the caller asks the device itself instead of
        // waiting for the launcher to wake up and do so. One thread asks at a time. A queue
        // that was paused after the launch is waited for as well (AwaitQueue holds until it
        // runs again): the launcher stands by for this caller and would only look after the
        // whole stand-by has passed.
        Guard g(win_mu_);
        if (!queue_wait_active_ && run_ != Run::kStopped) AwaitQueue(g);
    }
    AwaitRetired(ticket);
}

void RingXQueue::Wait(std::shared_ptr<HwCommand> hw_cmd)
{
    { Guard g(ring_mu_); unwaited_submits_ = 0; }
    if (!hw_cmd->Synchronizable()) {
        // No marker of its own: a later marker or a drain retires it.
        hw_cmd->WaitUntil(kCommandStateCompleted);
        return;
    }
    if (hw_cmd->GetState() >= kCommandStateCompleted) return;
    hw_cmd->WaitUntil(kCommandStateInFlight);
    Guard g(win_mu_);
    AwaitMarker(g, hw_cmd);
}

// ---- launcher ----------------------------------------------------------------------------

void RingXQueue::LauncherMain()
{
    while (true) {
        Pending next;
        switch (NextStep(&next)) {
        case Step::kLaunch:
            LaunchFromRing(std::static_pointer_cast<HwCommand>(std::move(next.cmd)));
            break;
        case Step::kBatch:
        {
            Guard g(win_mu_);
            if (auto marker = OldestMarker()) AwaitMarker(g, marker);
            break;
        }
        case Step::kDrain:
        {
            if (next.cmd) next.cmd->SetState(kCommandStateInFlight);
            { Guard g(win_mu_); AwaitQueue(g); }
            if (next.cmd) next.cmd->SetState(kCommandStateCompleted);
            break;
        }
        case Step::kStop:
        {
            { Guard g(win_mu_); AwaitQueue(g); run_ = Run::kStopped; }
            win_cv_.notify_all();
            return;
        }
        }
    }
}

void RingXQueue::ResizeWindow(int64_t threshold)
{
    XASSERT(win_count_ == 0, "the in-flight window can only be resized while it is empty");
    window_.assign(PowerOfTwoAtLeast((size_t)(threshold > 0 ? threshold : 1)), Flight {});
    win_head_ = 0;
}

std::shared_ptr<HwCommand> RingXQueue::OldestMarker()
{
    for (size_t i = 0; i < win_count_; ++i) {
        if (At(i).marked) return At(i).cmd;
    }
    return nullptr;
}

// At level 2 and above a deactivation flushes the flushable commands in flight but not a
// command that is neither flushable nor free to repeat: such a command is only handed over
// once the flushable ones ahead of it are done. `marker` receives the oldest marker that
// still lies behind the newest flushable command, when there is one
// (launch_worker.cpp:171-198).
bool RingXQueue::MustDrainFlushablesFirst(const HwCommand &cmd, std::shared_ptr<HwCommand> *marker)
{
    *marker = nullptr;
    if (level_ < kPreemptLevelDeactivate) return false;
    if (cmd.GetProps(kCommandPropertyDeactivatable | kCommandPropertyIdempotent) != kCommandPropertyNone) return false;
    for (size_t i = win_count_; i-- > 0;) {
        Flight &f = At(i);
        if (f.marked) *marker = f.cmd;
        if (f.flushable) return true;
    }
    *marker = nullptr;
    return false;
}

// One command from the ring through the window (launch_worker.cpp:164-263): the level-2
// rule above; with the window full, a wait for the oldest marker in it (for the whole queue
// when it holds none), otherwise a halt while the queue is paused; then the hand-over.
void RingXQueue::LaunchFromRing(std::shared_ptr<HwCommand> cmd)
{
    cmd->BeforeLaunch(); // cross-queue waits happen here, without any lock
    Guard g(win_mu_);

    std::shared_ptr<HwCommand> marker;
    if (MustDrainFlushablesFirst(*cmd, &marker)) {
        if (marker) AwaitMarker(g, marker);
        else AwaitQueue(g);
    }
    if (win_count_ >= (size_t)threshold_) {
        marker = OldestMarker();
        if (marker) AwaitMarker(g, marker);
        else AwaitQueue(g);
        // Somebody else may have completed the marker while the queue is paused (a waiting
        // caller retires what it waited for): the slot is free then, the launch still waits
        // for the resume. (launch_worker.cpp:200-217 launches in that case.)
        (void)HoldWhilePaused(g);
    } else {
        const bool running = HoldWhilePaused(g);
        XASSERT(running, "the launcher was asked to launch after it had been stopped");
    }
    HandOver(cmd);
}

// The same steps on the submitting thread, taken only when none of them would have to wait.
// The caller holds the ring lock and has seen the launcher parked on an empty ring.
bool RingXQueue::TryLaunchOnCaller(const std::shared_ptr<HwCommand> &cmd, bool mark)
{
    auto *ext = dynamic_cast<HwCommandExtension *>(cmd.get());   // null for callback commands too
    if (ext == nullptr || !ext->DirectLaunchable()) return false;
    Guard g(win_mu_);
    if (run_ != Run::kRunning) return false;
    std::shared_ptr<HwCommand> marker;
    if (win_count_ >= (size_t)threshold_) {
        // A full window is often full of finished commands: a submitter that never waits
        // (a framework that launches kernel after kernel) has nobody who retires them while
        // the launcher stands by. One look at the oldest marker, without waiting; the queue
        // is running and the window lock is held, so a completed marker means what it says.
        marker = OldestMarker();
        auto *marker_ext = dynamic_cast<HwCommandExtension *>(marker.get());
        if (marker_ext == nullptr || !marker_ext->CompletedWithoutWaiting()) return false;
        RetireThrough(marker->GetIdx());
        if (win_count_ >= (size_t)threshold_) return false;
    }
    if (MustDrainFlushablesFirst(*cmd, &marker)) return false;
    cmd->BeforeLaunch(); // does not block for a command that calls itself DirectLaunchable
    HandOver(cmd, mark);
    direct_launches_.fetch_add(1, std::memory_order_relaxed);
    return true;
}

// win_mu_ held. A dropped command completes here without reaching the adapter; every
// batch-th command since the last marker gets one (launch_worker.cpp:236-262).
void RingXQueue::HandOver(const std::shared_ptr<HwCommand> &cmd, bool mark)
{
    const int64_t idx = cmd->GetIdx();
    if (idx <= drop_through_) {
        cmd->SetState(kCommandStateCompleted);
        handed_over_.store(idx, std::memory_order_release);
        return;
    }
    if (mark || idx - last_marked_idx_ >= batch_) cmd->EnableSynchronization();

    // (the class is final: comparing the dynamic type is exact and costs no hierarchy walk)
    if (typeid(*cmd) == typeid(HwCallbackCommand)) {
        auto *cb = static_cast<HwCallbackCommand *>(cmd.get());
        XASSERT(cb->Launch(kHwQueue->GetHandle()) == kXSchedSuccess, "failed to launch HwCallbackCommand (%p)", (void *)cb);
    } else {
        kHwQueue->Launch(cmd);
    }
    cmd->SetState(kCommandStateInFlight);

    if (win_count_ == window_.size()) {
        // only after the threshold was lowered below what is in flight; keep order, grow
        std::vector<Flight> bigger(window_.size() * 2);
        for (size_t i = 0; i < win_count_; ++i) bigger[i] = std::move(At(i));
        window_.swap(bigger);
        win_head_ = 0;
    }
    Flight &f = At(win_count_++);
    f.cmd = cmd;
    f.idx = idx;
    f.marked = cmd->Synchronizable();
    f.flushable = cmd->GetProps(kCommandPropertyDeactivatable) != 0;
    if (f.marked) last_marked_idx_ = idx;
    handed_over_.store(idx, std::memory_order_release);
}

bool RingXQueue::HoldWhilePaused(Guard &g)
{
    while (run_ == Run::kPaused) win_cv_.wait(g);
    return run_ == Run::kRunning;
}

void RingXQueue::PublishRetired(int64_t idx)
{
    if (idx <= retired_.load(std::memory_order_relaxed)) return;
    retired_.store(idx, std::memory_order_release);
    retired_.notify_all();
}

void RingXQueue::RetireThrough(int64_t idx)
{
    while (win_count_ != 0 && At(0).idx <= idx) {
        Flight &f = At(0);
        f.cmd->SetState(kCommandStateCompleted);
        f.cmd = nullptr;
        win_head_ = (win_head_ + 1) & (window_.size() - 1);
        win_count_--;
    }
    PublishRetired(idx);
}

void RingXQueue::RetireEverything()
{
    while (win_count_ != 0) {
        Flight &f = At(0);
        f.cmd->SetState(kCommandStateCompleted);
        f.cmd = nullptr;
        win_head_ = (win_head_ + 1) & (window_.size() - 1);
        win_count_--;
    }
}

// The device wait itself runs with the window lock released. A wait that a Pause() fell into
// may have returned only because the queue was flushed: its result is thrown away and the
// wait starts over once the queue runs again (launch_worker.cpp:265-301). With callers that
// launch, commands may join the window while the lock is released: only what was in flight
// when the wait began is known to be done. One thread at a time waits for the whole queue;
// a second one waits for the first.
void RingXQueue::AwaitQueue(Guard &g)
{
    while (true) {
        if (!HoldWhilePaused(g)) return;
        if (win_count_ == 0) return;
        if (queue_wait_active_) { win_cv_.wait(g); continue; }
        const int64_t newest = At(win_count_ - 1).idx;
        const int64_t pauses = pauses_;
        queue_wait_active_ = true;
        g.unlock();
        kHwQueue->Synchronize();
        g.lock();
        queue_wait_active_ = false;
        win_cv_.notify_all();
        if (pauses == pauses_) { RetireThrough(newest); return; }
    }
}

// Same rule for one marker; the command may also be completed by somebody else (another
// waiter, a drop) whenever the lock is not held, hence the state check on every pass
// (launch_worker.cpp:303-368). Retires everything up to and including the marker.
void RingXQueue::AwaitMarker(Guard &g, const std::shared_ptr<HwCommand> &marker)
{
    XASSERT(marker->Synchronizable(), "the HwCommand should be synchronizable");
    while (true) {
        while (true) {
            if (marker->GetState() >= kCommandStateCompleted) return;
            if (run_ == Run::kRunning) break;
            if (run_ == Run::kStopped) return;
            win_cv_.wait(g);
        }
        XASSERT(marker->GetState() >= kCommandStateInFlight, "the HwCommand has not been launched");
        const int64_t pauses = pauses_;
        g.unlock();
        marker->Synchronize();
        g.lock();
        if (pauses == pauses_) break;
    }
    RetireThrough(marker->GetIdx());
}

CommandLog RingXQueue::InFlightLog()
{
    Guard g(win_mu_);
    CommandLog log;
    for (size_t i = 0; i < win_count_; ++i) log.push_back(At(i).cmd);
    return log;
}

// ---- suspend / resume ----------------------------------------------------------------------

// Optional waits first, then the launcher stops handing over, then the device action of the
// level, then the optional wait for the hardware queue (async_xqueue.cpp:91-113).
void RingXQueue::Suspend(int64_t flags)
{
    if (closing_.load()) return;
    if (suspended_.exchange(true)) return;

    if (flags & kQueueSuspendFlagWaitIdle) WaitForIdle();
    else if (flags & kQueueSuspendFlagWaitAll) WaitAll();

    bool in_flight;
    {
        Guard g(win_mu_);
        run_ = Run::kPaused;
        pauses_++;
        in_flight = win_count_ != 0;   // nothing joins the window while the queue is paused
    }
    // With nothing in flight there is nothing to flush (for adapters that say so).
    deactivated_.store(level_ >= kPreemptLevelDeactivate && (in_flight || !lazy_deactivation_), std::memory_order_release);
    if (deactivated_.load(std::memory_order_relaxed)) kHwQueue->Deactivate();
    if (level_ >= kPreemptLevelInterrupt) kHwQueue->Interrupt();
    if (flags & kQueueSuspendFlagSyncHwQueue) kHwQueue->Synchronize();
}

// Level 1 just lets the launcher go on: what is in flight may still be running and stays in
// the window. From level 2 on the adapter gets the window's contents to replay what it
// flushed. With DropCommands it gets an empty list, everything in flight or queued completes
// unexecuted, and so does every command up to the last index handed out
// (async_xqueue.cpp:115-150).
void RingXQueue::Resume(int64_t flags)
{
    if (!suspended_.exchange(false)) return;
    const bool drop = (flags & kQueueResumeFlagDropCommands) != 0;

    if (level_ > kPreemptLevelBlock) {
        // the launcher is paused, so the window does not change under the adapter
        const CommandLog log = drop ? CommandLog {} : InFlightLog();
        if (level_ >= kPreemptLevelInterrupt) kHwQueue->Restore(log);
        if (level_ >= kPreemptLevelDeactivate && deactivated_.exchange(false, std::memory_order_acq_rel)) kHwQueue->Reactivate(log);
    }
    if (drop && level_ > kPreemptLevelBlock) {
        DiscardPending();
        Guard g(win_mu_);
        RetireEverything();
        drop_through_ = next_idx_.load(std::memory_order_acquire) - 1;
        PublishRetired(drop_through_);
        run_ = Run::kRunning;
    } else {
        Guard g(win_mu_);
        run_ = Run::kRunning;
    }
    win_cv_.notify_all();
}

void RingXQueue::SetPreemptLevel(XPreemptLevel level)
{
    XASSERT(level > kPreemptLevelUnknown && level < kPreemptLevelMax, "invalid preempt level: %d", level);
    if (!GetFeatures(kQueueFeatureDynamicLevel)) {
        XASSERT(level == level_, "this XQueue's hardware queue cannot change level");
        return;
    }
    if (level > kHwQueue->GetMaxSupportedLevel()) {
        XWARN("preempt level %d is not supported by the HwQueue, max supported level is %d",
              level, kHwQueue->GetMaxSupportedLevel());
        return;
    }
    WaitAll(); // nothing in flight while the adapter switches (async_xqueue.cpp:152-174)
    kHwQueue->OnPreemptLevelChange(level);
    {
        Guard g(win_mu_);
        level_ = level;
    }
    SchedAgent::SendEvent(std::make_shared<XQueueConfigUpdateEvent>(kHandle, kDevice, level, threshold_, batch_));
}

void RingXQueue::SetLaunchConfig(int64_t threshold, int64_t batch)
{
    if (threshold <= 0 && batch <= 0) return;
    int64_t new_threshold, new_batch;
    {
        Guard g(win_mu_);
        new_threshold = threshold > 0 ? threshold : threshold_;
        new_batch = batch > 0 ? batch : batch_;
    }
    XASSERT(new_threshold >= new_batch,
            "command threshold (" FMT_64D ") must not be smaller than command batch size (" FMT_64D ")",
            new_threshold, new_batch);
    WaitAll(); // the window is empty when its size changes (async_xqueue.cpp:176-207)
    {
        Guard g(win_mu_);
        threshold_ = new_threshold;
        batch_ = new_batch;
        if (win_count_ == 0 && window_.size() < (size_t)threshold_) ResizeWindow(threshold_);
    }
    SchedAgent::SendEvent(std::make_shared<XQueueConfigUpdateEvent>(kHandle, kDevice, level_, new_threshold, new_batch));
}

} // namespace xsched::preempt
