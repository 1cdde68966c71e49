// reference preempt/src/xqueue/launch_worker.cpp
#include "xsched/utils/xassert.h"
#include "xsched/preempt/xqueue/async_xqueue.h"

namespace xsched::preempt
{

LaunchWorker::LaunchWorker(std::shared_ptr<HwQueue> hwq, std::shared_ptr<CommandBuffer> buf,
                           XPreemptLevel level, int64_t threshold, int64_t batch_size)
    : level_(level), threshold_(threshold), batch_size_(batch_size), kHwq(hwq), kCmdBuf(buf)
{
    // With fewer window slots than the marker period the window could fill up
    // without holding a single marker to wait on.
    XASSERT(threshold_ >= batch_size_, "threshold must not be smaller than command batch size");
    thread_ = std::make_unique<std::thread>([this]() {
        kHwq->OnXQueueCreate(); // lets the adapter bind its device / context to this thread
        this->Loop();
    });
}

// The owner enqueues an XQueueDestroyCommand first; the thread drains and exits.
LaunchWorker::~LaunchWorker() { thread_->join(); }

void LaunchWorker::Pause()
{
    std::lock_guard<std::mutex> lock(mtx_);
    state_ = kPaused;
    pause_count_ += 1;
}

void LaunchWorker::Resume()
{
    { std::lock_guard<std::mutex> lock(mtx_); state_ = kRunning; }
    cv_.notify_all();
}

void LaunchWorker::ResumeAndDrop(int64_t drop_idx)
{
    {
        std::lock_guard<std::mutex> lock(mtx_);
        RetireAll();
        drop_idx_ = drop_idx;
        state_ = kRunning;
    }
    cv_.notify_all();
}

CommandLog LaunchWorker::SnapshotCommandLog()
{
    std::lock_guard<std::mutex> lock(mtx_);
    return cmd_log_;
}

void LaunchWorker::SyncAll()
{
    Lock lock(mtx_);
    SyncAllLocked(lock);
}

void LaunchWorker::SyncCmd(std::shared_ptr<HwCommand> hw_cmd)
{
    Lock lock(mtx_);
    SyncCmdLocked(lock, hw_cmd);
}

void LaunchWorker::RetireAll()
{
    sync_cmd_log_.clear();
    for (auto &cmd : cmd_log_) cmd->SetState(kCommandStateCompleted);
    cmd_log_.clear();
}

bool LaunchWorker::WaitWhilePaused(Lock &lock)
{
    while (state_ == kPaused) cv_.wait(lock);
    return state_ == kRunning;
}

void LaunchWorker::Loop()
{
    while (true) {
        std::shared_ptr<XCommand> xcmd = kCmdBuf->Dequeue();

        switch (xcmd->GetType()) {
        case kCommandTypeHardware:
            LaunchHwCommand(std::static_pointer_cast<HwCommand>(xcmd));
            break;

        case kCommandTypeHostFunction:
        {
            // Runs after everything before it has completed, with the lock held.
            auto *fn = static_cast<HostFunctionCommand *>(xcmd.get());
            fn->SetState(kCommandStateInFlight);
            {
                Lock lock(mtx_);
                SyncAllLocked(lock);
                fn->Execute();
            }
            fn->SetState(kCommandStateCompleted);
            break;
        }

        case kCommandTypeXQueueWaitAll:
            xcmd->SetState(kCommandStateInFlight);
            SyncAll();
            xcmd->SetState(kCommandStateCompleted);
            break;

        case kCommandTypeBatchSynchronize:
        {
            xcmd->SetState(kCommandStateInFlight);
            Lock lock(mtx_);
            if (!sync_cmd_log_.empty()) {
                auto oldest_marker = sync_cmd_log_.front();
                SyncCmdLocked(lock, oldest_marker);
            }
            lock.unlock();
            xcmd->SetState(kCommandStateCompleted);
            break;
        }

        case kCommandTypeXQueueDestroy:
        {
            xcmd->SetState(kCommandStateInFlight);
            {
                Lock lock(mtx_);
                SyncAllLocked(lock);
                state_ = kTerminated;
            }
            cv_.notify_all();
            xcmd->SetState(kCommandStateCompleted);
            return;
        }

        default:
            XASSERT(false, "unknown command type: %d", xcmd->GetType());
        }
    }
}

// One command through the window (launch_worker.cpp:164-263):
//  1. Level >= 2 and the command is neither deactivatable nor idempotent: first
//     wait for the in-flight deactivatable commands ahead of it, because a
//     deactivation would flush those but not this one.
//  2. Window full: wait for the oldest marker that frees at least one slot
//     (or the whole queue when no marker is in flight). Otherwise: wait here
//     while the queue is paused.
//  3. Dropped (idx <= drop_idx): complete without launching.
//  4. batch_size commands since the last marker: this one carries a marker.
//  5. Launch, log it.
void LaunchWorker::LaunchHwCommand(std::shared_ptr<HwCommand> hw_cmd)
{
    hw_cmd->BeforeLaunch();
    Lock lock(mtx_);

    std::shared_ptr<HwCommand> marker;
    if (NeedsDrainBefore(hw_cmd, &marker)) {
        if (marker) SyncCmdLocked(lock, marker);
        else SyncAllLocked(lock);
    }

    if (cmd_log_.size() >= (size_t)threshold_) {
        const int64_t front_idx = cmd_log_.front()->GetIdx();
        marker = nullptr;
        for (auto &cmd : sync_cmd_log_) {
            if (cmd->GetIdx() >= front_idx) { marker = cmd; break; }
        }
        if (marker) SyncCmdLocked(lock, marker);
        else SyncAllLocked(lock);
    } else {
        const bool running = WaitWhilePaused(lock);
        XASSERT(running, "launch thread asked to launch after termination");
    }

    LaunchLocked(hw_cmd);
}

// Step 1's test. Newest to oldest: remember the earliest marker that still lies behind
// the newest deactivatable command.
bool LaunchWorker::NeedsDrainBefore(const std::shared_ptr<HwCommand> &hw_cmd, std::shared_ptr<HwCommand> *marker)
{
    if (level_ < kPreemptLevelDeactivate) return false;
    if (hw_cmd->GetProps(kCommandPropertyDeactivatable | kCommandPropertyIdempotent) != kCommandPropertyNone) {
        return false;
    }
    for (auto it = cmd_log_.rbegin(); it != cmd_log_.rend(); ++it) {
        if ((*it)->Synchronizable()) *marker = *it;
        if ((*it)->GetProps(kCommandPropertyDeactivatable)) return true;
    }
    *marker = nullptr;
    return false;
}

// Steps 3 to 5, lock held.
void LaunchWorker::LaunchLocked(const std::shared_ptr<HwCommand> &hw_cmd)
{
    if (hw_cmd->GetIdx() <= drop_idx_) {
        hw_cmd->SetState(kCommandStateCompleted);
        handled_idx_.store(hw_cmd->GetIdx(), std::memory_order_release);
        return;
    }

    if (hw_cmd->GetIdx() - last_synchronizable_idx_ >= batch_size_) {
        hw_cmd->EnableSynchronization();
    }

    if (hw_cmd->GetProps(kCommandPropertyCallback)) {
        auto *cb = static_cast<HwCallbackCommand *>(hw_cmd.get());
        XASSERT(cb->Launch(kHwq->GetHandle()) == kXSchedSuccess,
                "failed to launch HwCallbackCommand (%p)", (void *)cb);
    } else {
        kHwq->Launch(hw_cmd);
    }
    hw_cmd->SetState(kCommandStateInFlight);

    cmd_log_.emplace_back(hw_cmd);
    if (hw_cmd->Synchronizable()) {
        sync_cmd_log_.emplace_back(hw_cmd);
        last_synchronizable_idx_ = hw_cmd->GetIdx();
    }
    handled_idx_.store(hw_cmd->GetIdx(), std::memory_order_release);
}

// The same command through the same window on the SUBMITTING thread, but only when none
// of the steps would have to wait. The caller (CommandBuffer::Enqueue) holds the buffer
// lock and has seen the launch thread asleep on an empty buffer, so no other command
// can slip in between.
bool LaunchWorker::TryLaunchDirect(const std::shared_ptr<HwCommand> &hw_cmd)
{
    if (!hw_cmd->DirectLaunchable() || hw_cmd->GetProps(kCommandPropertyCallback)) return false;
    Lock lock(mtx_);
    if (state_ != kRunning) return false;
    if (cmd_log_.size() >= (size_t)threshold_) return false;
    std::shared_ptr<HwCommand> marker;
    if (NeedsDrainBefore(hw_cmd, &marker)) return false;
    hw_cmd->BeforeLaunch(); // never blocks for a command that declares itself DirectLaunchable
    LaunchLocked(hw_cmd);
    direct_launches_.fetch_add(1, std::memory_order_relaxed);
    return true;
}

// The blocking driver wait happens with the lock released. If a Pause() came in
// meanwhile, the wait may have returned only because the queue was flushed, so
// the result is discarded and the wait repeated after the resume
// (launch_worker.cpp:265-301).
void LaunchWorker::SyncAllLocked(Lock &lock)
{
    while (true) {
        if (!WaitWhilePaused(lock)) return;
        if (cmd_log_.empty()) return;

        // With direct launches another thread may add commands while the lock is
        // released: only what was in flight when the wait began is known to be done.
        const int64_t last_idx = cmd_log_.back()->GetIdx();
        const int64_t pause_cnt = pause_count_;
        lock.unlock();
        kHwq->Synchronize();
        lock.lock();
        if (pause_cnt == pause_count_) { RetireUpTo(last_idx); return; }
    }
}

// Same retry rule; in addition the command may be completed by another thread
// (a second waiter, a drop) whenever the lock is not held, hence the state check
// on every pass (launch_worker.cpp:303-368). Retires every logged command up to
// and including hw_cmd.
void LaunchWorker::SyncCmdLocked(Lock &lock, const std::shared_ptr<HwCommand> &hw_cmd)
{
    XASSERT(hw_cmd->Synchronizable(), "the HwCommand should be synchronizable");

    while (true) {
        while (true) {
            if (hw_cmd->GetState() >= kCommandStateCompleted) return;
            if (state_ == kRunning) break;
            if (state_ == kTerminated) return;
            cv_.wait(lock);
        }

        XASSERT(hw_cmd->GetState() >= kCommandStateInFlight, "the HwCommand has not been launched");

        const int64_t pause_cnt = pause_count_;
        lock.unlock();
        hw_cmd->Synchronize();
        lock.lock();
        if (pause_cnt == pause_count_) break;
    }

    RetireUpTo(hw_cmd->GetIdx());
}

void LaunchWorker::RetireUpTo(int64_t idx)
{
    while (!sync_cmd_log_.empty() && sync_cmd_log_.front()->GetIdx() <= idx) {
        sync_cmd_log_.pop_front();
    }
    while (!cmd_log_.empty() && cmd_log_.front()->GetIdx() <= idx) {
        cmd_log_.front()->SetState(kCommandStateCompleted);
        cmd_log_.pop_front();
    }
}

} // namespace xsched::preempt
