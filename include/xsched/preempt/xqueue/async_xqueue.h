// The asynchronous XQueue: command buffer + launch thread.
//
//   Submit() -> CommandBuffer -> LaunchWorker thread -> HwQueue::Launch()
//
// The launch thread keeps at most `threshold` commands in flight and attaches a
// completion marker to every `batch_size`-th one, so that a suspended queue
// drains within a bounded number of commands ("progressive launching").
// Behaviour follows reference preempt/src/xqueue/{command_buffer,launch_worker,
// async_xqueue}.cpp.
#pragma once

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>

#include "xsched/protocol/def.h"
#include "xsched/preempt/xqueue/xqueue.h"

namespace xsched::preempt
{

/// FIFO between submitters and the launch thread; also owns the Idle/Ready state
/// of the XQueue and synthesises the drain sequence (one batch sync, one full
/// sync) when it runs empty. reference command_buffer.cpp:8-155
class CommandBuffer
{
public:
    explicit CommandBuffer(XQueueHandle xq_h);

    void Enqueue(std::shared_ptr<XCommand> xcmd);
    std::shared_ptr<XCommand> Dequeue();
    /// Returns a drain marker covering everything enqueued so far (an existing
    /// one when possible; an already completed one when the queue is idle).
    /// `consumer_asleep`, when given, tells whether the launch thread was asleep on the
    /// buffer at that moment (it is woken for the marker either way).
    std::shared_ptr<XQueueWaitAllCommand> EnqueueXQueueWaitAllCommand(bool *consumer_asleep = nullptr);
    /// Complete and discard everything still buffered.
    void DropAll();

    void WaitForNextIdle();
    XQueueState GetXQueueState();

    /// Direct launch (see HwQueue::SupportDirectLaunch): `launch` is tried, with the
    /// buffer lock held, for a hardware command that arrives while the launch thread
    /// sleeps on an empty buffer; when it returns true the command has been launched and
    /// is not queued. The launch thread is still woken, off the submitter's path, to run
    /// the drain sequence that ends in the Idle event.
    using DirectLaunch = std::function<bool(const std::shared_ptr<HwCommand> &)>;
    void SetDirectLaunch(DirectLaunch launch) { direct_launch_ = std::move(launch); }

private:
    const XQueueHandle kXQueueHandle;

    std::mutex mtx_;
    std::condition_variable cv_;
    bool consumer_waiting_ = false;
    bool drain_needed_ = false;
    DirectLaunch direct_launch_;

    XQueueState xq_state_ = kQueueStateIdle;
    std::shared_ptr<XCommand> last_enqueued_cmd_;
    std::deque<std::shared_ptr<XCommand>> cmds_;

    uint64_t idle_cnt_ = 0;
    std::condition_variable idle_cv_;
};

/// The launch thread and its in-flight bookkeeping. reference launch_worker.cpp:6-368
class LaunchWorker
{
public:
    LaunchWorker(std::shared_ptr<HwQueue> hwq, std::shared_ptr<CommandBuffer> buf,
                 XPreemptLevel level, int64_t threshold, int64_t batch_size);
    ~LaunchWorker();

    void Pause();
    void Resume();
    /// Resume and discard: everything in flight is completed, and every command
    /// with idx <= drop_idx that shows up later is completed without launching.
    void ResumeAndDrop(int64_t drop_idx);

    /// Snapshot of the in-flight commands, oldest first.
    CommandLog SnapshotCommandLog();

    void SyncAll();
    /// `hw_cmd` must be synchronizable and already launched.
    void SyncCmd(std::shared_ptr<HwCommand> hw_cmd);

    /// Launch on the calling thread if that needs no waiting: queue running, window not
    /// full, no drain point. False: nothing happened, queue the command as usual.
    bool TryLaunchDirect(const std::shared_ptr<HwCommand> &hw_cmd);
    /// Index of the last hardware command that has been launched (or dropped).
    int64_t HandledIdx() const { return handled_idx_.load(std::memory_order_acquire); }
    int64_t DirectLaunches() const { return direct_launches_.load(std::memory_order_relaxed); }

    void SetPreemptLevel(XPreemptLevel level) { level_ = level; }
    void SetLaunchConfig(int64_t threshold, int64_t batch_size)
    { threshold_ = threshold; batch_size_ = batch_size; }
    int64_t GetThreshold() const { return threshold_; }
    int64_t GetBatchSize() const { return batch_size_; }

private:
    enum WorkerState { kRunning = 0, kPaused = 1, kTerminated = 2 };
    using Lock = std::unique_lock<std::mutex>;

    void Loop();
    void LaunchHwCommand(std::shared_ptr<HwCommand> hw_cmd);
    /// Drop check, marker rule, Launch(), log. Lock held.
    void LaunchLocked(const std::shared_ptr<HwCommand> &hw_cmd);
    bool NeedsDrainBefore(const std::shared_ptr<HwCommand> &hw_cmd, std::shared_ptr<HwCommand> *marker);
    void RetireUpTo(int64_t idx);
    /// Both return with the lock held. They release it around the blocking
    /// driver wait and start over when a Pause() happened meanwhile.
    void SyncAllLocked(Lock &lock);
    void SyncCmdLocked(Lock &lock, const std::shared_ptr<HwCommand> &hw_cmd);
    /// Block while paused; false when terminated.
    bool WaitWhilePaused(Lock &lock);
    void RetireAll();

    XPreemptLevel level_;
    int64_t threshold_;
    int64_t batch_size_;

    const std::shared_ptr<HwQueue> kHwq;
    const std::shared_ptr<CommandBuffer> kCmdBuf;

    CommandLog cmd_log_;        // in flight, oldest first
    CommandLog sync_cmd_log_;   // the marked subset of cmd_log_
    int64_t last_synchronizable_idx_ = -1;

    std::mutex mtx_;
    std::condition_variable cv_;

    int64_t drop_idx_ = -1;
    std::atomic<int64_t> handled_idx_ { 0 };
    std::atomic<int64_t> direct_launches_ { 0 };
    int64_t pause_count_ = 0;
    WorkerState state_ = kRunning;
    std::unique_ptr<std::thread> thread_;
};

class AsyncXQueue : public XQueue
{
public:
    AsyncXQueue(std::shared_ptr<HwQueue> hwq, XPreemptLevel level,
                int64_t threshold  = XSCHED_DEFAULT_COMMAND_THRESHOLD,
                int64_t batch_size = XSCHED_DEFAULT_COMMAND_BATCH_SIZE);
    virtual ~AsyncXQueue();

    virtual void Submit(std::shared_ptr<HwCommand> hw_cmd) override;
    virtual std::shared_ptr<XQueueWaitAllCommand> SubmitWaitAll() override;
    virtual void WaitAll() override;
    virtual void Wait(std::shared_ptr<HwCommand> hw_cmd) override;
    virtual XQueueState Query() override;
    virtual int64_t GetHwCommandCount() override;
    virtual int64_t GetDirectLaunchCount() override { return launch_worker_->DirectLaunches(); }

    virtual void Suspend(int64_t flags) override;
    virtual void Resume(int64_t flags) override;

    virtual void SetPreemptLevel(XPreemptLevel level) override;
    virtual void SetLaunchConfig(int64_t threshold, int64_t batch_size) override;

private:
    XPreemptLevel level_;
    const std::shared_ptr<CommandBuffer> cmd_buf_;
    const std::shared_ptr<LaunchWorker> launch_worker_;

    bool direct_ = false; // the adapter allows launches and drains on application threads
    std::atomic_bool suspended_ { false };
    std::atomic_bool terminated_ { false };
    std::atomic<int64_t> next_hw_cmd_idx_ { 1 };
};

} // namespace xsched::preempt
