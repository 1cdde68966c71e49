// reference preempt/src/xqueue/command_buffer.cpp
#include "xsched/utils/xassert.h"
#include "xsched/preempt/sched/agent.h"
#include "xsched/preempt/xqueue/async_xqueue.h"

using namespace xsched::sched;

namespace xsched::preempt
{

// The buffer starts with one drain marker so that "last enqueued command" is
// always defined and an idle queue always ends in a (completed) drain marker.
CommandBuffer::CommandBuffer(XQueueHandle xq_h): kXQueueHandle(xq_h)
{
    Enqueue(std::make_shared<XQueueWaitAllCommand>());
}

void CommandBuffer::WaitForNextIdle()
{
    std::unique_lock<std::mutex> lock(mtx_);
    if (xq_state_ == kQueueStateIdle) return;
    const uint64_t seen = idle_cnt_;
    idle_cv_.wait(lock, [&]() { return idle_cnt_ != seen; });
}

XQueueState CommandBuffer::GetXQueueState()
{
    std::lock_guard<std::mutex> lock(mtx_);
    return xq_state_;
}

// When the FIFO is empty the launch thread does not go to sleep right away: the
// buffer hands it, in turn, a batch-sync (retire the oldest marked batch), then
// a full drain marker, and only after that drain has completed does the XQueue
// become Idle (command_buffer.cpp:39-97). The Idle/Ready events are sent with
// the buffer lock held so that a scheduler sees them in the order they happened.
std::shared_ptr<XCommand> CommandBuffer::Dequeue()
{
    std::unique_lock<std::mutex> lock(mtx_);

    while (cmds_.empty()) {
        drain_needed_ = false;
        switch (last_enqueued_cmd_->GetType()) {
        case kCommandTypeXQueueWaitAll:
            if (xq_state_ == kQueueStateReady) {
                xq_state_ = kQueueStateIdle;
                idle_cnt_++;
                idle_cv_.notify_all();
                SchedAgent::SendEvent(std::make_shared<XQueueIdleEvent>(kXQueueHandle));
            }
            consumer_waiting_ = true;
            cv_.wait(lock, [this]() { return !cmds_.empty() || drain_needed_; });
            consumer_waiting_ = false;
            // Woken with an empty buffer: a command was launched directly meanwhile and
            // is now the last one enqueued, so the next pass starts the drain sequence.
            break;

        case kCommandTypeBatchSynchronize:
        {
            auto drain = std::make_shared<XQueueWaitAllCommand>();
            drain->SetState(kCommandStatePending);
            last_enqueued_cmd_ = drain;
            return drain;
        }

        default:
        {
            auto batch = std::make_shared<BatchSynchronizeCommand>();
            batch->SetState(kCommandStatePending);
            last_enqueued_cmd_ = batch;
            return batch;
        }
        }
    }

    auto xcmd = std::move(cmds_.front());
    cmds_.pop_front();
    return xcmd;
}

void CommandBuffer::Enqueue(std::shared_ptr<XCommand> xcmd)
{
    const auto ready_time = std::chrono::system_clock::now();
    XASSERT(xcmd != nullptr, "xcmd should not be nullptr");
    xcmd->SetState(kCommandStatePending);

    bool wake;
    {
        std::lock_guard<std::mutex> lock(mtx_);
        const bool hardware = xcmd->GetType() == kCommandTypeHardware;
        if (hardware && xq_state_ == kQueueStateIdle) {
            xq_state_ = kQueueStateReady;
            SchedAgent::SendEvent(std::make_shared<XQueueReadyEvent>(kXQueueHandle, ready_time));
        }
        last_enqueued_cmd_ = xcmd;
        // The launch thread sleeps and nothing is queued: submission order is launch
        // order even if this thread launches, and the lock keeps it so.
        if (hardware && direct_launch_ && consumer_waiting_ && cmds_.empty() &&
            direct_launch_(std::static_pointer_cast<HwCommand>(xcmd))) {
            drain_needed_ = true;
        } else {
            cmds_.emplace_back(std::move(xcmd));
        }
        wake = consumer_waiting_;
    }
    if (wake) cv_.notify_one();
}

void CommandBuffer::DropAll()
{
    std::lock_guard<std::mutex> lock(mtx_);
    for (auto &xcmd : cmds_) xcmd->SetState(kCommandStateCompleted);
    cmds_.clear();
}

std::shared_ptr<XQueueWaitAllCommand> CommandBuffer::EnqueueXQueueWaitAllCommand(bool *consumer_asleep)
{
    std::unique_lock<std::mutex> lock(mtx_);
    if (consumer_asleep) *consumer_asleep = consumer_waiting_;

    // Idle: the tail is the drain marker that made the queue idle (completed).
    // Not idle but the tail is already a drain marker: share it.
    if (xq_state_ == kQueueStateIdle || last_enqueued_cmd_->GetType() == kCommandTypeXQueueWaitAll) {
        auto tail = std::dynamic_pointer_cast<XQueueWaitAllCommand>(last_enqueued_cmd_);
        XASSERT(tail != nullptr, "an idle XQueue must end in a drain marker");
        return tail;
    }

    auto drain = std::make_shared<XQueueWaitAllCommand>();
    drain->SetState(kCommandStatePending);
    last_enqueued_cmd_ = drain;
    cmds_.emplace_back(drain);
    const bool wake = consumer_waiting_;
    lock.unlock();
    if (wake) cv_.notify_one();
    return drain;
}

} // namespace xsched::preempt
