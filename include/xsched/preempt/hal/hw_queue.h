// HwQueue: the plugin interface a hardware adapter implements, one instance per
// native queue (HIP stream, …). Virtual order and threading contract follow
// reference preempt/include/xsched/preempt/hal/hw_queue.h:19-94.
#pragma once

#include <functional>
#include <list>
#include <memory>

#include "xsched/types.h"
#include "xsched/utils/common.h"
#include "xsched/preempt/hal/hw_command.h"

namespace xsched::preempt
{

class XQueue;

/// Commands launched but not yet known complete, oldest first.
using CommandLog = std::list<std::shared_ptr<HwCommand>>;

class HwQueue
{
public:
    HwQueue() = default;
    virtual ~HwQueue() = default;

    /// Level 1. Enqueue on the native queue. Called with the launch lock held:
    /// must not block on another queue or command.
    virtual void Launch(std::shared_ptr<HwCommand> hw_cmd) = 0;

    /// Level 1. Wait until the native queue is empty; may also return once its
    /// contents have been flushed (Level 2) or killed (Level 3).
    virtual void Synchronize() = 0;

    /// Level 2. Keep the device from starting further work of this queue
    /// (stall it, or flush what is in flight).
    virtual void Deactivate() {}

    /// Level 2. Undo Deactivate(); `log` lists what was in flight so flushed
    /// commands can be replayed.
    virtual void Reactivate(const CommandLog &log) { UNUSED(log); }

    /// Level 3. Stop the command that is running right now.
    virtual void Interrupt() {}

    /// Level 3. Undo Interrupt().
    virtual void Restore(const CommandLog &log) { UNUSED(log); }

    virtual XDevice GetDevice() = 0;
    virtual HwQueueHandle GetHandle() = 0;
    virtual bool SupportDynamicLevel() = 0;
    virtual XPreemptLevel GetMaxSupportedLevel() = 0;

    /// The XQueue's level has changed (also called once at creation).
    virtual void OnPreemptLevelChange(XPreemptLevel level) { UNUSED(level); }

    /// First call on the freshly started launch thread (bind device / context).
    virtual void OnXQueueCreate() {}

    /// Called on the submitting thread for each command, before it is buffered.
    virtual void OnHwCommandSubmit(std::shared_ptr<HwCommand> hw_cmd) { UNUSED(hw_cmd); }

    std::shared_ptr<XQueue> GetXQueue() { return xq_; }
    void SetXQueue(std::shared_ptr<XQueue> xq) { xq_ = xq; }

private:
    std::shared_ptr<XQueue> xq_ = nullptr;
};

/// Registry of hardware queues by handle.
class HwQueueManager
{
public:
    STATIC_CLASS(HwQueueManager);
    static XResult Add(HwQueueHandle hwq_h, std::function<std::shared_ptr<HwQueue>()> create);
    static XResult Del(HwQueueHandle hwq_h);
    static std::shared_ptr<HwQueue> Get(HwQueueHandle hwq_h);
    static std::shared_ptr<XQueue> GetXQueue(HwQueueHandle hwq_h);
};

} // namespace xsched::preempt
