// HwCommand: plugin base class for anything a hardware queue can execute.
// Virtual order and contracts follow reference
// preempt/include/xsched/preempt/hal/hw_command.h:16-110.
#pragma once

#include <memory>
#include <mutex>
#include <unordered_map>

#include "xsched/types.h"
#include "xsched/utils/common.h"
#include "xsched/preempt/xqueue/xcommand.h"

namespace xsched::preempt
{

class XQueue;

class HwCommand : public XCommand
{
public:
    HwCommand(XCommandProperties props = kCommandPropertyNone);
    virtual ~HwCommand() = default;

    /// Block until the device has finished this command. Needs
    /// EnableSynchronization() before launch. May return early when the command
    /// was flushed by a deactivation or killed by an interrupt.
    virtual void Synchronize() = 0;

    /// Whether Synchronize() may be called.
    virtual bool Synchronizable() = 0;

    /// Ask the adapter to attach a completion marker (event, fence, …) at launch.
    /// Returns false when the command cannot carry one.
    virtual bool EnableSynchronization() = 0;

    /// Runs on the launch thread right before launch, without the launch lock;
    /// the place for cross-queue waits.
    virtual void BeforeLaunch() {}

    /// Process-unique handle.
    virtual HwCommandHandle GetHandle() { return (uint64_t)this ^ ((uint64_t)GetProcessId() << 48); }

    /// 1-based submission index inside its XQueue; -1 before submission.
    int64_t GetIdx() const { return idx_; }
    void SetIdx(int64_t idx) { idx_ = idx; }

    /// 0 until submitted.
    XQueueHandle GetXQueueHandle() const { return xqueue_handle_; }

    /// Wait for real completion (replays after a flush included).
    virtual void Wait() final override;

    void OnSubmit(std::shared_ptr<XQueue> xqueue);

private:
    friend class XCommand;   // a completed command lets go of its XQueue
    int64_t idx_ = -1;
    XQueueHandle xqueue_handle_ = 0;
    std::shared_ptr<XQueue> xqueue_ = nullptr;
};

/// Command whose launch body is a user callback (HwCommandCreateCallback()).
class HwCallbackCommand final : public HwCommand
{
public:
    HwCallbackCommand(LaunchCallback launch, void *data)
        : HwCommand(kCommandPropertyNone), launch_(launch), data_(data) {}
    virtual ~HwCallbackCommand() = default;

    virtual void Synchronize()           override {}
    virtual bool Synchronizable()        override { return false; }
    virtual bool EnableSynchronization() override { return false; }
    XResult Launch(HwQueueHandle hwq) { return launch_(hwq, data_); }

private:
    LaunchCallback launch_ = nullptr;
    void *data_ = nullptr;
};

/// Handle table for commands that have been created but not yet submitted.
class HwCommandManager
{
public:
    STATIC_CLASS(HwCommandManager);
    static HwCommandHandle Add(std::shared_ptr<HwCommand> hw_cmd);
    static std::shared_ptr<HwCommand> Del(HwCommandHandle hw_cmd_h);
    static std::shared_ptr<HwCommand> Get(HwCommandHandle hw_cmd_h);
};

} // namespace xsched::preempt
