// XCommand: the unit that travels through an XQueue's command buffer.
//
// Type / property / state enumerators and the public methods match reference
// preempt/include/xsched/preempt/xqueue/xcommand.h:15-139 so that hardware
// adapters written against XSched compile unchanged, and the data members keep
// that header's order, types and sizes so that an adapter BUILT against it runs
// on this library as well (its inline constructor and accessors see the same
// object). The state word is a lock-free atomic of the enumerator's size
// (waiters sleep on it directly); the mutex only guards the small amount of
// pointer state subclasses keep; the condition variable is not used by this
// implementation and stays for the layout.
#pragma once

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <functional>
#include <list>
#include <memory>
#include <mutex>

#include "xsched/types.h"

namespace xsched::preempt
{

enum XCommandType
{
    kCommandTypeHardware         = 0, // a HwCommand: goes to the hardware queue
    kCommandTypeHostFunction     = 1, // runs on the launch thread after a full drain
    kCommandTypeXQueueWaitAll    = 2, // full drain marker
    kCommandTypeBatchSynchronize = 3, // retire the oldest marked batch
    kCommandTypeXQueueDestroy    = 4, // full drain, then the launch thread exits
};

typedef int64_t XCommandProperties;

enum XCommandProperty
{
    // Neither flushable nor replayable: at Level >= 2 it is launched only after
    // every earlier deactivatable command has completed.
    kCommandPropertyNone           = 0x0000,
    // May be flushed by HwQueue::Deactivate() and re-executed by Reactivate().
    kCommandPropertyDeactivatable  = 0x0001,
    // Writes no memory; replaying it is harmless, so it never waits.
    kCommandPropertyIdempotent     = 0x0002,
    // Submit() returns only once the command has been launched.
    kCommandPropertyBlockingSubmit = 0x0004,
    kCommandPropertyMaskAll        = -1,
};

enum XCommandState
{
    kCommandStateCreated   = 0,
    kCommandStatePending   = 1, // in the command buffer
    kCommandStateInFlight  = 2, // handed to the hardware queue
    kCommandStateCompleted = 3, // finished, dropped or flushed for good
    kCommandStateMax       = 4,
};

class XCommand : public std::enable_shared_from_this<XCommand>
{
public:
    XCommand(XCommandType type, XCommandProperties props = kCommandPropertyNone)
        : kCommandType(type), props_(props) {}
    virtual ~XCommand() = default;

    virtual void Wait() { this->WaitUntil(kCommandStateCompleted); }

    XCommandState GetState();

    /// States only move forward; listeners see every state passed through.
    void SetState(XCommandState state);
    void WaitUntil(XCommandState state);
    void AddStateListener(std::function<void(XCommandState)> listener)
    { state_listeners_.push_back(std::move(listener)); }

    /// Lock for short critical sections on subclass members.
    std::unique_lock<std::mutex> GetLock() { return std::unique_lock<std::mutex>(mtx_); }

    XCommandType GetType() const { return kCommandType; }
    void SetProps(XCommandProperties props) { props_ |= props; }
    XCommandProperties GetProps(XCommandProperties mask = kCommandPropertyMaskAll) const
    { return props_ & mask; }

private:
    const XCommandType kCommandType;
    std::atomic<int32_t> state_ { kCommandStateCreated };
    XCommandProperties props_;

    std::mutex mtx_;
    std::condition_variable state_cv_;
    std::list<std::function<void(XCommandState)>> state_listeners_;
};

class HostFunctionCommand final : public XCommand
{
public:
    HostFunctionCommand(std::function<void()> f)
        : XCommand(kCommandTypeHostFunction), func_(std::move(f)) {}
    void Execute() { func_(); }
private:
    std::function<void()> func_;
};

class XQueueWaitAllCommand final : public XCommand
{ public: XQueueWaitAllCommand(): XCommand(kCommandTypeXQueueWaitAll) {} };

class BatchSynchronizeCommand final : public XCommand
{ public: BatchSynchronizeCommand(): XCommand(kCommandTypeBatchSynchronize) {} };

class XQueueDestroyCommand final : public XCommand
{ public: XQueueDestroyCommand(): XCommand(kCommandTypeXQueueDestroy) {} };

} // namespace xsched::preempt
