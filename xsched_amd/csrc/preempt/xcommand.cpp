// XCommand state machine and the HwCommand / HwQueue handle tables.
// reference preempt/src/xqueue/xcommand.cpp, preempt/src/hal/{hw_command,hw_queue}.cpp
#include <chrono>
#include <unordered_map>

#include "xsched/xqueue.h"
#include "xsched/utils/xassert.h"
#include "xsched/preempt/hal/hw_command.h"
#include "xsched/preempt/hal/hw_queue.h"
#include "xsched/preempt/xqueue/xqueue.h"

namespace xsched::preempt
{

// ---- XCommand --------------------------------------------------------------

static constexpr int64_t kWaitSpinMicros = 150;

XCommandState XCommand::GetState()
{
    return (XCommandState)state_.load(std::memory_order_acquire);
}

void XCommand::SetState(XCommandState new_state)
{
    XASSERT(new_state >= kCommandStateCreated && new_state <= kCommandStateCompleted,
            "invalid state: %d", new_state);
    const int32_t old_state = state_.exchange(new_state, std::memory_order_acq_rel);
    XASSERT(new_state >= old_state, "command state must not move backwards (%d -> %d)",
            old_state, new_state);
    if (new_state == old_state) return;

    state_.notify_all();
    for (int s = old_state + 1; s <= new_state; ++s) {
        for (auto &listener : state_listeners_) listener(XCommandState(s));
    }
    if (new_state == kCommandStateCompleted && kCommandType == kCommandTypeHardware) {
        // A completed command lets go of its XQueue so the queue can be destroyed while
        // the application still holds the command (hw_command.cpp:9-16 does this with a
        // state listener, i.e. two allocations per command).
        auto *cmd = static_cast<HwCommand *>(this);
        std::lock_guard<std::mutex> lock(mtx_);
        cmd->xqueue_ = nullptr;
    }
}

// Short waits (a command of a few microseconds) are polled: sleeping on the state
// word costs a wake-up through the kernel, which is several times such a command.
void XCommand::WaitUntil(XCommandState state)
{
    int32_t cur = state_.load(std::memory_order_acquire);
    if (cur >= (int32_t)state) return;
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::microseconds(kWaitSpinMicros);
    for (int probes = 1; ; ++probes) {
        cur = state_.load(std::memory_order_acquire);
        if (cur >= (int32_t)state) return;
        if ((probes & 63) == 0 && std::chrono::steady_clock::now() >= deadline) break;
        __builtin_ia32_pause();
    }
    while (cur < (int32_t)state) {
        state_.wait(cur, std::memory_order_acquire);
        cur = state_.load(std::memory_order_acquire);
    }
}

// ---- HwCommand -------------------------------------------------------------

HwCommand::HwCommand(XCommandProperties props): XCommand(kCommandTypeHardware, props) {}

void HwCommand::Wait()
{
    auto lock = this->GetLock();
    const XQueueHandle xq_h = xqueue_handle_;
    std::shared_ptr<XQueue> xq = xqueue_;
    lock.unlock();

    if (xq_h == 0) {
        // Launched directly on a hardware queue: only the device can tell.
        XASSERT(this->Synchronizable(), "a command that was never submitted to an XQueue "
                "can only be waited for if it is synchronizable");
        return this->Synchronize();
    }
    if (xq == nullptr) {
        // The back pointer is dropped at completion only.
        XASSERT(this->GetState() >= kCommandStateCompleted,
                "command lost its XQueue before completing");
        return;
    }
    xq->Wait(std::static_pointer_cast<HwCommand>(shared_from_this()));
}

void HwCommand::OnSubmit(std::shared_ptr<XQueue> xqueue)
{
    XASSERT(xqueue != nullptr, "XQueue is nullptr");
    auto lock = this->GetLock();
    xqueue_ = xqueue;
    xqueue_handle_ = xqueue->GetHandle();
}

// ---- HwCommandManager ------------------------------------------------------

namespace
{
std::mutex g_cmd_mtx;
std::unordered_map<HwCommandHandle, std::shared_ptr<HwCommand>> g_cmds;
std::mutex g_hwq_mtx;
std::unordered_map<HwQueueHandle, std::shared_ptr<HwQueue>> g_hwqs;
} // namespace

HwCommandHandle HwCommandManager::Add(std::shared_ptr<HwCommand> hw_cmd)
{
    const HwCommandHandle h = hw_cmd->GetHandle();
    std::lock_guard<std::mutex> lock(g_cmd_mtx);
    g_cmds[h] = std::move(hw_cmd);
    return h;
}

std::shared_ptr<HwCommand> HwCommandManager::Del(HwCommandHandle h)
{
    std::lock_guard<std::mutex> lock(g_cmd_mtx);
    auto it = g_cmds.find(h);
    if (it == g_cmds.end()) return nullptr;
    auto cmd = std::move(it->second);
    g_cmds.erase(it);
    return cmd;
}

std::shared_ptr<HwCommand> HwCommandManager::Get(HwCommandHandle h)
{
    std::lock_guard<std::mutex> lock(g_cmd_mtx);
    auto it = g_cmds.find(h);
    return it == g_cmds.end() ? nullptr : it->second;
}

// ---- HwQueueManager --------------------------------------------------------

XResult HwQueueManager::Add(HwQueueHandle h, std::function<std::shared_ptr<HwQueue>()> create)
{
    std::lock_guard<std::mutex> lock(g_hwq_mtx);
    if (g_hwqs.count(h)) {
        XWARN("HwQueue with handle 0x" FMT_64X " already exists", h);
        return kXSchedSuccess;
    }
    auto hwq = create();
    if (hwq == nullptr) {
        XWARN("failed to create HwQueue with handle 0x" FMT_64X, h);
        return kXSchedErrorUnknown;
    }
    XASSERT(hwq->GetHandle() == h, "HwQueue handle mismatch");
    g_hwqs[h] = std::move(hwq);
    return kXSchedSuccess;
}

XResult HwQueueManager::Del(HwQueueHandle h)
{
    std::lock_guard<std::mutex> lock(g_hwq_mtx);
    auto it = g_hwqs.find(h);
    if (it == g_hwqs.end()) {
        XWARN("HwQueue with handle 0x" FMT_64X " does not exist", h);
        return kXSchedErrorNotFound;
    }
    if (auto xq = it->second->GetXQueue()) {
        XWARN("HwQueue 0x" FMT_64X " still carries XQueue 0x" FMT_64X
              "; destroy that with XQueueDestroy() first", h, xq->GetHandle());
        return kXSchedErrorNotAllowed;
    }
    g_hwqs.erase(it);
    return kXSchedSuccess;
}

std::shared_ptr<HwQueue> HwQueueManager::Get(HwQueueHandle h)
{
    std::lock_guard<std::mutex> lock(g_hwq_mtx);
    auto it = g_hwqs.find(h);
    return it == g_hwqs.end() ? nullptr : it->second;
}

std::shared_ptr<XQueue> HwQueueManager::GetXQueue(HwQueueHandle h)
{
    auto hwq = Get(h);
    return hwq ? hwq->GetXQueue() : nullptr;
}

} // namespace xsched::preempt

using namespace xsched::preempt;

// ---- C exports (reference hw_queue.cpp:66-101, hw_command.cpp:82-99) --------

EXPORT_C_FUNC XResult HwQueueDestroy(HwQueueHandle hwq) { return HwQueueManager::Del(hwq); }

EXPORT_C_FUNC XResult HwQueueLaunch(HwQueueHandle hwq, HwCommandHandle hw_cmd)
{
    auto q = HwQueueManager::Get(hwq);
    if (q == nullptr) {
        XWARN("HwQueue with handle 0x" FMT_64X " does not exist", hwq);
        return kXSchedErrorNotFound;
    }
    auto cmd = HwCommandManager::Del(hw_cmd); // ownership moves to the queue
    if (cmd == nullptr) {
        XWARN("HwCommand with handle 0x" FMT_64X " does not exist or is not registered", hw_cmd);
        return kXSchedErrorNotFound;
    }
    if (auto cb = std::dynamic_pointer_cast<HwCallbackCommand>(cmd)) return cb->Launch(hwq);
    q->Launch(cmd);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HwQueueSynchronize(HwQueueHandle hwq)
{
    auto q = HwQueueManager::Get(hwq);
    if (q == nullptr) {
        XWARN("HwQueue with handle 0x" FMT_64X " does not exist", hwq);
        return kXSchedErrorNotFound;
    }
    q->Synchronize();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HwCommandCreateCallback(HwCommandHandle *hw_cmd, LaunchCallback launch, void *data)
{
    if (hw_cmd == nullptr) return kXSchedErrorInvalidValue;
    *hw_cmd = HwCommandManager::Add(std::make_shared<HwCallbackCommand>(launch, data));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HwCommandDestroy(HwCommandHandle hw_cmd)
{
    if (HwCommandManager::Del(hw_cmd) == nullptr) {
        XWARN("HwCommand with handle 0x" FMT_64X " does not exist or is not registered", hw_cmd);
        return kXSchedErrorNotFound;
    }
    return kXSchedSuccess;
}
