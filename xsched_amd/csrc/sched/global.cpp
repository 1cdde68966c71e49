// Daemon client. reference sched/src/scheduler/global.cpp:17-69
#include <thread>

#include "xsched/protocol/def.h"
#include "xsched/sched/ipc/channel.h"
#include "xsched/utils/xassert.h"
#include "global.h"

namespace xsched::sched
{

// The client listens on a channel keyed by its pid and talks to the daemon's
// well-known channel. The receiver exists before the first event is sent, so the
// daemon can answer the ProcessCreate event right away.
struct GlobalScheduler::DaemonLink
{
    const ipc::ChannelKey own_key;
    ipc::Node from_daemon;
    ipc::Node to_daemon;
    std::thread listener;

    DaemonLink()
        : own_key((ipc::ChannelKey)GetProcessId())
        , from_daemon(own_key, ipc::NodeType::kReceiver)
        , to_daemon((ipc::ChannelKey)XSCHED_SERVER_CHANNEL_KEY, ipc::NodeType::kSender)
    {
    }

    /// Operation records until a terminate record or the end of the channel.
    template <typename Fn> void Listen(Fn &&execute)
    {
        while (auto msg = from_daemon.Receive()) {
            if (!Operation::WireRecordOk(msg->Data(), msg->Size())) {
                XWARN("dropped a malformed operation record of %zu bytes", msg->Size());
                continue;
            }
            auto op = Operation::CopyConstructor(msg->Data());
            if (UNLIKELY(op->Type() == kOperationTerminate)) return;
            execute(std::move(op));
        }
    }

    /// Wakes the listener with a terminate record sent to this process itself, then
    /// takes both ends down.
    void Close()
    {
        if (listener.joinable()) {
            TerminateOperation bye;
            ipc::Node self(own_key, ipc::NodeType::kSender);
            if (!self.Send(bye.Data(), bye.Size())) from_daemon.Remove();
            listener.join();
        }
        from_daemon.Remove();
        to_daemon.Remove();
    }
};

GlobalScheduler::GlobalScheduler(): Scheduler(kSchedulerGlobal) {}
GlobalScheduler::~GlobalScheduler() { Stop(); }

void GlobalScheduler::Run()
{
    link_ = std::make_unique<DaemonLink>();
    DaemonLink *link = link_.get();
    link->listener = std::thread([this, link]() {
        link->Listen([this](std::shared_ptr<const Operation> op) { Execute(op); });
    });
}

void GlobalScheduler::Stop()
{
    if (!link_) return;
    link_->Close();
    link_ = nullptr;
}

void GlobalScheduler::RecvEvent(std::shared_ptr<const Event> event)
{
    if (LIKELY(link_ && link_->to_daemon.Send(event->Data(), event->Size()))) return;
    // No daemon: scheduling cannot work as configured, which is fatal
    // (global.cpp:49-55) - except while this process is going away anyway.
    if (event->Type() == kEventProcessDestroy) return;
    XERRO("failed to send event (type %d) to the scheduler daemon; is it running?", event->Type());
}

} // namespace xsched::sched
