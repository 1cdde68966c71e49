// Daemon client. reference sched/src/scheduler/global.cpp:17-69
#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "global.h"

namespace xsched::sched
{

GlobalScheduler::GlobalScheduler(): Scheduler(kSchedulerGlobal) {}
GlobalScheduler::~GlobalScheduler() { this->Stop(); }

// The client listens on a channel keyed by its pid and talks to the daemon's
// well-known channel. The receiver exists before the first event is sent, so the
// daemon can answer the ProcessCreate event right away.
void GlobalScheduler::Run()
{
    client_key_ = (ipc::ChannelKey)GetProcessId();
    recv_chan_ = std::make_unique<ipc::Node>(client_key_, ipc::NodeType::kReceiver);
    send_chan_ = std::make_unique<ipc::Node>((ipc::ChannelKey)XSCHED_SERVER_CHANNEL_KEY,
                                             ipc::NodeType::kSender);
    thread_ = std::make_unique<std::thread>(&GlobalScheduler::Worker, this);
}

void GlobalScheduler::Stop()
{
    if (thread_) {
        // Wake the receiver with a terminate record sent to ourselves.
        TerminateOperation op;
        ipc::Node self(client_key_, ipc::NodeType::kSender);
        if (!self.Send(op.Data(), op.Size())) recv_chan_->Remove();
        thread_->join();
        thread_ = nullptr;
    }
    if (recv_chan_) { recv_chan_->Remove(); recv_chan_ = nullptr; }
    if (send_chan_) { send_chan_->Remove(); send_chan_ = nullptr; }
}

void GlobalScheduler::RecvEvent(std::shared_ptr<const Event> event)
{
    if (LIKELY(send_chan_ && send_chan_->Send(event->Data(), event->Size()))) return;
    // No daemon: scheduling cannot work as configured, which is fatal
    // (global.cpp:49-55) - except while this process is going away anyway.
    if (event->Type() == kEventProcessDestroy) return;
    XERRO("failed to send event (type %d) to the scheduler daemon; is it running?", event->Type());
}

void GlobalScheduler::Worker()
{
    while (true) {
        auto msg = recv_chan_->Receive();
        if (msg == nullptr) return;
        if (!Operation::WireRecordOk(msg->Data(), msg->Size())) {
            XWARN("dropped a malformed operation record of %zu bytes", msg->Size());
            continue;
        }
        auto op = Operation::CopyConstructor(msg->Data());
        if (UNLIKELY(op->Type() == kOperationTerminate)) return;
        Execute(op);
    }
}

} // namespace xsched::sched
