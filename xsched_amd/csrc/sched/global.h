// GlobalScheduler: client side of the scheduler daemon. Events are forwarded as
// raw records to the daemon; a receiver thread executes the operations it sends
// back. Role follows reference sched/src/scheduler/global.cpp:17-69; the
// transport is this build's own datagram channel (see xsched/sched/ipc/channel.h)
// because the reference's channel library is not part of its source tree.
#pragma once

#include <memory>
#include <thread>

#include "xsched/sched/ipc/channel.h"
#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::sched
{

class GlobalScheduler : public Scheduler
{
public:
    GlobalScheduler();
    virtual ~GlobalScheduler();

    virtual void Run() override;
    virtual void Stop() override;
    virtual void RecvEvent(std::shared_ptr<const Event> event) override;

private:
    void Worker();

    ipc::ChannelKey client_key_ = 0;
    std::unique_ptr<std::thread> thread_;
    std::unique_ptr<ipc::Node> recv_chan_;
    std::unique_ptr<ipc::Node> send_chan_;
};

} // namespace xsched::sched
