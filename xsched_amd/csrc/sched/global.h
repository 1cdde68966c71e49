// GlobalScheduler: client side of the scheduler daemon. Events are forwarded as
// raw records to the daemon; a receiver thread executes the operations it sends
// back. Role follows reference sched/src/scheduler/global.cpp:17-69; the
// transport is this build's own datagram channel (see xsched/sched/ipc/channel.h)
// because the reference's channel library is not part of its source tree.
#pragma once

#include <memory>

#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::sched
{

class GlobalScheduler : public Scheduler
{
public:
    GlobalScheduler();
    ~GlobalScheduler() override;

    void Run() override;
    void Stop() override;
    void RecvEvent(std::shared_ptr<const Event> event) override;

private:
    /// The two ends of the conversation with the daemon and the thread that listens;
    /// exists between Run() and Stop().
    struct DaemonLink;
    std::unique_ptr<DaemonLink> link_;
};

} // namespace xsched::sched
