// LocalScheduler: the in-process scheduler. Events go in through RecvEvent(); a thread of its
// own folds them into a mirror of every XQueue and process, asks the policy once per round
// and hands one scheduling operation per process to the executor. The public face is what
// the scheduler daemon and the agent use (reference
// sched/include/xsched/sched/scheduler/local.h:20-36); everything else is private to
// csrc/sched/local.cpp.
#pragma once

#include <memory>

#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::sched
{

class LocalScheduler : public Scheduler
{
public:
    explicit LocalScheduler(XPolicyType type);
    ~LocalScheduler() override;

    void Run() override;
    void Stop() override;
    void RecvEvent(std::shared_ptr<const Event> event) override;

    /// Stops, installs the new policy, marks every XQueue as running and starts again; the
    /// next round tells the processes.
    void SetPolicy(XPolicyType type);
    XPolicyType GetPolicy() const;
    /// The id for an operation the caller is about to send to process `pid` itself (the
    /// daemon's configuration requests); 0 for a process that never announced itself.
    OperationId NextOperationId(PID pid);
    /// Lets the thread that brings an event run the scheduling round itself when no other
    /// round is under way, instead of waking the scheduler's own thread for it: for every
    /// event (owners whose event-bringing threads hold no lock that an operation could need:
    /// the daemon's receiver), or for XQueueReady events only (in-process: the submitter
    /// holds its queue's ring lock, which suspending and resuming OTHER queues does not need;
    /// a resume can take tens of microseconds of launches and stays with the round thread).
    enum { kRoundsOnCallersOff = 0, kRoundsOnCallersReady = 1, kRoundsOnCallersAll = 2 };
    void RunRoundsOnCallers(int mode);

private:
    class Rounds;
    std::unique_ptr<Rounds> rounds_;
};

} // namespace xsched::sched
