// SchedAgent: process-wide relay between the XQueues of this process and the
// active scheduler (app-managed, local, or the daemon client). Chosen from
// XSCHED_SCHEDULER / XSCHED_POLICY at load and replaceable through
// XHintSetScheduler(). Follows reference preempt/src/sched/agent.cpp:21-140.
#pragma once

#include <atomic>
#include <memory>
#include <shared_mutex>

#include "xsched/types.h"
#include "xsched/sched/protocol/event.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::preempt
{

class SchedAgent
{
public:
    SchedAgent();
    ~SchedAgent();

    static void SendHint(std::shared_ptr<const sched::Hint> hint)   { Instance().RelayHint(hint); }
    static void SendEvent(std::shared_ptr<const sched::Event> event) { Instance().RelayEvent(event); }
    static XResult SetScheduler(XSchedulerType scheduler, XPolicyType policy)
    { return Instance().ReplaceScheduler(scheduler, policy); }

    /// Whether a queue that becomes ready should tell the scheduler BEFORE it launches the
    /// command that made it so. True for the daemon client: its decision comes back through
    /// two other processes, the longest leg of a preemption, so it starts first and the
    /// event costs the submitter one datagram. False in-process: the event may run a whole
    /// scheduling round on the submitter's thread (suspensions, deactivations, replays on
    /// other queues); the command goes to the device first and the round overlaps with its
    /// way there, with none of the submitter's queue locks held.
    static bool ReadyEventGoesFirst() { return Instance().ready_event_first_.load(std::memory_order_relaxed); }

private:
    static SchedAgent &Instance();
    void RelayHint(std::shared_ptr<const sched::Hint> hint);
    void RelayEvent(std::shared_ptr<const sched::Event> event);
    XResult ReplaceScheduler(XSchedulerType scheduler, XPolicyType policy);
    void InitScheduler(XSchedulerType scheduler, XPolicyType policy);
    void FiniScheduler();

    // Relays hold it shared; replacing the scheduler holds it exclusively.
    std::shared_mutex mtx_;
    std::shared_ptr<sched::Scheduler> scheduler_;
    std::atomic<bool> ready_event_first_ { false };
};

/// Applies scheduler operations to the XQueues of this process: resume the
/// running set first, then suspend the rest (reference
/// preempt/src/sched/executor.cpp:26-102).
class SchedExecutor
{
public:
    STATIC_CLASS(SchedExecutor);
    static void Start();
    static void Stop();
    static void Execute(std::shared_ptr<const sched::Operation> op);
};

} // namespace xsched::preempt
