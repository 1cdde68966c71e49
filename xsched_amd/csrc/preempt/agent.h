// SchedAgent: process-wide relay between the XQueues of this process and the
// active scheduler (app-managed, local, or the daemon client). Chosen from
// XSCHED_SCHEDULER / XSCHED_POLICY at load and replaceable through
// XHintSetScheduler(). Follows reference preempt/src/sched/agent.cpp:21-140.
#pragma once

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
