// Scheduler: consumes events, emits operations through an executor callback.
// Interface follows reference sched/include/xsched/sched/scheduler/scheduler.h:12-36.
#pragma once

#include <functional>
#include <memory>

#include "xsched/types.h"
#include "xsched/sched/protocol/event.h"
#include "xsched/sched/protocol/operation.h"

namespace xsched::sched
{

typedef std::function<void(std::shared_ptr<const Operation>)> Executor;

class Scheduler
{
public:
    explicit Scheduler(XSchedulerType type): kType(type) {}
    virtual ~Scheduler() = default;

    virtual void Run() = 0;
    virtual void Stop() = 0;
    virtual void RecvEvent(std::shared_ptr<const Event> event) = 0;

    XSchedulerType GetType() const { return kType; }
    void SetExecutor(Executor executor) { executor_ = executor; }

protected:
    void Execute(std::shared_ptr<const Operation> operation) { if (executor_) executor_(operation); }

private:
    const XSchedulerType kType;
    Executor executor_ = nullptr;
};

/// A valid policy selects the local scheduler; otherwise kSchedulerGlobal selects
/// the daemon client and everything else the app-managed (no-op) scheduler
/// (reference sched/src/scheduler/scheduler.cpp:19-34).
std::shared_ptr<Scheduler> CreateScheduler(XSchedulerType scheduler, XPolicyType policy);

/// Application drives Suspend/Resume itself; events are dropped.
class AppManagedScheduler : public Scheduler
{
public:
    AppManagedScheduler(): Scheduler(kSchedulerAppManaged) {}
    virtual void Run() override {}
    virtual void Stop() override {}
    virtual void RecvEvent(std::shared_ptr<const Event>) override {}
};

} // namespace xsched::sched
