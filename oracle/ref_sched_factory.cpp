// ORACLE - test infrastructure only; compiled ONLY into the libraries under oracle/_ref/.
//
// The reference's XQueue core is compiled from its own sources for the launch-trace
// oracle. Two of its files, sched/src/scheduler/scheduler.cpp and global.cpp, include the
// un-vendored ipc library's header and are left out; no replacement of that library is
// written. What the remaining sources still need from scheduler.cpp is the scheduler
// factory, which is given here WITHOUT the daemon branch: the trace tests run app-managed
// or with the reference's own LocalScheduler, both of which come from reference sources.
#include <memory>

#include "xsched/sched/scheduler/app_managed.h"
#include "xsched/sched/scheduler/local.h"
#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::sched
{

void Scheduler::Execute(std::shared_ptr<const Operation> operation)
{
    if (executor_) executor_(operation);
}

std::shared_ptr<Scheduler> CreateScheduler(XSchedulerType, XPolicyType policy)
{
    if (policy > kPolicyUnknown && policy < kPolicyMax) return std::make_shared<LocalScheduler>(policy);
    return std::make_shared<AppManagedScheduler>();
}

} // namespace xsched::sched
