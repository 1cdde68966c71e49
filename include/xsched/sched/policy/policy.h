// Policy: a pure decision function over the scheduler's Status. It answers with
// Suspend()/Resume() calls per XQueue and may ask to be run again at a time
// point. Interface follows reference sched/include/xsched/sched/policy/policy.h:14-44.
#pragma once

#include <chrono>
#include <functional>
#include <memory>

#include "xsched/types.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/protocol/status.h"

namespace xsched::sched
{

typedef std::chrono::system_clock::time_point TimePoint;
typedef std::function<void (const TimePoint)> AddTimerFunc;
typedef std::function<void (const XQueueHandle)> OperateFunc;

class Policy
{
public:
    explicit Policy(XPolicyType type): kType(type) {}
    virtual ~Policy() = default;

    void SetSuspendFunc(OperateFunc suspend) { suspend_func_ = suspend; }
    void SetResumeFunc(OperateFunc resume) { resume_func_ = resume; }
    void SetAddTimerFunc(AddTimerFunc add_timer) { add_timer_func_ = add_timer; }

    virtual void Sched(const Status &status) = 0;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) = 0;

    const XPolicyType kType;

protected:
    void Suspend(XQueueHandle xqueue)       { if (suspend_func_) suspend_func_(xqueue); }
    void Resume(XQueueHandle xqueue)        { if (resume_func_) resume_func_(xqueue); }
    void AddTimer(const TimePoint tp)       { if (add_timer_func_) add_timer_func_(tp); }

private:
    OperateFunc suspend_func_ = nullptr;
    OperateFunc resume_func_ = nullptr;
    AddTimerFunc add_timer_func_ = nullptr;
};

/// Whether CreatePolicy() has a class for the type (every named type except the strict
/// process partition, which the reference declares but never implemented either).
bool PolicyAvailable(XPolicyType type);

/// Fatal for a type without a class.
std::unique_ptr<Policy> CreatePolicy(XPolicyType type);

} // namespace xsched::sched
