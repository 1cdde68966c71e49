// Highest-Priority-First: per device, only the ready XQueues of the highest
// priority run (reference sched/src/policy/hpf.cpp:8-68).
#pragma once

#include <unordered_map>

#include "xsched/sched/policy/policy.h"

namespace xsched::sched
{

class HighestPriorityFirstPolicy : public Policy
{
public:
    HighestPriorityFirstPolicy(): Policy(kPolicyHighestPriorityFirst) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    Priority PriorityOf(XQueueHandle handle) const;
    std::unordered_map<XQueueHandle, Priority> priorities_;
};

} // namespace xsched::sched
