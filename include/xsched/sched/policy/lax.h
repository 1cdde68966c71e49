// Laxity policy: an XQueue runs at its lax priority until `laxity` microseconds
// after it became ready, then at its critical priority; queues below the highest
// effective ready priority are suspended (reference sched/src/policy/lax.cpp:8-72).
#pragma once

#include <unordered_map>

#include "xsched/sched/policy/policy.h"

namespace xsched::sched
{

class LaxityPolicy : public Policy
{
public:
    LaxityPolicy(): Policy(kPolicyLaxity) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

    /// Test seam: a fixed "now" instead of the system clock (0 = system clock).
    void SetNowForTest(int64_t now_us) { test_now_us_ = now_us; }

private:
    struct LaxityInfo { Laxity lax; Priority lax_prio; Priority crit_prio; };
    std::unordered_map<XQueueHandle, LaxityInfo> laxity_infos_;
    int64_t test_now_us_ = 0;
};

} // namespace xsched::sched
