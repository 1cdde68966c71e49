// The two policies of the preemptible-queue path (HPF, LAX) and the policy factory;
// the other policies live in policy_extra.cpp.
// reference sched/src/policy/{policy,hpf,lax}.cpp
#include <map>

#include "xsched/utils/xassert.h"
#include "xsched/sched/policy/extra.h"
#include "xsched/sched/policy/hpf.h"
#include "xsched/sched/policy/lax.h"
#include "xsched/sched/policy/policy.h"

namespace xsched::sched
{

bool PolicyAvailable(XPolicyType type)
{
    return type > kPolicyUnknown && type < kPolicyMax && type != kPolicyStrictProcessUtilizationPartition;
}

std::unique_ptr<Policy> CreatePolicy(XPolicyType type)
{
    switch (type) {
    case kPolicyHighestPriorityFirst: return std::make_unique<HighestPriorityFirstPolicy>();
    case kPolicyLaxity:               return std::make_unique<LaxityPolicy>();
    case kPolicyHeterogeneousHighestPriorityFirst: return std::make_unique<GlobalPriorityPolicy>();
    case kPolicyCPUHighestPriorityFirst:           return std::make_unique<ProcessPriorityPolicy>();
    case kPolicyUtilizationPartition:              return std::make_unique<QueueSharePolicy>();
    case kPolicyProcessUtilizationPartition:       return std::make_unique<ProcessSharePolicy>();
    case kPolicyKEarliestDeadlineFirst:            return std::make_unique<EarliestDeadlinePolicy>();
    case kPolicyActiveWindowFirst:                 return std::make_unique<ActiveWindowPolicy>();
    case kPolicyCompletelyFairScheduler:           return std::make_unique<FairSharePolicy>();
    case kPolicyMultiLevelFeedbackQueue:           return std::make_unique<FeedbackLevelsPolicy>();
    default:
        // reference policy.cpp:39-69 knows no other type either (the strict variant of the
        // process partition is declared in types.h but has no class)
        XASSERT(false, "invalid policy type: %d", type);
        return nullptr;
    }
}

// ---- Highest Priority First (reference hpf.cpp:8-68) ------------------------
// Pass 1: per device, the highest priority among READY queues.
// Pass 2: every queue (ready or not) strictly below its device's maximum is
// suspended, all others resumed. A device without a ready queue has maximum
// PRIORITY_MIN, so nothing on it is suspended.

void HighestPriorityFirstPolicy::Sched(const Status &status)
{
    std::map<XDevice, Priority> top;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;
        const Priority prio = PriorityOf(xq.handle);
        auto it = top.find(xq.device);
        if (it == top.end()) top.emplace(xq.device, prio);
        else if (prio > it->second) it->second = prio;
    }

    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        auto it = top.find(xq.device);
        const Priority bar = it == top.end() ? (Priority)PRIORITY_MIN : it->second;
        if (PriorityOf(xq.handle) < bar) this->Suspend(xq.handle);
        else this->Resume(xq.handle);
    }
}

void HighestPriorityFirstPolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    if (hint->Type() != kHintTypePriority) return;
    auto h = std::dynamic_pointer_cast<const PriorityHint>(hint);
    XASSERT(h != nullptr, "hint type mismatch");

    Priority prio = h->Prio();
    if (prio < PRIORITY_MIN) prio = PRIORITY_MIN;
    if (prio > PRIORITY_MAX) prio = PRIORITY_MAX;
    if (prio != h->Prio()) {
        XWARN("priority %d of XQueue 0x" FMT_64X " clamped to %d", h->Prio(), h->Handle(), prio);
    }
    priorities_[h->Handle()] = prio;
}

Priority HighestPriorityFirstPolicy::PriorityOf(XQueueHandle handle) const
{
    auto it = priorities_.find(handle);
    return it == priorities_.end() ? (Priority)PRIORITY_DEFAULT : it->second;
}

// ---- Laxity (reference lax.cpp:8-72) ----------------------------------------
// expiry(q)    = ready_time(q) + laxity(q)
// effective(q) = lax_prio while q is not ready or now < expiry(q), else crit_prio;
//                PRIORITY_DEFAULT for queues without a hint
// bar          = max effective priority over READY queues (PRIORITY_MIN if none)
// Queues below the bar are suspended. The earliest expiry still in the future
// among ready hinted queues becomes a timer so the decision is re-evaluated then.

void LaxityPolicy::Sched(const Status &status)
{
    const TimePoint now = test_now_us_ != 0
        ? TimePoint(std::chrono::microseconds(test_now_us_))
        : std::chrono::system_clock::now();

    Priority bar = PRIORITY_MIN;
    bool have_timer = false;
    TimePoint next_expiry = (TimePoint::max)();

    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;

        auto it = laxity_infos_.find(xq.handle);
        if (it == laxity_infos_.end()) {
            if (PRIORITY_DEFAULT > bar) bar = PRIORITY_DEFAULT;
            continue;
        }
        const TimePoint expiry = xq.ready_time + std::chrono::microseconds(it->second.lax);
        const Priority prio = now < expiry ? it->second.lax_prio : it->second.crit_prio;
        if (prio > bar) bar = prio;
        if (now < expiry && expiry < next_expiry) {
            next_expiry = expiry;
            have_timer = true;
        }
    }

    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        Priority prio = PRIORITY_DEFAULT;
        auto it = laxity_infos_.find(xq.handle);
        if (it != laxity_infos_.end()) {
            const TimePoint expiry = xq.ready_time + std::chrono::microseconds(it->second.lax);
            prio = (!xq.ready || now < expiry) ? it->second.lax_prio : it->second.crit_prio;
        }
        if (prio < bar) this->Suspend(xq.handle);
        else this->Resume(xq.handle);
    }

    if (have_timer) this->AddTimer(next_expiry);
}

void LaxityPolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    if (hint->Type() != kHintTypeLaxity) return;
    auto h = std::dynamic_pointer_cast<const LaxityHint>(hint);
    XASSERT(h != nullptr, "hint type mismatch");
    laxity_infos_[h->Handle()] = LaxityInfo {
        h->Lax() < 0 ? (Laxity)NO_LAXITY : h->Lax(), h->LaxPrio(), h->CritPrio()
    };
}

} // namespace xsched::sched
