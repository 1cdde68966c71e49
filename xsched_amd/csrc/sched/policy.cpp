// The two policies of the preemptible-queue path (HPF, LAX) and the policy factory;
// the other policies live in policy_extra.cpp.
// reference sched/src/policy/{policy,hpf,lax}.cpp
#include <map>
#include <unordered_map>

#include "xsched/utils/xassert.h"
#include "policy_extra.h"
#include "xsched/sched/policy/policy.h"

namespace xsched::sched
{

std::unique_ptr<Policy> MakePriorityBarPolicy();
std::unique_ptr<Policy> MakeLaxityBarPolicy();

bool PolicyAvailable(XPolicyType type)
{
    return type > kPolicyUnknown && type < kPolicyMax && type != kPolicyStrictProcessUtilizationPartition;
}

std::unique_ptr<Policy> CreatePolicy(XPolicyType type)
{
    switch (type) {
    case kPolicyHighestPriorityFirst: return MakePriorityBarPolicy();
    case kPolicyLaxity:               return MakeLaxityBarPolicy();
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

// ---- the two policies of the preemptible-queue path -----------------------------------------
// Both are "bar" policies: every XQueue has an effective priority, the bar is the highest one
// among READY queues of a scope, and a queue below its scope's bar is suspended while every
// other queue runs. They differ in what the effective priority is and in the scope:
//
//   HPF  the hinted priority (default PRIORITY_DEFAULT, clamped to the valid range);
//        one bar per device (reference sched/src/policy/hpf.cpp:8-68)
//   LAX  lax_prio until `laxity` us after the queue became ready (and while it is not
//        ready), crit_prio from then on, PRIORITY_DEFAULT without a hint; ONE bar for all
//        devices; the earliest expiry still ahead among ready hinted queues is asked for as
//        a timer (reference sched/src/policy/lax.cpp:8-72)

namespace
{

/// Highest effective priority among ready queues, per scope key; a scope without a ready
/// queue has no entry and its bar is PRIORITY_MIN (nothing below it).
class Bars
{
public:
    void Raise(uint64_t scope, Priority prio)
    {
        auto [it, fresh] = top_.emplace(scope, prio);
        if (!fresh && prio > it->second) it->second = prio;
    }
    Priority Of(uint64_t scope) const
    {
        auto it = top_.find(scope);
        return it == top_.end() ? (Priority)PRIORITY_MIN : it->second;
    }
private:
    std::map<uint64_t, Priority> top_;
};

class PriorityBarPolicy final : public Policy
{
public:
    PriorityBarPolicy(): Policy(kPolicyHighestPriorityFirst) {}

    void Sched(const Status &status) override
    {
        Bars bars;
        for (auto &entry : status.xqueue_status) {
            if (entry.second->ready) bars.Raise(entry.second->device, Hinted(entry.first));
        }
        for (auto &entry : status.xqueue_status) {
            if (Hinted(entry.first) < bars.Of(entry.second->device)) Suspend(entry.first);
            else Resume(entry.first);
        }
    }

    void RecvHint(std::shared_ptr<const Hint> hint) override
    {
        if (hint->Type() != kHintTypePriority) return;
        auto *h = static_cast<const PriorityHint *>(hint.get());
        const Priority asked = h->Prio();
        const Priority kept = asked < PRIORITY_MIN ? (Priority)PRIORITY_MIN
                            : asked > PRIORITY_MAX ? (Priority)PRIORITY_MAX : asked;
        if (kept != asked) XWARN("priority %d of XQueue 0x" FMT_64X " clamped to %d", asked, h->Handle(), kept);
        hinted_[h->Handle()] = kept;
    }

private:
    Priority Hinted(XQueueHandle handle) const
    {
        auto it = hinted_.find(handle);
        return it == hinted_.end() ? (Priority)PRIORITY_DEFAULT : it->second;
    }
    std::unordered_map<XQueueHandle, Priority> hinted_;
};

class LaxityBarPolicy final : public Policy
{
public:
    LaxityBarPolicy(): Policy(kPolicyLaxity) {}

    void Sched(const Status &status) override
    {
        const TimePoint now = std::chrono::system_clock::now();
        Bars bars; // one scope
        bool alarm = false;
        TimePoint earliest = (TimePoint::max)();
        for (auto &entry : status.xqueue_status) {
            const XQueueStatus &xq = *entry.second;
            if (!xq.ready) continue;
            bars.Raise(0, Effective(xq, now));
            auto it = terms_.find(xq.handle);
            if (it == terms_.end()) continue;
            const TimePoint expiry = xq.ready_time + std::chrono::microseconds(it->second.lax);
            if (now < expiry && expiry < earliest) { earliest = expiry; alarm = true; }
        }
        for (auto &entry : status.xqueue_status) {
            if (Effective(*entry.second, now) < bars.Of(0)) Suspend(entry.first);
            else Resume(entry.first);
        }
        if (alarm) AddTimer(earliest);
    }

    void RecvHint(std::shared_ptr<const Hint> hint) override
    {
        if (hint->Type() != kHintTypeLaxity) return;
        auto *h = static_cast<const LaxityHint *>(hint.get());
        terms_[h->Handle()] = Terms { h->Lax() < 0 ? (Laxity)NO_LAXITY : h->Lax(), h->LaxPrio(), h->CritPrio() };
    }

private:
    struct Terms { Laxity lax; Priority relaxed; Priority critical; };

    Priority Effective(const XQueueStatus &xq, TimePoint now) const
    {
        auto it = terms_.find(xq.handle);
        if (it == terms_.end()) return PRIORITY_DEFAULT;
        const TimePoint expiry = xq.ready_time + std::chrono::microseconds(it->second.lax);
        return (!xq.ready || now < expiry) ? it->second.relaxed : it->second.critical;
    }
    std::unordered_map<XQueueHandle, Terms> terms_;
};

} // namespace

std::unique_ptr<Policy> MakePriorityBarPolicy() { return std::make_unique<PriorityBarPolicy>(); }
std::unique_ptr<Policy> MakeLaxityBarPolicy() { return std::make_unique<LaxityBarPolicy>(); }

} // namespace xsched::sched
