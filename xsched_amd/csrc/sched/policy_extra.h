// The policies beyond HPF and LAX: one class each behind the Policy interface,
// behaviour as in the reference's sched/src/policy/{hhpf,chpf,up,pup,kedf,awf,cfs,mlfq}.cpp
// (every class comment cites the lines it follows). They are pure host logic over the
// scheduler's Status mirror; the preemptible-queue path itself only needs HPF and LAX.
#pragma once

#include <chrono>
#include <list>
#include <map>
#include <set>
#include <unordered_map>
#include <unordered_set>

#include "xsched/types.h"
#include "xsched/sched/policy/policy.h"

namespace xsched::sched
{

/// HPF with one bar for the whole machine instead of one per device
/// (reference hhpf.cpp:8-56).
class GlobalPriorityPolicy : public Policy
{
public:
    GlobalPriorityPolicy(): Policy(kPolicyHeterogeneousHighestPriorityFirst) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    Priority PriorityOf(XQueueHandle handle) const;
    std::unordered_map<XQueueHandle, Priority> priorities_;
};

/// HPF per device where a queue's priority is the Linux scheduling priority of its
/// process, read from /proc/<pid>/sched at every round; hints are ignored
/// (reference chpf.cpp:10-72).
class ProcessPriorityPolicy : public Policy
{
public:
    ProcessPriorityPolicy(): Policy(kPolicyCPUHighestPriorityFirst) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint>) override {}
};

/// Time-slices ONE queue at a time; a queue's share of the timeslice is its
/// utilization hint over the sum of all hints (reference up.cpp:6-164).
class QueueSharePolicy : public Policy
{
public:
    QueueSharePolicy(): Policy(kPolicyUtilizationPartition) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    std::chrono::microseconds BudgetOf(Utilization share) const;
    void RunFirstReady(const Status &status);
    void RunOnly(XQueueHandle handle, Utilization share, const Status &status);

    XQueueHandle current_ = 0;
    TimePoint current_until_;
    std::map<XQueueHandle, Utilization> shares_;
    std::chrono::microseconds timeslice_ { TIMESLICE_DEFAULT };
};

/// Time-slices one PROCESS at a time through a run queue; unused time is carried
/// over as budget, decaying by a tenth of what exceeds one share
/// (reference pup.cpp:7-200).
class ProcessSharePolicy : public Policy
{
public:
    ProcessSharePolicy(): Policy(kPolicyProcessUtilizationPartition) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    struct Turn { PID pid; bool ready; bool running; int64_t budget_us; };
    int64_t ShareUs(PID pid) const;
    int64_t BudgetWithCarry(PID pid, int64_t carried) const;
    static bool AnyQueueReady(PID pid, const Status &status);
    void GiveDeviceTo(PID pid, const Status &status);

    std::list<Turn> turns_;
    std::set<PID> queued_;
    std::map<PID, Utilization> shares_;
    TimePoint slice_end_ = (TimePoint::min)();
    Timeslice slice_us_ = TIMESLICE_DEFAULT;
};

/// The k ready queues with the earliest deadline (ready time + hinted deadline) run
/// (reference kedf.cpp:10-78).
class EarliestDeadlinePolicy : public Policy
{
public:
    EarliestDeadlinePolicy(): Policy(kPolicyKEarliestDeadlineFirst) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    size_t k_ = 1;
    std::unordered_map<XQueueHandle, Deadline> deadlines_;
};

/// While a process that owns the active window of some display has a ready queue,
/// only the queues of such processes run (reference awf.cpp:6-51).
class ActiveWindowPolicy : public Policy
{
public:
    ActiveWindowPolicy(): Policy(kPolicyActiveWindowFirst) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    std::unordered_set<PID> active_;
    std::unordered_map<uint64_t, PID> by_display_;
};

/// Per device the ready queue with the least weighted run time runs for a 1 ms slice;
/// the weight is 1024 * 1.2^priority (reference cfs.cpp:10-124).
class FairSharePolicy : public Policy
{
public:
    FairSharePolicy(): Policy(kPolicyCompletelyFairScheduler) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint> hint) override;

private:
    struct Account
    {
        double weight = 1024.0;
        double vruntime = 0.0;
        TimePoint resumed_at;
        bool running = false;
        Priority priority = PRIORITY_DEFAULT;
    };
    std::unordered_map<XQueueHandle, Account> accounts_;
    std::chrono::microseconds slice_ { 1000 };
};

/// Four feedback levels per device: a queue that uses up its slice (10 ms << level)
/// drops a level, one that has waited 100 ms beyond its discounted pending time rises
/// one; the best level runs, longest-pending first (reference mlfq.cpp:7-173).
class FeedbackLevelsPolicy : public Policy
{
public:
    FeedbackLevelsPolicy(): Policy(kPolicyMultiLevelFeedbackQueue) {}
    virtual void Sched(const Status &status) override;
    virtual void RecvHint(std::shared_ptr<const Hint>) override {}

private:
    struct Entry
    {
        int level = 0;
        bool running = false;
        bool was_ready = false;
        TimePoint idle_since, level_since, requested_at, pending_since, resumed_at;
        std::chrono::microseconds pending { 0 };
        std::chrono::microseconds slice_used { 0 };
    };
    static constexpr int kLowestLevel = 3;
    static constexpr int64_t kRecoveryUs = 100000;
    static constexpr int64_t kTickUs = 5000;
    static std::chrono::microseconds SliceOf(int level) { return std::chrono::microseconds(10000 * (1 << level)); }

    std::map<XQueueHandle, Entry> entries_;
};

} // namespace xsched::sched
