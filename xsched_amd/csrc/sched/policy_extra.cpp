// The policies declared in xsched/sched/policy/extra.h. Each follows the decisions of
// the reference policy it names, call for call (Suspend / Resume / AddTimer in the same
// order over the same iteration orders), because the local scheduler turns them into
// operations that tests compare with the reference's.
#include <algorithm>
#include <cmath>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "xsched/utils/log.h"
#include "xsched/utils/xassert.h"
#include "policy_extra.h"

using namespace std::chrono;

namespace xsched::sched
{

namespace
{

Priority ClampPriority(const PriorityHint &hint)
{
    Priority prio = hint.Prio();
    if (prio < PRIORITY_MIN) prio = PRIORITY_MIN;
    if (prio > PRIORITY_MAX) prio = PRIORITY_MAX;
    if (prio != hint.Prio()) {
        XWARN("priority %d of XQueue 0x" FMT_64X " clamped to %d", hint.Prio(), hint.Handle(), prio);
    }
    return prio;
}

} // namespace

// ---- one bar for all devices (reference hhpf.cpp:8-30) ---------------------------

void GlobalPriorityPolicy::Sched(const Status &status)
{
    Priority bar = PRIORITY_MIN;
    for (auto &entry : status.xqueue_status) {
        if (entry.second->ready) bar = std::max(bar, PriorityOf(entry.second->handle));
    }
    for (auto &entry : status.xqueue_status) {
        const XQueueHandle handle = entry.second->handle;
        if (PriorityOf(handle) < bar) this->Suspend(handle);
        else this->Resume(handle);
    }
}

void GlobalPriorityPolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    if (hint->Type() != kHintTypePriority) return;
    auto h = std::dynamic_pointer_cast<const PriorityHint>(hint);
    XASSERT(h != nullptr, "hint type mismatch");
    priorities_[h->Handle()] = ClampPriority(*h);
}

Priority GlobalPriorityPolicy::PriorityOf(XQueueHandle handle) const
{
    auto it = priorities_.find(handle);
    return it == priorities_.end() ? (Priority)PRIORITY_DEFAULT : it->second;
}

// ---- the process's Linux priority (reference chpf.cpp:10-62) ---------------------
// /proc/<pid>/sched: the first line that contains "prio" reads "prio : <n>"; real-time
// priorities are below 100 and count as they are, the normal range (100 and up, lower
// is better) is negated. A process whose file cannot be read has priority 0.

void ProcessPriorityPolicy::Sched(const Status &status)
{
    std::map<PID, Priority> of_process;
    for (auto &entry : status.process_status) {
        std::ifstream file("/proc/" + std::to_string(entry.first) + "/sched");
        std::string line;
        while (std::getline(file, line)) {
            if (line.find("prio") == std::string::npos) continue;
            std::istringstream in(line);
            std::string name, colon;
            Priority prio;
            in >> name >> colon >> prio;
            of_process[entry.first] = prio >= 100 ? -prio : prio;
            break;
        }
    }

    std::map<XDevice, Priority> top;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;
        const Priority prio = of_process[xq.pid];
        auto it = top.find(xq.device);
        if (it == top.end()) top.emplace(xq.device, prio);
        else if (prio > it->second) it->second = prio;
    }
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        auto it = top.find(xq.device);
        const Priority bar = it == top.end() ? (Priority)PRIORITY_MIN : it->second;
        if (of_process[xq.pid] < bar) this->Suspend(xq.handle);
        else this->Resume(xq.handle);
    }
}

// ---- one queue at a time, by utilization share (reference up.cpp:6-164) ----------
// The hinted queues take turns in handle order. The running one keeps the device until
// its budget (timeslice * share / sum of shares) is used up or it falls idle; then the
// next READY hinted queue after it (wrapping once around) takes over. If none is ready
// the policy forgets who ran and leaves everything as it is.

void QueueSharePolicy::Sched(const Status &status)
{
    for (auto it = shares_.begin(); it != shares_.end();) {
        if (status.xqueue_status.count(it->first) == 0) it = shares_.erase(it);
        else ++it;
    }
    if (current_ != 0 && status.xqueue_status.count(current_) == 0) current_ = 0;
    if (shares_.empty()) return;
    if (current_ == 0) { RunFirstReady(status); return; }

    const XQueueStatus &running = *status.xqueue_status.find(current_)->second;
    if (system_clock::now() < current_until_ && running.ready) return;

    auto mine = shares_.find(current_);
    XASSERT(mine != shares_.end(), "no utilization for the running XQueue 0x" FMT_64X, current_);

    auto ready = [&](XQueueHandle handle) {
        auto it = status.xqueue_status.find(handle);
        return it != status.xqueue_status.end() && it->second->ready;
    };
    for (auto it = std::next(mine); it != shares_.end(); ++it) {
        if (ready(it->first)) { RunOnly(it->first, it->second, status); return; }
    }
    for (auto it = shares_.begin(); it != mine; ++it) {
        if (ready(it->first)) { RunOnly(it->first, it->second, status); return; }
    }
    current_ = 0;
}

void QueueSharePolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    switch (hint->Type()) {
    case kHintTypeUtilization: {
        auto h = std::dynamic_pointer_cast<const UtilizationHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        if (h->Util() < UTILIZATION_MIN || h->Util() > UTILIZATION_MAX) {
            XWARN("utilization %d is out of range", h->Util());
            break;
        }
        shares_[h->Handle()] = h->Util();
        break;
    }
    case kHintTypeTimeslice: {
        auto h = std::dynamic_pointer_cast<const TimesliceHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        timeslice_ = microseconds(h->Ts());
        break;
    }
    default:
        XWARN("hint type %d means nothing to this policy", hint->Type());
        break;
    }
}

microseconds QueueSharePolicy::BudgetOf(Utilization share) const
{
    Utilization total = 0;
    for (auto &entry : shares_) total += entry.second;
    if (total == 0) return microseconds(TIMESLICE_DEFAULT);
    return microseconds((int64_t)timeslice_.count() * share / total);
}

void QueueSharePolicy::RunFirstReady(const Status &status)
{
    current_ = 0;
    bool chosen = false; // not "current_ != 0": handle 0 means "nobody" to Sched() only
    for (auto &entry : status.xqueue_status) {
        auto share = shares_.find(entry.first);
        if (chosen || !entry.second->ready || share == shares_.end()) {
            this->Suspend(entry.first);
            continue;
        }
        chosen = true;
        this->Resume(entry.first);
        current_ = entry.first;
        current_until_ = system_clock::now() + BudgetOf(share->second);
        this->AddTimer(current_until_);
    }
}

void QueueSharePolicy::RunOnly(XQueueHandle handle, Utilization share, const Status &status)
{
    for (auto &entry : status.xqueue_status) {
        if (entry.first != handle) this->Suspend(entry.first);
    }
    this->Resume(handle);
    current_ = handle;
    current_until_ = system_clock::now() + BudgetOf(share);
    this->AddTimer(current_until_);
}

// ---- one process at a time (reference pup.cpp:7-200) -----------------------------
// Processes that own XQueues wait in a run queue. The one at the front runs until its
// slice ends or none of its queues is ready; it then goes to the back and keeps what was
// left of the slice as budget. Processes at the front that are not ready go to the back
// too, their budget grown by one share. A budget above one share loses a tenth of the
// excess each time it is topped up.

void ProcessSharePolicy::Sched(const Status &status)
{
    const TimePoint now = system_clock::now();

    for (auto it = shares_.begin(); it != shares_.end();) {
        if (status.process_status.count(it->first) == 0) it = shares_.erase(it);
        else ++it;
    }

    auto owns_queues = [](const ProcessStatus &ps) {
        return !ps.running_xqueues.empty() || !ps.suspended_xqueues.empty();
    };
    bool any_ready = false;
    for (auto it = turns_.begin(); it != turns_.end();) {
        auto ps = status.process_status.find(it->pid);
        if (ps == status.process_status.end() || !owns_queues(*ps->second)) {
            queued_.erase(it->pid);
            it = turns_.erase(it);
            continue;
        }
        it->ready = AnyQueueReady(it->pid, status);
        any_ready = any_ready || it->ready;
        ++it;
    }
    for (auto &entry : status.process_status) {
        if (!owns_queues(*entry.second) || queued_.count(entry.first) != 0) continue;
        const bool ready = AnyQueueReady(entry.first, status);
        any_ready = any_ready || ready;
        turns_.push_back(Turn { entry.first, ready, false, 0 });
        queued_.insert(entry.first);
    }
    if (turns_.empty() || !any_ready) return;

    if (turns_.front().running) {
        const bool slice_left = slice_end_ > now;
        const Turn front = turns_.front();
        if (slice_left && front.ready) return;
        turns_.pop_front();
        const int64_t left_us = slice_left ? duration_cast<microseconds>(slice_end_ - now).count() : 0;
        turns_.push_back(Turn { front.pid, front.ready, false, left_us });
    }

    while (!turns_.front().ready) {
        const Turn front = turns_.front();
        const int64_t budget = BudgetWithCarry(front.pid, front.budget_us);
        turns_.pop_front();
        turns_.push_back(Turn { front.pid, false, false, budget });
    }

    const PID next = turns_.front().pid;
    slice_end_ = now + microseconds(BudgetWithCarry(next, turns_.front().budget_us));
    this->AddTimer(slice_end_);
    GiveDeviceTo(next, status);
}

void ProcessSharePolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    switch (hint->Type()) {
    case kHintTypeUtilization: {
        auto h = std::dynamic_pointer_cast<const UtilizationHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        if (h->Pid() == 0) break;
        if (h->Util() < UTILIZATION_MIN || h->Util() > UTILIZATION_MAX) {
            XWARN("utilization %d is out of range", h->Util());
            break;
        }
        shares_[h->Pid()] = h->Util();
        break;
    }
    case kHintTypeTimeslice: {
        auto h = std::dynamic_pointer_cast<const TimesliceHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        if (h->Ts() < TIMESLICE_MIN || h->Ts() > TIMESLICE_MAX) {
            XWARN("timeslice " FMT_64D " is out of range", h->Ts());
            break;
        }
        slice_us_ = h->Ts();
        break;
    }
    default:
        XWARN("hint type %d means nothing to this policy", hint->Type());
        break;
    }
}

/// One share: the average slice times the number of queued processes, split by
/// utilization (100 for a process without a hint).
int64_t ProcessSharePolicy::ShareUs(PID pid) const
{
    auto share_of = [this](PID p) -> int64_t {
        auto it = shares_.find(p);
        return it == shares_.end() ? (int64_t)UTILIZATION_DEFAULT : (int64_t)it->second;
    };
    int64_t total = 0;
    for (auto &turn : turns_) total += share_of(turn.pid);
    if (total == 0) return 0;
    return (int64_t)((uint64_t)slice_us_ * turns_.size() * (uint64_t)share_of(pid) / (uint64_t)total);
}

int64_t ProcessSharePolicy::BudgetWithCarry(PID pid, int64_t carried) const
{
    const int64_t share = ShareUs(pid);
    if (carried > share) carried = (int64_t)((double)share + (double)(carried - share) * 0.9);
    return carried + share;
}

bool ProcessSharePolicy::AnyQueueReady(PID pid, const Status &status)
{
    auto ps = status.process_status.find(pid);
    XASSERT(ps != status.process_status.end(), "process " FMT_PID " is not in the status", pid);
    auto ready = [&](XQueueHandle handle) {
        auto it = status.xqueue_status.find(handle);
        return it != status.xqueue_status.end() && it->second->ready;
    };
    for (XQueueHandle handle : ps->second->running_xqueues) if (ready(handle)) return true;
    for (XQueueHandle handle : ps->second->suspended_xqueues) if (ready(handle)) return true;
    return false;
}

/// Resumes the suspended queues of `pid`, suspends the running queues of every other
/// queued process. The sets are copied first: the callbacks edit them.
void ProcessSharePolicy::GiveDeviceTo(PID pid, const Status &status)
{
    for (auto &turn : turns_) {
        auto ps = status.process_status.find(turn.pid);
        if (ps == status.process_status.end()) continue;
        turn.running = turn.pid == pid;
        if (turn.running) {
            const std::vector<XQueueHandle> handles(ps->second->suspended_xqueues.begin(), ps->second->suspended_xqueues.end());
            for (XQueueHandle handle : handles) this->Resume(handle);
        } else {
            const std::vector<XQueueHandle> handles(ps->second->running_xqueues.begin(), ps->second->running_xqueues.end());
            for (XQueueHandle handle : handles) this->Suspend(handle);
        }
    }
}

// ---- k earliest deadlines (reference kedf.cpp:10-78) -----------------------------
// A queue that is idle or has no deadline hint sorts last (deadline = end of time).
// The order among equal deadlines is whatever std::sort leaves, as in the reference.

void EarliestDeadlinePolicy::Sched(const Status &status)
{
    struct Due { XQueueHandle handle; TimePoint at; };
    std::vector<Due> due;
    due.reserve(status.xqueue_status.size());
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        TimePoint at = (TimePoint::max)();
        auto hinted = deadlines_.find(xq.handle);
        if (xq.ready && hinted != deadlines_.end()) at = xq.ready_time + microseconds(hinted->second);
        due.push_back(Due { xq.handle, at });
    }
    std::sort(due.begin(), due.end(), [](const Due &a, const Due &b) { return a.at < b.at; });

    for (size_t i = 0; i < k_ && i < due.size(); ++i) this->Resume(due[i].handle);
    for (size_t i = k_; i < due.size(); ++i) this->Suspend(due[i].handle);
}

void EarliestDeadlinePolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    switch (hint->Type()) {
    case kHintTypeDeadline: {
        auto h = std::dynamic_pointer_cast<const DeadlineHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        deadlines_[h->Handle()] = h->Ddl();
        break;
    }
    case kHintTypeKDeadline: {
        auto h = std::dynamic_pointer_cast<const KDeadlineHint>(hint);
        XASSERT(h != nullptr, "hint type mismatch");
        if (h->K() < 1) { XWARN("k must be at least 1"); break; }
        k_ = h->K();
        break;
    }
    default:
        XWARN("hint type %d means nothing to this policy", hint->Type());
        break;
    }
}

// ---- the active window's process first (reference awf.cpp:6-51) ------------------

void ActiveWindowPolicy::Sched(const Status &status)
{
    bool active_ready = false;
    for (auto &entry : status.xqueue_status) {
        if (entry.second->ready && active_.count(entry.second->pid) != 0) { active_ready = true; break; }
    }
    for (auto &entry : status.xqueue_status) {
        if (!active_ready || active_.count(entry.second->pid) != 0) this->Resume(entry.first);
        else this->Suspend(entry.first);
    }
}

void ActiveWindowPolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    if (hint->Type() != kHintTypeWindowActive) return;
    auto h = std::dynamic_pointer_cast<const WindowActiveHint>(hint);
    XASSERT(h != nullptr, "hint type mismatch");
    if (h->Pid() == 0) return;
    // one active process per display
    auto it = by_display_.find(h->Display());
    if (it != by_display_.end()) active_.erase(it->second);
    active_.insert(h->Pid());
    by_display_[h->Display()] = h->Pid();
}

// ---- least weighted run time first (reference cfs.cpp:10-124) --------------------
// vruntime(q) grows by elapsed microseconds * 1024 / weight(q) while q runs. A queue
// seen ready for the first time starts at the least vruntime among the device's ready
// queues that already have an account. Idle queues get an account too (at zero) when
// they are first looked at in the last pass, exactly as the reference's map does.

void FairSharePolicy::Sched(const Status &status)
{
    const TimePoint now = system_clock::now();

    for (auto &entry : status.xqueue_status) {
        auto it = accounts_.find(entry.second->handle);
        if (it == accounts_.end() || !it->second.running) continue;
        const int64_t ran_us = duration_cast<microseconds>(now - it->second.resumed_at).count();
        it->second.vruntime += ran_us * (1024.0 / it->second.weight);
    }

    bool any_ready = false;
    std::map<XDevice, double> least;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;
        any_ready = true;
        auto it = accounts_.find(xq.handle);
        if (it == accounts_.end()) continue;
        auto low = least.find(xq.device);
        if (low == least.end()) least.emplace(xq.device, it->second.vruntime);
        else if (it->second.vruntime < low->second) low->second = it->second.vruntime;
    }

    std::map<XDevice, XQueueHandle> chosen;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;
        if (accounts_.find(xq.handle) == accounts_.end()) {
            Account fresh;
            fresh.resumed_at = now;
            auto low = least.find(xq.device);
            fresh.vruntime = low == least.end() ? 0.0 : low->second;
            if (low == least.end()) least.emplace(xq.device, fresh.vruntime);
            accounts_[xq.handle] = fresh;
        }
        auto pick = chosen.find(xq.device);
        if (pick == chosen.end()) chosen.emplace(xq.device, xq.handle);
        else if (accounts_[xq.handle].vruntime < accounts_[pick->second].vruntime) pick->second = xq.handle;
    }

    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        Account &account = accounts_[xq.handle];
        if (!xq.ready) { account.running = false; continue; }
        if (chosen[xq.device] == xq.handle) {
            if (!account.running) this->Resume(xq.handle);
            account.running = true;
            account.resumed_at = now;
        } else {
            this->Suspend(xq.handle);
            account.running = false;
        }
    }

    if (any_ready) this->AddTimer(now + slice_);
}

void FairSharePolicy::RecvHint(std::shared_ptr<const Hint> hint)
{
    if (hint->Type() != kHintTypePriority) return;
    auto h = std::dynamic_pointer_cast<const PriorityHint>(hint);
    if (h == nullptr) return;
    Account &account = accounts_[h->Handle()];
    account.priority = h->Prio();
    account.weight = 1024.0 * std::pow(1.2, h->Prio());
}

// ---- feedback levels (reference mlfq.cpp:7-173) ----------------------------------

void FeedbackLevelsPolicy::Sched(const Status &status)
{
    const TimePoint now = system_clock::now();
    auto us_between = [](TimePoint from, TimePoint to) { return duration_cast<microseconds>(to - from); };

    // ready / idle edges
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        auto it = entries_.find(xq.handle);
        if (it == entries_.end()) {
            Entry fresh;
            fresh.idle_since = fresh.level_since = fresh.requested_at = fresh.pending_since = fresh.resumed_at = now;
            it = entries_.emplace(xq.handle, fresh).first;
        }
        Entry &e = it->second;
        if (xq.ready && !e.was_ready) { e.requested_at = now; e.pending_since = now; }
        else if (!xq.ready && e.was_ready) e.idle_since = now;
        e.was_ready = xq.ready;
    }

    // ready queues per device and level, as the levels stand before this round
    std::map<XDevice, std::map<int, int>> crowd;
    for (auto &entry : status.xqueue_status) {
        if (entry.second->ready) crowd[entry.second->device][entries_[entry.second->handle].level]++;
    }

    bool any_ready = false;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        Entry &e = entries_[xq.handle];
        if (!xq.ready) continue;
        any_ready = true;

        if (!e.running) {
            e.pending += us_between(e.pending_since, now);
            e.pending_since = now;
        } else {
            e.slice_used += us_between(e.resumed_at, now);
            e.resumed_at = now;
        }

        // rise: time since the level last changed, minus the pending time discounted by
        // 0.9 / (queues sharing the level), exceeds the threshold
        const int sharing = crowd[xq.device][e.level];
        const double discount = sharing > 1 ? 0.9 / sharing : 1.0;
        const double effective = us_between(e.level_since, now).count() - e.pending.count() * discount;
        if (effective > kRecoveryUs) {
            if (e.level > 0) e.level--;
            e.level_since = now;
            e.pending = microseconds(0);
            e.slice_used = microseconds(0);
        }

        // drop: the slice of the level is used up
        if (e.running && e.slice_used >= SliceOf(e.level)) {
            if (e.level < kLowestLevel) e.level++;
            e.level_since = now;
            e.slice_used = microseconds(0);
            e.pending = microseconds(0);
            e.running = false;
            this->Suspend(xq.handle);
            e.pending_since = now;
        }
    }

    // best level per device; among equals the one that has been pending longest
    std::map<XDevice, XQueueHandle> chosen;
    std::map<XDevice, int> best_level;
    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        if (!xq.ready) continue;
        const Entry &e = entries_[xq.handle];
        auto best = best_level.find(xq.device);
        if (best == best_level.end() || e.level < best->second) {
            best_level[xq.device] = e.level;
            chosen[xq.device] = xq.handle;
        } else if (e.level == best->second && e.pending > entries_[chosen[xq.device]].pending) {
            chosen[xq.device] = xq.handle;
        }
    }

    for (auto &entry : status.xqueue_status) {
        const XQueueStatus &xq = *entry.second;
        Entry &e = entries_[xq.handle];
        if (!xq.ready) { e.running = false; continue; }
        if (chosen[xq.device] == xq.handle) {
            if (!e.running) {
                this->Resume(xq.handle);
                e.running = true;
                e.pending_since = now;
            }
            e.resumed_at = now;
        } else if (e.running) {
            this->Suspend(xq.handle);
            e.running = false;
            e.pending_since = now;
        }
    }

    if (any_ready) this->AddTimer(now + microseconds(kTickUs));
}

} // namespace xsched::sched
