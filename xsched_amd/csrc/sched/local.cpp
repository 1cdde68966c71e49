// The in-process scheduler: an inbox, a ledger of operations, a mirror of the XQueues, a
// heap of alarms and one thread that turns them over in rounds.
//
//   round = take everything in the inbox (or an alarm that has come due)
//           -> fold each event into the mirror (hints go to the policy)
//           -> policy.Sched(mirror): it answers by marking XQueues suspended / running
//           -> one scheduling operation per process that has XQueues
//
// What a round decides and emits (operation ids included) is that of reference
// sched/src/scheduler/local.cpp:42-446; tests replay recorded event scripts through both.
#include <algorithm>
#include <array>
#include <atomic>
#include <condition_variable>
#include <map>
#include <mutex>
#include <queue>
#include <thread>
#include <vector>

#include "global.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/names.h"
#include "xsched/sched/policy/policy.h"
#include "xsched/sched/protocol/status.h"
#include "xsched/sched/scheduler/local.h"
#include "spin.h"

using namespace xsched::protocol;

namespace xsched::sched
{

// A valid policy selects the local scheduler whatever the type says; otherwise the daemon
// client or the scheduler that does nothing (reference sched/src/scheduler/scheduler.cpp:19-34).
std::shared_ptr<Scheduler> CreateScheduler(XSchedulerType scheduler, XPolicyType policy)
{
    if (policy > kPolicyUnknown && policy < kPolicyMax) {
        XINFO("using local scheduler with policy %s", GetPolicyTypeName(policy).c_str());
        return std::make_shared<LocalScheduler>(policy);
    }
    if (scheduler == kSchedulerGlobal) {
        XINFO("using global scheduler");
        return std::make_shared<GlobalScheduler>();
    }
    XINFO("using app-managed scheduler");
    return std::make_shared<AppManagedScheduler>();
}

namespace
{

using EventPtr = std::shared_ptr<const Event>;
using Clock = std::chrono::system_clock;

/// Events waiting for the next round, and the alarms policies have set.
class Inbox
{
public:
    void Put(EventPtr event)
    {
        { std::lock_guard<std::mutex> g(mu_); waiting_.push_back(std::move(event)); }
        n_put_.fetch_add(1, std::memory_order_release);
        cv_.notify_one();
    }

    void SetAlarm(TimePoint at)
    {
        { std::lock_guard<std::mutex> g(mu_); alarms_.push(at); }
        cv_.notify_one();   // the round thread may be asleep with no alarm to wake it
    }

    void ClearAlarms()
    {
        std::lock_guard<std::mutex> g(mu_);
        while (!alarms_.empty()) alarms_.pop();
    }

    /// Blocks until there are events or an alarm is due; removes nothing but the alarms that
    /// are due (all of them together). True when an alarm ended the wait.
    bool AwaitWork()
    {
        // Poll for a while after the last batch before blocking (off unless XSCHED_SPIN_US is
        // set); alarms are looked at by the blocking path, which the poll leaves in time.
        const auto window = SpinWindow();
        if (window.count() > 0) {
            uint64_t seen;
            TimePoint give_up;
            {
                std::lock_guard<std::mutex> g(mu_);
                seen = n_taken_;
                give_up = last_batch_ + window;
                if (!alarms_.empty() && alarms_.top() < give_up) give_up = alarms_.top();
            }
            while (n_put_.load(std::memory_order_acquire) == seen && Clock::now() < give_up) __builtin_ia32_pause();
        }
        std::unique_lock<std::mutex> g(mu_);
        while (waiting_.empty()) {
            if (alarms_.empty()) { cv_.wait(g); continue; }
            const TimePoint first = alarms_.top();
            const TimePoint now = Clock::now();
            if (now < first) { cv_.wait_until(g, first); continue; }
            while (!alarms_.empty() && !(now < alarms_.top())) alarms_.pop();
            return true;
        }
        return false;
    }

    /// `batch` receives the events that are waiting (possibly none); never blocks.
    void TakeNow(std::vector<EventPtr> *batch)
    {
        batch->clear();
        std::lock_guard<std::mutex> g(mu_);
        batch->swap(waiting_);
        n_taken_ = n_put_.load(std::memory_order_acquire); // under mu_: every Put() counted so far is in the batch
        last_batch_ = Clock::now();
    }

private:
    std::mutex mu_;
    std::condition_variable cv_;
    std::vector<EventPtr> waiting_;
    std::atomic<uint64_t> n_put_ { 0 };
    uint64_t n_taken_ = 0;          // under mu_
    TimePoint last_batch_ {};       // under mu_
    std::priority_queue<TimePoint, std::vector<TimePoint>, std::greater<TimePoint>> alarms_;
};

/// Per process: the id of the newest operation sent and of the newest one reported done.
/// Kept outside the round thread's data: completions arrive on the callers' threads.
class Ledger
{
public:
    void Open(PID pid)  { { std::lock_guard<std::mutex> g(mu_); book_.try_emplace(pid); } cv_.notify_all(); }
    void Close(PID pid) { { std::lock_guard<std::mutex> g(mu_); book_.erase(pid); } cv_.notify_all(); }

    /// 0 for a process that never announced itself.
    OperationId Issue(PID pid)
    {
        std::lock_guard<std::mutex> g(mu_);
        auto it = book_.find(pid);
        return it == book_.end() ? 0 : ++it->second.sent;
    }

    void Done(PID pid, OperationId id)
    {
        {
            std::lock_guard<std::mutex> g(mu_);
            auto it = book_.find(pid);
            if (it == book_.end()) {
                XWARN("operation " FMT_64U " completed by unknown process " FMT_PID, id, pid);
                return;
            }
            XASSERT(id <= it->second.sent, "unknown operation " FMT_64U " completed", id);
            it->second.done = std::max(it->second.done, id);
        }
        cv_.notify_all();
    }

private:
    struct Line { OperationId sent = 0, done = 0; };
    std::mutex mu_;
    std::condition_variable cv_;
    std::map<PID, Line> book_;
};

/// The Status a policy reads, and the only code that edits it.
class Mirror
{
public:
    const Status &View() const { return status_; }

    ProcessStatus &Process(PID pid)
    {
        auto &slot = status_.process_status[pid];
        if (slot == nullptr) {
            slot = std::make_unique<ProcessStatus>();
            slot->info.pid = pid;
        }
        return *slot;
    }

    XQueueStatus *Find(XQueueHandle handle)
    {
        auto it = status_.xqueue_status.find(handle);
        return it == status_.xqueue_status.end() ? nullptr : it->second.get();
    }

    /// A queue heard of for the first time; it starts out running.
    XQueueStatus &Adopt(PID pid, XQueueHandle handle)
    {
        auto fresh = std::make_unique<XQueueStatus>();
        fresh->handle = handle;
        fresh->device = kDeviceTypeUnknown;
        fresh->level = kPreemptLevelUnknown;
        fresh->pid = pid;
        fresh->threshold = 0;
        fresh->batch_size = 0;
        fresh->ready = false;
        fresh->suspended = false;
        fresh->ready_time = Clock::now();
        XQueueStatus &ref = *fresh;
        status_.xqueue_status[handle] = std::move(fresh);
        Process(pid).running_xqueues.insert(handle);
        return ref;
    }

    void ForgetQueue(XQueueHandle handle, PID claimed_owner)
    {
        auto it = status_.xqueue_status.find(handle);
        if (it == status_.xqueue_status.end()) return;
        XASSERT(claimed_owner == it->second->pid, "XQueue destroyed by a process that does not own it");
        auto owner = status_.process_status.find(it->second->pid);
        if (owner == status_.process_status.end()) return;
        owner->second->running_xqueues.erase(handle);
        owner->second->suspended_xqueues.erase(handle);
        status_.xqueue_status.erase(it);
    }

    void ForgetProcess(PID pid)
    {
        auto it = status_.process_status.find(pid);
        if (it == status_.process_status.end()) return;
        for (XQueueHandle h : it->second->running_xqueues) status_.xqueue_status.erase(h);
        for (XQueueHandle h : it->second->suspended_xqueues) status_.xqueue_status.erase(h);
        status_.process_status.erase(it);
    }

    /// The policy's verdict on one queue; a verdict that changes nothing is not recorded.
    void Mark(XQueueHandle handle, bool suspended)
    {
        XQueueStatus *xq = Find(handle);
        if (xq == nullptr || xq->suspended == suspended) return;
        xq->suspended = suspended;
        auto owner = status_.process_status.find(xq->pid);
        if (owner == status_.process_status.end()) return;
        ProcessStatus &ps = *owner->second;
        auto &from = suspended ? ps.running_xqueues : ps.suspended_xqueues;
        auto &to = suspended ? ps.suspended_xqueues : ps.running_xqueues;
        from.erase(handle);
        to.insert(handle);
        (suspended ? ps.xqueues_to_suspend : ps.xqueues_to_resume).insert(handle);
    }

    void Answer(StatusQuery *query, const XQueueStatus *only)
    {
        for (auto &entry : status_.xqueue_status) {
            if (only != nullptr && entry.second.get() != only) continue;
            query->status_.emplace_back(std::make_unique<XQueueStatus>(*entry.second));
        }
        if (query->QueryProcess()) {
            for (auto &entry : status_.process_status) {
                if (only != nullptr && entry.first != only->pid) continue;
                query->processes_.emplace_back(std::make_unique<ProcessInfo>(entry.second->info));
            }
        }
    }

private:
    Status status_;
};

} // namespace

/// Up to how many queues a submitter runs the round that its own Ready event asks for
/// (XSCHED_INLINE_READY_ROUNDS_MAX_QUEUES).
static size_t MaxQueuesForSubmitterRounds()
{
    static const size_t n = []() {
        int64_t v = 8;
        return GetEnvInt64("XSCHED_INLINE_READY_ROUNDS_MAX_QUEUES", v) && v >= 0 ? (size_t)v : (size_t)8;
    }();
    return n;
}

class LocalScheduler::Rounds
{

public:
    Rounds(LocalScheduler *owner, XPolicyType type): owner_(owner) { Install(type); }

    void Install(XPolicyType type)
    {
        type_ = type;
        policy_ = CreatePolicy(type);
        policy_->SetSuspendFunc([this](XQueueHandle h) { mirror_.Mark(h, true); });
        policy_->SetResumeFunc([this](XQueueHandle h) { mirror_.Mark(h, false); });
        policy_->SetAddTimerFunc([this](TimePoint at) { inbox_.SetAlarm(at); });
    }

    void Start() { thread_ = std::thread([this]() { Turn(); }); }

    void Halt()
    {
        if (thread_.joinable()) {
            inbox_.Put(std::make_shared<SchedulerTerminateEvent>());
            thread_.join();
        }
        inbox_.ClearAlarms();
    }

    /// Ledger entries change on the caller's thread: the round thread may be the one that
    /// waits for them. A completion is never queued (reference local.cpp:42-96).
    ///
    /// With rounds on the callers' threads switched on, the thread that brings an event runs
    /// the round itself when nobody else is in one (what waits in the inbox goes first, so
    /// events are folded in the order in which they came); otherwise the event is queued and
    /// the round thread, which also keeps the alarms, takes it. That saves the wake-up of the
    /// round thread, 10-50 us when it sleeps, between an event and the operations it causes.
    void Accept(EventPtr event)
    {
        switch (event->Type()) {
        case kEventProcessCreate:  ledger_.Open(event->Pid()); break;
        case kEventProcessDestroy: ledger_.Close(event->Pid()); break;
        case kEventOperationComplete:
            ledger_.Done(event->Pid(), static_cast<const OperationCompleteEvent *>(event.get())->OpId());
            return;
        default: break;
        }
        const int mode = on_callers_.load(std::memory_order_acquire);
        const bool here = mode == kRoundsOnCallersAll || (mode == kRoundsOnCallersReady && event->Type() == kEventXQueueReady);
        if (here && round_mu_.try_lock()) {
            std::unique_lock<std::mutex> round(round_mu_, std::adopt_lock);
            // A round costs its caller a pass over every queue; for a submitter that is time
            // before its own launch. With many queues the round thread's wake-up is the
            // smaller price (measured with 16: +3 us at every queue's median).
            if (mode == kRoundsOnCallersReady && mirror_.View().xqueue_status.size() > MaxQueuesForSubmitterRounds()) {
                round.unlock();
                inbox_.Put(std::move(event));
                return;
            }
            std::vector<EventPtr> batch;
            inbox_.TakeNow(&batch);
            batch.push_back(std::move(event));
            // the terminate event is the round thread's to see: it goes back in
            if (Round(batch)) inbox_.Put(std::make_shared<SchedulerTerminateEvent>());
            return;
        }
        inbox_.Put(std::move(event));
    }

    void RoundsOnCallers(int mode) { on_callers_.store(mode, std::memory_order_release); }

    void SwitchTo(XPolicyType type)
    {
        if (type == type_) return;
        const std::string before = GetPolicyTypeName(type_);
        Halt();
        {
            std::lock_guard<std::mutex> round(round_mu_); // callers may be running rounds
            Install(type);
            // the new policy starts from "everything runs"
            std::vector<XQueueHandle> all;
            for (auto &entry : mirror_.View().xqueue_status) all.push_back(entry.first);
            for (XQueueHandle h : all) mirror_.Mark(h, false);
        }
        Start();
        XINFO("policy changed from %s to %s", before.c_str(), GetPolicyTypeName(type).c_str());
    }

    XPolicyType Type() const { return type_; }
    OperationId IssueId(PID pid) { return ledger_.Issue(pid); }

private:
    void Turn()
    {
        std::vector<EventPtr> batch;
        while (true) {
            const bool alarm = inbox_.AwaitWork();
            std::lock_guard<std::mutex> round(round_mu_);
            inbox_.TakeNow(&batch);
            if (batch.empty() && !alarm) continue;   // a caller's round has taken what woke this thread
            if (Round(batch)) return;
        }
    }

    /// One round (round_mu_ held): fold the events, ask the policy, tell the processes. True
    /// when the batch held the terminate event.
    bool Round(const std::vector<EventPtr> &batch)
    {
        bool last_round = false;
        for (auto &event : batch) {
            if (UNLIKELY(event->Type() == kEventSchedulerTerminate)) last_round = true;
            else Fold(*event);
        }
        policy_->Sched(mirror_.View());
        // one operation per process that has XQueues, whether or not anything changed
        for (auto &entry : mirror_.View().process_status) {
            const ProcessStatus &ps = *entry.second;
            if (ps.running_xqueues.empty() && ps.suspended_xqueues.empty()) continue;
            owner_->Execute(std::make_shared<SchedOperation>(ledger_.Issue(ps.info.pid), ps));
        }
        return last_round;
    }

    // ---- folding one event into the mirror, one function per event type ----------------

    void FoldHint(const Event &e) { policy_->RecvHint(static_cast<const HintEvent &>(e).GetHint()); }

    void FoldProcessCreate(const Event &e)
    {
        mirror_.Process(e.Pid()).info.cmdline = static_cast<const ProcessCreateEvent &>(e).Cmdline();
    }

    void FoldProcessDestroy(const Event &e) { mirror_.ForgetProcess(e.Pid()); }

    void FoldQueueConfig(const Event &e) // creation and configuration updates carry the same record
    {
        const auto *rec = (const XQueueConfigData *)e.Data();
        XQueueStatus *xq = mirror_.Find(rec->handle);
        if (xq == nullptr) xq = &mirror_.Adopt(e.Pid(), rec->handle);
        xq->device = rec->device;
        xq->level = rec->level;
        xq->threshold = rec->threshold;
        xq->batch_size = rec->batch_size;
    }

    void FoldQueueDestroy(const Event &e)
    {
        mirror_.ForgetQueue(static_cast<const XQueueDestroyEvent &>(e).Handle(), e.Pid());
    }

    void FoldQueueReady(const Event &e)
    {
        auto &ready = static_cast<const XQueueReadyEvent &>(e);
        XQueueStatus *xq = mirror_.Find(ready.Handle());
        if (xq == nullptr) xq = &mirror_.Adopt(e.Pid(), ready.Handle()); // ready before its creation was heard of
        xq->ready = true;
        xq->ready_time = ready.ReadyTime();
    }

    void FoldQueueIdle(const Event &e)
    {
        const XQueueHandle handle = static_cast<const XQueueIdleEvent &>(e).Handle();
        XQueueStatus *xq = mirror_.Find(handle);
        if (xq == nullptr) xq = &mirror_.Adopt(e.Pid(), handle);
        xq->ready = false;
    }

    void FoldQueryOne(const Event &e)
    {
        auto &ask = static_cast<const XQueueQueryEvent &>(e);
        StatusQuery *query = ask.QueryData();
        if (const XQueueStatus *xq = mirror_.Find(ask.Handle())) mirror_.Answer(query, xq);
        query->Notify();
    }

    void FoldQueryAll(const Event &e)
    {
        StatusQuery *query = static_cast<const XQueueQueryAllEvent &>(e).QueryData();
        mirror_.Answer(query, nullptr);
        query->Notify();
    }

    void Fold(const Event &e)
    {
        using Folder = void (Rounds::*)(const Event &);
        static const std::map<EventType, Folder> folders = {
            { kEventHint, &Rounds::FoldHint },
            { kEventProcessCreate, &Rounds::FoldProcessCreate },
            { kEventProcessDestroy, &Rounds::FoldProcessDestroy },
            { kEventXQueueCreate, &Rounds::FoldQueueConfig },
            { kEventXQueueConfigUpdate, &Rounds::FoldQueueConfig },
            { kEventXQueueDestroy, &Rounds::FoldQueueDestroy },
            { kEventXQueueReady, &Rounds::FoldQueueReady },
            { kEventXQueueIdle, &Rounds::FoldQueueIdle },
            { kEventXQueueQuery, &Rounds::FoldQueryOne },
            { kEventXQueueQueryAll, &Rounds::FoldQueryAll },
        };
        auto it = folders.find(e.Type());
        if (it != folders.end()) (this->*(it->second))(e);
    }

    LocalScheduler *const owner_;
    XPolicyType type_ = kPolicyUnknown;
    std::unique_ptr<Policy> policy_;
    Inbox inbox_;
    Ledger ledger_;
    std::mutex round_mu_;                    // the mirror, the policy, and who takes events out of the inbox
    std::atomic<int> on_callers_ { kRoundsOnCallersOff };
    Mirror mirror_;
    std::thread thread_;
};

LocalScheduler::LocalScheduler(XPolicyType type)
    : Scheduler(kSchedulerLocal), rounds_(std::make_unique<Rounds>(this, type)) {}

LocalScheduler::~LocalScheduler() { rounds_->Halt(); }

void LocalScheduler::Run() { rounds_->Start(); }
void LocalScheduler::Stop() { rounds_->Halt(); }
void LocalScheduler::RecvEvent(std::shared_ptr<const Event> event) { rounds_->Accept(std::move(event)); }
void LocalScheduler::SetPolicy(XPolicyType type) { rounds_->SwitchTo(type); }
XPolicyType LocalScheduler::GetPolicy() const { return rounds_->Type(); }
OperationId LocalScheduler::NextOperationId(PID pid) { return rounds_->IssueId(pid); }
void LocalScheduler::RunRoundsOnCallers(int mode) { rounds_->RoundsOnCallers(mode); }

} // namespace xsched::sched
