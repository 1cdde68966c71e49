// In-process scheduler. reference sched/src/scheduler/{local,scheduler}.cpp
#include <algorithm>

#include "xsched/utils/xassert.h"
#include "xsched/protocol/names.h"
#include "xsched/sched/scheduler/global.h"
#include "xsched/sched/scheduler/local.h"
#include "xsched/sched/scheduler/scheduler.h"

using namespace std::chrono;
using namespace xsched::protocol;

namespace xsched::sched
{

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

LocalScheduler::LocalScheduler(XPolicyType type): Scheduler(kSchedulerLocal), policy_type_(type)
{
    InstallPolicy(type);
}

LocalScheduler::~LocalScheduler() { this->Stop(); }

void LocalScheduler::InstallPolicy(XPolicyType type)
{
    policy_type_ = type;
    policy_ = CreatePolicy(type);
    policy_->SetSuspendFunc([this](XQueueHandle h) { this->Suspend(h); });
    policy_->SetResumeFunc([this](XQueueHandle h) { this->Resume(h); });
    policy_->SetAddTimerFunc([this](TimePoint tp) { this->AddTimer(tp); });
}

void LocalScheduler::Run()
{
    thread_ = std::make_unique<std::thread>(&LocalScheduler::Worker, this);
}

void LocalScheduler::Stop()
{
    if (thread_) {
        this->RecvEvent(std::make_shared<SchedulerTerminateEvent>());
        thread_->join();
        thread_ = nullptr;
    }
    timers_.clear();
}

// Operation bookkeeping is updated right here on the caller's thread, because the
// worker thread itself may sit in WaitAllOperations() (local.cpp:42-96).
void LocalScheduler::RecvEvent(std::shared_ptr<const Event> event)
{
    switch (event->Type()) {
    case kEventProcessCreate:
    {
        { std::lock_guard<std::mutex> lock(op_mtx_); ops_.try_emplace(event->Pid()); }
        op_cv_.notify_all();
        break;
    }
    case kEventProcessDestroy:
    {
        { std::lock_guard<std::mutex> lock(op_mtx_); ops_.erase(event->Pid()); }
        op_cv_.notify_all();
        break;
    }
    case kEventOperationComplete:
    {
        auto done = static_cast<const OperationCompleteEvent *>(event.get());
        {
            std::lock_guard<std::mutex> lock(op_mtx_);
            auto it = ops_.find(done->Pid());
            if (it == ops_.end()) {
                XWARN("operation " FMT_64U " completed by unknown process " FMT_PID,
                      done->OpId(), done->Pid());
                return;
            }
            XASSERT(done->OpId() <= it->second.issued_id,
                    "unknown operation " FMT_64U " completed", done->OpId());
            it->second.completed_id = std::max(it->second.completed_id, done->OpId());
        }
        op_cv_.notify_all();
        return; // not queued
    }
    default:
        break;
    }

    { std::lock_guard<std::mutex> lock(event_mtx_); event_queue_.emplace_back(std::move(event)); }
    event_cv_.notify_one();
}

void LocalScheduler::SetPolicy(XPolicyType type)
{
    if (type == policy_type_) return;
    const std::string old = GetPolicyTypeName(policy_type_);
    this->Stop();
    InstallPolicy(type);
    // Start the new policy from "everything runs".
    for (auto &status : status_.xqueue_status) Resume(status.first);
    this->Run();
    XINFO("policy changed from %s to %s", old.c_str(), GetPolicyTypeName(type).c_str());
}

void LocalScheduler::WaitAllOperations()
{
    std::unique_lock<std::mutex> lock(op_mtx_);
    op_cv_.wait(lock, [this]() {
        for (auto &p : ops_) if (p.second.completed_id < p.second.issued_id) return false;
        return true;
    });
}

void LocalScheduler::WaitOperations(PID pid)
{
    std::unique_lock<std::mutex> lock(op_mtx_);
    op_cv_.wait(lock, [this, pid]() {
        auto it = ops_.find(pid);
        return it == ops_.end() || it->second.completed_id >= it->second.issued_id;
    });
}

OperationId LocalScheduler::NextOperationId(PID pid)
{
    std::lock_guard<std::mutex> lock(op_mtx_);
    auto it = ops_.find(pid);
    return it == ops_.end() ? 0 : ++(it->second.issued_id);
}

// One round = take every queued event, fold it into Status, run the policy once,
// send one SchedOperation per process. Rounds are triggered by events or by the
// earliest timer a policy asked for (local.cpp:142-196).
void LocalScheduler::Worker()
{
    std::vector<std::shared_ptr<const Event>> batch;
    std::unique_lock<std::mutex> lock(event_mtx_);

    while (true) {
        while (event_queue_.empty()) {
            if (timers_.empty()) { event_cv_.wait(lock); continue; }
            const auto first = timers_.front();
            const auto now = system_clock::now();
            if (now < first) { event_cv_.wait_until(lock, first); continue; }
            while (!timers_.empty() && !(now < timers_.front())) timers_.pop_front();
            break;
        }
        batch.clear();
        batch.swap(event_queue_);
        lock.unlock();

        bool terminate = false;
        for (auto &event : batch) {
            if (UNLIKELY(event->Type() == kEventSchedulerTerminate)) { terminate = true; continue; }
            this->UpdateStatus(*event);
        }

        policy_->Sched(status_);
        this->ExecuteOperations();
        std::sort(timers_.begin(), timers_.end());
        if (terminate) return;
        lock.lock();
    }
}

void LocalScheduler::ExecuteOperations()
{
    for (auto &entry : status_.process_status) {
        ProcessStatus &ps = *entry.second;
        if (ps.running_xqueues.empty() && ps.suspended_xqueues.empty()) continue;
        Execute(std::make_shared<SchedOperation>(NextOperationId(ps.info.pid), ps));
    }
}

void LocalScheduler::CreateXQueueStatus(PID pid, XQueueHandle handle, XDevice device,
                                        XPreemptLevel level, int64_t threshold,
                                        int64_t batch_size, bool ready,
                                        system_clock::time_point ready_time)
{
    auto xq = std::make_unique<XQueueStatus>();
    xq->handle = handle;
    xq->device = device;
    xq->level = level;
    xq->pid = pid;
    xq->threshold = threshold;
    xq->batch_size = batch_size;
    xq->ready = ready;
    xq->suspended = false;
    xq->ready_time = ready_time;
    status_.xqueue_status[handle] = std::move(xq);

    auto &ps = status_.process_status[pid];
    if (ps == nullptr) {
        ps = std::make_unique<ProcessStatus>();
        ps->info.pid = pid;
    }
    ps->running_xqueues.insert(handle);
}

void LocalScheduler::UpdateStatus(const Event &event)
{
    switch (event.Type()) {
    case kEventHint:
        policy_->RecvHint(static_cast<const HintEvent &>(event).GetHint());
        break;
    case kEventProcessCreate:
    {
        auto &e = static_cast<const ProcessCreateEvent &>(event);
        auto &ps = status_.process_status[e.Pid()];
        if (ps == nullptr) {
            ps = std::make_unique<ProcessStatus>();
            ps->info.pid = e.Pid();
        }
        ps->info.cmdline = e.Cmdline();
        break;
    }
    case kEventProcessDestroy:
    {
        auto pit = status_.process_status.find(event.Pid());
        if (pit == status_.process_status.end()) break;
        for (XQueueHandle h : pit->second->running_xqueues)   status_.xqueue_status.erase(h);
        for (XQueueHandle h : pit->second->suspended_xqueues) status_.xqueue_status.erase(h);
        status_.process_status.erase(pit);
        break;
    }
    case kEventXQueueCreate:
    case kEventXQueueConfigUpdate:
    {
        // Both carry the same record (XQueueConfigData).
        auto *d = (const XQueueConfigData *)event.Data();
        auto it = status_.xqueue_status.find(d->handle);
        if (it == status_.xqueue_status.end()) {
            CreateXQueueStatus(event.Pid(), d->handle, d->device, d->level,
                               d->threshold, d->batch_size, false, system_clock::now());
        } else {
            it->second->device = d->device;
            it->second->level = d->level;
            it->second->threshold = d->threshold;
            it->second->batch_size = d->batch_size;
        }
        break;
    }
    case kEventXQueueDestroy:
    {
        auto &e = static_cast<const XQueueDestroyEvent &>(event);
        auto qit = status_.xqueue_status.find(e.Handle());
        if (qit == status_.xqueue_status.end()) break;
        const PID pid = qit->second->pid;
        XASSERT(e.Pid() == pid, "XQueue destroyed by a process that does not own it");
        auto pit = status_.process_status.find(pid);
        if (pit == status_.process_status.end()) break;
        pit->second->running_xqueues.erase(e.Handle());
        pit->second->suspended_xqueues.erase(e.Handle());
        status_.xqueue_status.erase(qit);
        break;
    }
    case kEventXQueueReady:
    {
        auto &e = static_cast<const XQueueReadyEvent &>(event);
        auto it = status_.xqueue_status.find(e.Handle());
        if (it == status_.xqueue_status.end()) {
            CreateXQueueStatus(e.Pid(), e.Handle(), kDeviceTypeUnknown, kPreemptLevelUnknown,
                               0, 0, true, e.ReadyTime());
        } else {
            it->second->ready = true;
            it->second->ready_time = e.ReadyTime();
        }
        break;
    }
    case kEventXQueueIdle:
    {
        auto &e = static_cast<const XQueueIdleEvent &>(event);
        auto it = status_.xqueue_status.find(e.Handle());
        if (it == status_.xqueue_status.end()) {
            CreateXQueueStatus(e.Pid(), e.Handle(), kDeviceTypeUnknown, kPreemptLevelUnknown,
                               0, 0, false, system_clock::now());
        } else {
            it->second->ready = false;
        }
        break;
    }
    case kEventXQueueQuery:
    {
        auto &e = static_cast<const XQueueQueryEvent &>(event);
        StatusQuery *query = e.QueryData();
        auto it = status_.xqueue_status.find(e.Handle());
        if (it != status_.xqueue_status.end()) {
            query->status_.emplace_back(std::make_unique<XQueueStatus>(*it->second));
            if (query->QueryProcess()) {
                auto pit = status_.process_status.find(it->second->pid);
                if (pit != status_.process_status.end()) {
                    query->processes_.emplace_back(std::make_unique<ProcessInfo>(pit->second->info));
                }
            }
        }
        query->Notify();
        break;
    }
    case kEventXQueueQueryAll:
    {
        auto &e = static_cast<const XQueueQueryAllEvent &>(event);
        StatusQuery *query = e.QueryData();
        for (auto &s : status_.xqueue_status) {
            query->status_.emplace_back(std::make_unique<XQueueStatus>(*s.second));
        }
        if (query->QueryProcess()) {
            for (auto &p : status_.process_status) {
                query->processes_.emplace_back(std::make_unique<ProcessInfo>(p.second->info));
            }
        }
        query->Notify();
        break;
    }
    default:
        break;
    }
}

void LocalScheduler::Suspend(XQueueHandle handle)
{
    auto qit = status_.xqueue_status.find(handle);
    if (qit == status_.xqueue_status.end() || qit->second->suspended) return;
    qit->second->suspended = true;

    auto pit = status_.process_status.find(qit->second->pid);
    if (pit == status_.process_status.end()) return;
    pit->second->running_xqueues.erase(handle);
    pit->second->suspended_xqueues.insert(handle);
    pit->second->xqueues_to_suspend.insert(handle);
}

void LocalScheduler::Resume(XQueueHandle handle)
{
    auto qit = status_.xqueue_status.find(handle);
    if (qit == status_.xqueue_status.end() || !qit->second->suspended) return;
    qit->second->suspended = false;

    auto pit = status_.process_status.find(qit->second->pid);
    if (pit == status_.process_status.end()) return;
    pit->second->running_xqueues.insert(handle);
    pit->second->suspended_xqueues.erase(handle);
    pit->second->xqueues_to_resume.insert(handle);
}

void LocalScheduler::AddTimer(const system_clock::time_point tp) { timers_.push_back(tp); }

} // namespace xsched::sched
