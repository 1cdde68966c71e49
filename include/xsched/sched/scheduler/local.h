// LocalScheduler: in-process scheduler. One worker thread drains an event queue,
// updates the Status mirror, runs the policy and emits one SchedOperation per
// process; completion of operations is tracked per process. Behaviour follows
// reference sched/src/scheduler/local.cpp:12-446.
#pragma once

#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "xsched/sched/policy/policy.h"
#include "xsched/sched/protocol/status.h"
#include "xsched/sched/scheduler/scheduler.h"

namespace xsched::sched
{

class LocalScheduler : public Scheduler
{
public:
    explicit LocalScheduler(XPolicyType type);
    virtual ~LocalScheduler();

    virtual void Run() override;
    virtual void Stop() override;
    virtual void RecvEvent(std::shared_ptr<const Event> event) override;

    void SetPolicy(XPolicyType type);
    XPolicyType GetPolicy() const { return policy_type_; }

    void WaitAllOperations();
    void WaitOperations(PID pid);
    OperationId NextOperationId(PID pid);

private:
    void InstallPolicy(XPolicyType type);
    void Worker();
    void ExecuteOperations();
    void CreateXQueueStatus(PID pid, XQueueHandle handle, XDevice dev, XPreemptLevel level,
                            int64_t threshold, int64_t batch_size, bool ready,
                            std::chrono::system_clock::time_point ready_time);
    void UpdateStatus(const Event &event);
    void Suspend(XQueueHandle handle);
    void Resume(XQueueHandle handle);
    void AddTimer(const std::chrono::system_clock::time_point tp);

    Status status_;
    std::deque<std::chrono::system_clock::time_point> timers_;

    XPolicyType policy_type_;
    std::unique_ptr<Policy> policy_;
    std::unique_ptr<std::thread> thread_;

    std::mutex event_mtx_;
    std::condition_variable event_cv_;
    std::vector<std::shared_ptr<const Event>> event_queue_;

    struct OperationInfo { OperationId issued_id = 0; OperationId completed_id = 0; };
    std::mutex op_mtx_;
    std::condition_variable op_cv_;
    std::map<PID, OperationInfo> ops_;
};

} // namespace xsched::sched
