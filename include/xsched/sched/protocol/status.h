// The scheduler's mirror of every XQueue and process it manages; policies read
// it. Field set follows reference sched/include/xsched/sched/protocol/status.h:17-70.
#pragma once

#include <chrono>
#include <condition_variable>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "xsched/types.h"
#include "xsched/utils/common.h"

namespace xsched::sched
{

struct XQueueStatus
{
    XQueueHandle  handle;
    XDevice       device;
    XPreemptLevel level;
    PID           pid;
    int64_t       threshold;
    int64_t       batch_size;
    bool          ready;      // has work (kQueueStateReady)
    bool          suspended;  // as last decided by the policy
    std::chrono::system_clock::time_point ready_time; // of the latest Idle -> Ready edge
};

struct ProcessInfo
{
    PID pid;
    std::string cmdline;
};

struct ProcessStatus
{
    ProcessInfo info;
    std::set<XQueueHandle> running_xqueues;
    std::set<XQueueHandle> suspended_xqueues;
    std::set<XQueueHandle> xqueues_to_resume;
    std::set<XQueueHandle> xqueues_to_suspend;
};

struct Status
{
    std::map<XQueueHandle, std::unique_ptr<XQueueStatus>> xqueue_status;
    std::map<PID, std::unique_ptr<ProcessStatus>> process_status;
};

/// Rendezvous object for an in-process status query: the asker waits, the
/// scheduler thread fills the vectors and notifies.
class StatusQuery
{
public:
    explicit StatusQuery(bool query_process) : kQueryProcess(query_process) {}

    void Wait();
    void Notify();
    void Reset();
    bool QueryProcess() const { return kQueryProcess; }

    std::vector<std::unique_ptr<XQueueStatus>> status_;
    std::vector<std::unique_ptr<ProcessInfo>> processes_;

private:
    const bool kQueryProcess;
    bool ready_ = false;
    std::mutex mtx_;
    std::condition_variable cv_;
};

} // namespace xsched::sched
