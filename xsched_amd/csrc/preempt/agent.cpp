// Scheduler agent, operation executor and the XHint* C exports.
// reference preempt/src/sched/{agent,executor,hint}.cpp
#include <atomic>
#include <cstdlib>
#include <fstream>

#include "xsched/hint.h"
#include "xsched/xqueue.h"
#include "xsched/utils/env.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "xsched/protocol/names.h"
#include "agent.h"
#include "xsched/preempt/xqueue/xqueue.h"
#include "xsched/sched/policy/policy.h"
#include "xsched/sched/scheduler/local.h"

using namespace xsched::sched;
using namespace xsched::protocol;

namespace xsched::preempt
{

namespace
{

std::atomic_bool g_executing { false };

std::string ProcessCmdline()
{
    std::string cmdline, arg;
    std::ifstream f("/proc/self/cmdline");
    while (f.good() && std::getline(f, arg, '\0') && !arg.empty()) cmdline += arg + " ";
    const size_t cap = ProcessCreateEvent::CmdlineCapacity() - 1;
    if (cmdline.size() > cap) {
        // Keep head and tail, like the reference's ShrinkString (utils/str.h).
        const size_t head = (cap - 3 + 1) / 2, tail = cap - 3 - head;
        cmdline = cmdline.substr(0, head) + "..." + cmdline.substr(cmdline.size() - tail);
    }
    return cmdline;
}

} // namespace

// The agent lives for the whole process and is never destroyed: XQueues owned by
// static objects may still send events while the process exits. An atexit hook
// reports the process as gone and stops the scheduler; later events are dropped.
SchedAgent &SchedAgent::Instance()
{
    static SchedAgent *agent = []() {
        auto *a = new SchedAgent();
        std::atexit([]() { Instance().FiniScheduler(); SchedExecutor::Stop(); });
        return a;
    }();
    return *agent;
}

SchedAgent::SchedAgent()
{
    XSchedulerType scheduler = kSchedulerUnknown;
    XPolicyType policy = kPolicyUnknown;
    const std::string scheduler_str = GetEnv(XSCHED_SCHEDULER_ENV_NAME);
    const std::string policy_str = GetEnv(XSCHED_POLICY_ENV_NAME);
    if (!scheduler_str.empty()) scheduler = GetSchedulerType(scheduler_str);
    if (!policy_str.empty()) policy = GetPolicyType(policy_str);

    SchedExecutor::Start();
    InitScheduler(scheduler, policy);
}

SchedAgent::~SchedAgent() { FiniScheduler(); }

void SchedAgent::RelayHint(std::shared_ptr<const Hint> hint)
{
    std::shared_lock<std::shared_mutex> lock(mtx_);
    if (scheduler_ == nullptr) {
        XWARN("scheduler not initialized, hint type(%d) dropped", hint->Type());
        return;
    }
    scheduler_->RecvEvent(std::make_shared<HintEvent>(hint));
}

void SchedAgent::RelayEvent(std::shared_ptr<const Event> event)
{
    std::shared_lock<std::shared_mutex> lock(mtx_);
    if (scheduler_ == nullptr) return; // shutting down
    scheduler_->RecvEvent(event);
}

void SchedAgent::InitScheduler(XSchedulerType scheduler_type, XPolicyType policy_type)
{
    auto scheduler = CreateScheduler(scheduler_type, policy_type);
    scheduler->SetExecutor(SchedExecutor::Execute);
    if (auto local = std::dynamic_pointer_cast<LocalScheduler>(scheduler)) {
        // A queue that becomes ready is what preempts others: its submitter runs that round
        // itself instead of waking the scheduler's thread (10-50 us when it sleeps). Only
        // when a suspension waits for nothing: with one of the wait flags it would need the
        // ring lock of the queue it suspends, which a submitter may be holding - its own.
        const bool waits = GetEnvOption(XSCHED_SCHEDULER_SUSPEND_WAIT_ALL_ENV_NAME, false) ||
                           GetEnvOption(XSCHED_SCHEDULER_SUSPEND_WAIT_IDLE_ENV_NAME, false) ||
                           GetEnvOption(XSCHED_SCHEDULER_SUSPEND_SYNC_HWQ_ENV_NAME, false);
        if (!waits && GetEnvOption("XSCHED_INLINE_READY_ROUNDS", true)) local->RunRoundsOnCallers(LocalScheduler::kRoundsOnCallersReady);
    }
    scheduler->Run();
    static const std::string cmdline = ProcessCmdline();
    scheduler->RecvEvent(std::make_shared<ProcessCreateEvent>(cmdline));

    std::unique_lock<std::shared_mutex> lock(mtx_);
    scheduler_ = scheduler;
    ready_event_first_.store(scheduler->GetType() == kSchedulerGlobal, std::memory_order_relaxed);
}

void SchedAgent::FiniScheduler()
{
    std::shared_ptr<Scheduler> scheduler;
    {
        std::unique_lock<std::shared_mutex> lock(mtx_);
        scheduler.swap(scheduler_);
    }
    if (scheduler == nullptr) return;
    scheduler->RecvEvent(std::make_shared<ProcessDestroyEvent>());
    scheduler->Stop();
}

XResult SchedAgent::ReplaceScheduler(XSchedulerType scheduler_type, XPolicyType policy_type)
{
    if (scheduler_type <= kSchedulerUnknown || scheduler_type >= kSchedulerMax) {
        XWARN("invalid scheduler type: %d", scheduler_type);
        return kXSchedErrorInvalidValue;
    }

    std::shared_ptr<Scheduler> current;
    {
        std::shared_lock<std::shared_mutex> lock(mtx_);
        current = scheduler_;
    }
    if (current == nullptr) {
        XWARN("scheduler not initialized, replace scheduler failed");
        return kXSchedErrorUnknown;
    }

    if (current->GetType() == scheduler_type) {
        if (scheduler_type != kSchedulerLocal) return kXSchedSuccess;
        if (!PolicyAvailable(policy_type)) {
            XWARN("invalid policy type: %d", policy_type);
            return kXSchedErrorInvalidValue;
        }
        auto local = std::dynamic_pointer_cast<LocalScheduler>(current);
        XASSERT(local != nullptr, "scheduler is not a local scheduler");
        local->SetPolicy(policy_type);
        return kXSchedSuccess;
    }

    // A local scheduler is selected by its policy (see CreateScheduler()).
    if (scheduler_type == kSchedulerLocal && !PolicyAvailable(policy_type)) {
        XWARN("invalid policy type: %d", policy_type);
        return kXSchedErrorInvalidValue;
    }
    if (scheduler_type != kSchedulerLocal) policy_type = kPolicyUnknown;

    FiniScheduler();
    InitScheduler(scheduler_type, policy_type);
    return kXSchedSuccess;
}

// ---- executor --------------------------------------------------------------

void SchedExecutor::Start() { g_executing.store(true); }
void SchedExecutor::Stop()  { g_executing.store(false); }

static void ExecuteSched(const SchedOperation &op)
{
    static const int64_t suspend_flags =
        (GetEnvOption(XSCHED_SCHEDULER_SUSPEND_SYNC_HWQ_ENV_NAME, false)  ? kQueueSuspendFlagSyncHwQueue : 0) |
        (GetEnvOption(XSCHED_SCHEDULER_SUSPEND_WAIT_ALL_ENV_NAME, false)  ? kQueueSuspendFlagWaitAll     : 0) |
        (GetEnvOption(XSCHED_SCHEDULER_SUSPEND_WAIT_IDLE_ENV_NAME, false) ? kQueueSuspendFlagWaitIdle    : 0);

    const size_t running = op.RunningCnt();
    const size_t suspended = op.SuspendedCnt();
    const XQueueHandle *handles = op.Handles();

    // Resume first so the device never sits idle between the two halves. A handle
    // may be gone already: operations are asynchronous to XQueue destruction.
    for (size_t i = 0; i < running; ++i) {
        if (auto xq = XQueueManager::Get(handles[i])) xq->Resume(kQueueResumeFlagNone);
    }
    for (size_t i = 0; i < suspended; ++i) {
        if (auto xq = XQueueManager::Get(handles[running + i])) xq->Suspend(suspend_flags);
    }
}

static void ExecuteConfig(const ConfigOperation &op)
{
    if (op.Level() > kPreemptLevelUnknown) {
        XResult res = XQueueSetPreemptLevel(op.Handle(), op.Level());
        if (res != kXSchedSuccess) {
            XWARN("XQueueSetPreemptLevel failed, xq: 0x" FMT_64X ", level: %d, result: %d",
                  op.Handle(), op.Level(), res);
        }
    }
    if (op.Threshold() > 0 || op.BatchSize() > 0) {
        XResult res = XQueueSetLaunchConfig(op.Handle(), op.Threshold(), op.BatchSize());
        if (res != kXSchedSuccess) {
            XWARN("XQueueSetLaunchConfig failed, xq: 0x" FMT_64X ", threshold: " FMT_64D
                  ", batch size: " FMT_64D ", result: %d", op.Handle(), op.Threshold(),
                  op.BatchSize(), res);
        }
    }
}

void SchedExecutor::Execute(std::shared_ptr<const Operation> op)
{
    XASSERT(op->Pid() == GetProcessId(),
            "operation " FMT_64U " sent to the wrong process, target: " FMT_PID ", receiver " FMT_PID,
            op->Id(), op->Pid(), GetProcessId());

    const OperationType type = g_executing.load() ? op->Type() : kOperationNone;
    switch (type) {
    case kOperationNone:   break;
    case kOperationSched:  ExecuteSched(static_cast<const SchedOperation &>(*op)); break;
    case kOperationConfig: ExecuteConfig(static_cast<const ConfigOperation &>(*op)); break;
    default: XERRO("unsupported operation type: %d", type);
    }
    SchedAgent::SendEvent(std::make_shared<OperationCompleteEvent>(op->Id()));
}

} // namespace xsched::preempt

using namespace xsched::preempt;

// ---- XHint* (reference hint.cpp:12-71) --------------------------------------

#define REQUIRE_XQUEUE(handle) \
    do { XResult r_ = XQueueManager::Exists(handle); \
         if (r_ != kXSchedSuccess) { \
             XWARN("XQueue with handle 0x" FMT_64X " does not exist", handle); return r_; } } while (0)

EXPORT_C_FUNC XResult XHintSetScheduler(XSchedulerType scheduler, XPolicyType policy)
{
    return SchedAgent::SetScheduler(scheduler, policy);
}

EXPORT_C_FUNC XResult XHintPriority(XQueueHandle xq, Priority prio)
{
    REQUIRE_XQUEUE(xq);
    SchedAgent::SendHint(std::make_shared<PriorityHint>(xq, prio));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XHintUtilization(XQueueHandle xq, Utilization util)
{
    REQUIRE_XQUEUE(xq);
    SchedAgent::SendHint(std::make_shared<UtilizationHint>(GetProcessId(), xq, util));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XHintTimeslice(Timeslice ts_us)
{
    SchedAgent::SendHint(std::make_shared<TimesliceHint>(ts_us));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XHintLaxity(XQueueHandle xq, Laxity lax_us, Priority lax_prio, Priority crit_prio)
{
    REQUIRE_XQUEUE(xq);
    SchedAgent::SendHint(std::make_shared<LaxityHint>(xq, lax_us, lax_prio, crit_prio));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XHintDeadline(XQueueHandle xq, Deadline ddl_us)
{
    REQUIRE_XQUEUE(xq);
    SchedAgent::SendHint(std::make_shared<DeadlineHint>(xq, ddl_us));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XHintKDeadline(size_t k)
{
    SchedAgent::SendHint(std::make_shared<KDeadlineHint>(k));
    return kXSchedSuccess;
}
