// ORACLE - test infrastructure only. A C interface over XSched's scheduling classes
// (Policy, LocalScheduler, Status, Hint / Event / Operation records, name tables). The SAME source is
// compiled twice:
//   * against the reference's own headers and sources under /root/reference
//     (oracle/_ref/libsched_ref.so, symbols ref_*), and
//   * against this repository's headers and libpreempt.so
//     (oracle/libsched_probe.so, symbols probe_*),
// so tests can feed both the same inputs and compare decisions and wire bytes. That
// it compiles against both also shows the two class interfaces agree at source level.
#include <chrono>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "xsched/types.h"
#include "xsched/protocol/device.h"
#include "xsched/protocol/names.h"
#include "xsched/sched/policy/policy.h"
#include "xsched/sched/protocol/event.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/protocol/operation.h"
#include "xsched/sched/protocol/status.h"
#include "xsched/sched/scheduler/local.h"

#ifndef DRV_PREFIX
#error "define DRV_PREFIX (ref_ or probe_)"
#endif
#define DRV_CAT2(a, b) a##b
#define DRV_CAT(a, b) DRV_CAT2(a, b)
#define DRV(name) DRV_CAT(DRV_PREFIX, name)
#define DRV_EXPORT extern "C" __attribute__((visibility("default")))

using namespace xsched::sched;
using namespace xsched::protocol;

namespace
{

struct PolicyBox
{
    std::unique_ptr<Policy> policy;
    std::map<XQueueHandle, int8_t> decision; // 1 suspend, 0 resume (last call wins)
    std::vector<int64_t> timers_us;
};

size_t CopyOut(const void *data, size_t size, void *out, size_t cap)
{
    if (out != nullptr && size <= cap) memcpy(out, data, size);
    return size;
}

int64_t ToMicros(std::chrono::system_clock::time_point tp)
{
    return std::chrono::duration_cast<std::chrono::microseconds>(tp.time_since_epoch()).count();
}

} // namespace

// ---- policies -------------------------------------------------------------------

DRV_EXPORT void *DRV(policy_create)(int type)
{
    auto *box = new PolicyBox();
    box->policy = CreatePolicy((XPolicyType)type);
    box->policy->SetSuspendFunc([box](XQueueHandle h) { box->decision[h] = 1; });
    box->policy->SetResumeFunc([box](XQueueHandle h) { box->decision[h] = 0; });
    box->policy->SetAddTimerFunc([box](TimePoint tp) { box->timers_us.push_back(ToMicros(tp)); });
    return box;
}

DRV_EXPORT void DRV(policy_destroy)(void *p) { delete (PolicyBox *)p; }

DRV_EXPORT void DRV(policy_hint_priority)(void *p, uint64_t xq, int prio)
{
    ((PolicyBox *)p)->policy->RecvHint(std::make_shared<PriorityHint>(xq, prio));
}

DRV_EXPORT void DRV(policy_hint_laxity)(void *p, uint64_t xq, int64_t lax, int lax_prio, int crit_prio)
{
    ((PolicyBox *)p)->policy->RecvHint(std::make_shared<LaxityHint>(xq, lax, lax_prio, crit_prio));
}

/// One scheduling round over `n` XQueues. decision[i]: 1 = suspend, 0 = resume,
/// -1 = the policy said nothing about queue i. Returns the number of timers requested
/// (their absolute times in microseconds go to timers_us, up to max_timers).
DRV_EXPORT int DRV(policy_sched)(void *p, int n, const uint64_t *handles, const uint64_t *devices,
                                 const uint8_t *ready, const int64_t *ready_time_us,
                                 int8_t *decision, int64_t *timers_us, int max_timers)
{
    auto *box = (PolicyBox *)p;
    Status status;
    for (int i = 0; i < n; ++i) {
        auto xq = std::make_unique<XQueueStatus>();
        xq->handle = handles[i];
        xq->device = devices[i];
        xq->level = kPreemptLevelBlock;
        xq->pid = 1;
        xq->threshold = 16;
        xq->batch_size = 8;
        xq->ready = ready[i] != 0;
        xq->suspended = false;
        xq->ready_time = std::chrono::system_clock::time_point(std::chrono::microseconds(ready_time_us[i]));
        status.xqueue_status[handles[i]] = std::move(xq);
    }
    box->decision.clear();
    box->timers_us.clear();
    box->policy->Sched(status);
    for (int i = 0; i < n; ++i) {
        auto it = box->decision.find(handles[i]);
        decision[i] = it == box->decision.end() ? (int8_t)-1 : it->second;
    }
    const int nt = (int)box->timers_us.size();
    for (int i = 0; i < nt && i < max_timers; ++i) timers_us[i] = box->timers_us[i];
    return nt;
}

/// Any hint, from its wire bytes.
DRV_EXPORT int DRV(policy_recv_hint)(void *p, const void *hint_bytes)
{
    auto hint = Hint::CopyConstructor(hint_bytes);
    if (hint == nullptr) return 0;
    ((PolicyBox *)p)->policy->RecvHint(hint);
    return 1;
}

/// policy_sched with processes: queue i belongs to pids[i] and is listed among that
/// process's suspended (suspended[i] != 0) or running XQueues.
DRV_EXPORT int DRV(policy_sched_processes)(void *p, int n, const uint64_t *handles, const uint64_t *devices,
                                           const uint8_t *ready, const int64_t *ready_time_us, const int *pids,
                                           const uint8_t *suspended, int8_t *decision, int64_t *timers_us,
                                           int max_timers)
{
    auto *box = (PolicyBox *)p;
    Status status;
    for (int i = 0; i < n; ++i) {
        auto xq = std::make_unique<XQueueStatus>();
        xq->handle = handles[i];
        xq->device = devices[i];
        xq->level = kPreemptLevelBlock;
        xq->pid = (PID)pids[i];
        xq->threshold = 16;
        xq->batch_size = 8;
        xq->ready = ready[i] != 0;
        xq->suspended = suspended[i] != 0;
        xq->ready_time = std::chrono::system_clock::time_point(std::chrono::microseconds(ready_time_us[i]));
        status.xqueue_status[handles[i]] = std::move(xq);
        auto &ps = status.process_status[(PID)pids[i]];
        if (ps == nullptr) {
            ps = std::make_unique<ProcessStatus>();
            ps->info.pid = (PID)pids[i];
        }
        (suspended[i] != 0 ? ps->suspended_xqueues : ps->running_xqueues).insert(handles[i]);
    }
    box->decision.clear();
    box->timers_us.clear();
    box->policy->Sched(status);
    for (int i = 0; i < n; ++i) {
        auto it = box->decision.find(handles[i]);
        decision[i] = it == box->decision.end() ? (int8_t)-1 : it->second;
    }
    const int nt = (int)box->timers_us.size();
    for (int i = 0; i < nt && i < max_timers; ++i) timers_us[i] = box->timers_us[i];
    return nt;
}

// ---- wire records ----------------------------------------------------------------

DRV_EXPORT size_t DRV(bytes_hint_priority)(uint64_t xq, int prio, void *out, size_t cap)
{ PriorityHint h(xq, prio); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_utilization)(int pid, uint64_t xq, int util, void *out, size_t cap)
{ UtilizationHint h(pid, xq, util); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_timeslice)(int64_t ts, void *out, size_t cap)
{ TimesliceHint h(ts); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_deadline)(uint64_t xq, int64_t ddl, void *out, size_t cap)
{ DeadlineHint h(xq, ddl); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_kdeadline)(uint64_t k, void *out, size_t cap)
{ KDeadlineHint h((size_t)k); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_laxity)(uint64_t xq, int64_t lax, int lp, int cp, void *out, size_t cap)
{ LaxityHint h(xq, lax, lp, cp); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_hint_window_active)(int pid, uint64_t display, void *out, size_t cap)
{ WindowActiveHint h((PID)pid, display); return CopyOut(h.Data(), h.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_hint_priority)(uint64_t xq, int prio, void *out, size_t cap)
{ HintEvent e(std::make_shared<PriorityHint>(xq, prio)); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_hint)(const void *hint_bytes, void *out, size_t cap)
{
    auto hint = Hint::CopyConstructor(hint_bytes);
    if (hint == nullptr) return 0;
    HintEvent e(hint);
    return CopyOut(e.Data(), e.Size(), out, cap);
}

DRV_EXPORT size_t DRV(bytes_event_process_create)(const char *cmdline, void *out, size_t cap)
{ ProcessCreateEvent e{std::string(cmdline)}; return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_process_destroy)(int pid, void *out, size_t cap)
{ ProcessDestroyEvent e((PID)pid); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_xqueue_create)(uint64_t xq, uint64_t dev, int level, int64_t thr,
                                                  int64_t batch, void *out, size_t cap)
{ XQueueCreateEvent e(xq, dev, (XPreemptLevel)level, thr, batch); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_xqueue_config)(uint64_t xq, uint64_t dev, int level, int64_t thr,
                                                  int64_t batch, void *out, size_t cap)
{ XQueueConfigUpdateEvent e(xq, dev, (XPreemptLevel)level, thr, batch); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_xqueue_destroy)(uint64_t xq, void *out, size_t cap)
{ XQueueDestroyEvent e(xq); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_xqueue_ready)(uint64_t xq, int64_t ready_us, void *out, size_t cap)
{
    XQueueReadyEvent e(xq, std::chrono::system_clock::time_point(std::chrono::microseconds(ready_us)));
    return CopyOut(e.Data(), e.Size(), out, cap);
}

DRV_EXPORT size_t DRV(bytes_event_xqueue_idle)(uint64_t xq, void *out, size_t cap)
{ XQueueIdleEvent e(xq); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_operation_complete)(uint64_t op_id, void *out, size_t cap)
{ OperationCompleteEvent e(op_id); return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_event_terminate)(void *out, size_t cap)
{ SchedulerTerminateEvent e; return CopyOut(e.Data(), e.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_operation_sched)(uint64_t id, int pid, const uint64_t *running, int n_running,
                                              const uint64_t *suspended, int n_suspended, void *out, size_t cap)
{
    ProcessStatus ps;
    ps.info.pid = (PID)pid;
    for (int i = 0; i < n_running; ++i) ps.running_xqueues.insert(running[i]);
    for (int i = 0; i < n_suspended; ++i) ps.suspended_xqueues.insert(suspended[i]);
    SchedOperation op(id, ps);
    return CopyOut(op.Data(), op.Size(), out, cap);
}

DRV_EXPORT size_t DRV(bytes_operation_config)(uint64_t id, int pid, uint64_t xq, int level, int64_t thr,
                                               int64_t batch, void *out, size_t cap)
{ ConfigOperation op(id, (PID)pid, xq, (XPreemptLevel)level, thr, batch); return CopyOut(op.Data(), op.Size(), out, cap); }

DRV_EXPORT size_t DRV(bytes_operation_terminate)(void *out, size_t cap)
{ TerminateOperation op; return CopyOut(op.Data(), op.Size(), out, cap); }

/// Round trip: rebuild an event from bytes with the class's own CopyConstructor and
/// serialise it again.
DRV_EXPORT size_t DRV(event_roundtrip)(const void *in, void *out, size_t cap)
{
    auto e = Event::CopyConstructor(in);
    return e ? CopyOut(e->Data(), e->Size(), out, cap) : 0;
}

DRV_EXPORT size_t DRV(operation_roundtrip)(const void *in, void *out, size_t cap)
{
    auto op = Operation::CopyConstructor(in);
    return op ? CopyOut(op->Data(), op->Size(), out, cap) : 0;
}

// ---- local scheduler ------------------------------------------------------------
// The whole LocalScheduler (event queue, worker thread, Status mirror, operation ids)
// driven through its public interface only. Events go in as wire bytes, so a test can
// set any process id; every operation the scheduler hands to its executor is kept as
// wire bytes, in order.

namespace
{

struct LocalBox
{
    std::unique_ptr<LocalScheduler> sched;
    std::mutex mtx;
    std::vector<std::vector<char>> ops;
};

} // namespace

DRV_EXPORT void *DRV(local_create)(int policy)
{
    auto *box = new LocalBox();
    box->sched = std::make_unique<LocalScheduler>((XPolicyType)policy);
    box->sched->SetExecutor([box](std::shared_ptr<const Operation> op) {
        const char *bytes = (const char *)op->Data();
        std::lock_guard<std::mutex> lock(box->mtx);
        box->ops.emplace_back(bytes, bytes + op->Size());
    });
    return box;
}

DRV_EXPORT void DRV(local_destroy)(void *b) { delete (LocalBox *)b; }
DRV_EXPORT void DRV(local_run)(void *b) { ((LocalBox *)b)->sched->Run(); }
DRV_EXPORT void DRV(local_stop)(void *b) { ((LocalBox *)b)->sched->Stop(); }
DRV_EXPORT void DRV(local_set_policy)(void *b, int policy) { ((LocalBox *)b)->sched->SetPolicy((XPolicyType)policy); }

DRV_EXPORT int DRV(local_recv_event)(void *b, const void *bytes)
{
    auto event = Event::CopyConstructor(bytes);
    if (event == nullptr) return 0;
    ((LocalBox *)b)->sched->RecvEvent(event);
    return 1;
}

/// Moves the recorded operations out as [uint64 size][bytes]... Returns the bytes
/// needed; nothing is consumed when `cap` is too small.
DRV_EXPORT size_t DRV(local_take_operations)(void *b, void *out, size_t cap)
{
    auto *box = (LocalBox *)b;
    std::lock_guard<std::mutex> lock(box->mtx);
    size_t need = 0;
    for (auto &op : box->ops) need += sizeof(uint64_t) + op.size();
    if (out == nullptr || need > cap) return need;
    char *dst = (char *)out;
    for (auto &op : box->ops) {
        const uint64_t size = op.size();
        memcpy(dst, &size, sizeof(size));
        memcpy(dst + sizeof(size), op.data(), op.size());
        dst += sizeof(size) + op.size();
    }
    box->ops.clear();
    return need;
}

// ---- names and devices ----------------------------------------------------------

DRV_EXPORT int DRV(policy_type_by_name)(const char *name) { return (int)GetPolicyType(name); }
DRV_EXPORT const char *DRV(policy_name)(int type) { return GetPolicyTypeName((XPolicyType)type).c_str(); }
DRV_EXPORT int DRV(scheduler_type_by_name)(const char *name) { return (int)GetSchedulerType(name); }
DRV_EXPORT const char *DRV(scheduler_name)(int type) { return GetSchedulerTypeName((XSchedulerType)type).c_str(); }
DRV_EXPORT const char *DRV(level_name)(int level) { return GetPreemptLevelName((XPreemptLevel)level).c_str(); }
DRV_EXPORT const char *DRV(platform_name)(int plat) { return GetPlatformName((XPlatform)plat).c_str(); }
DRV_EXPORT uint64_t DRV(make_device)(int type, uint32_t id) { return MakeDevice((XDeviceType)type, id); }
DRV_EXPORT int DRV(device_type)(uint64_t dev) { return (int)GetDeviceType(dev); }
DRV_EXPORT uint32_t DRV(device_id)(uint64_t dev) { return GetDeviceId(dev); }
