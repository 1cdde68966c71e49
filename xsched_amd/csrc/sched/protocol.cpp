// Construction and re-hydration of the wire records (events, operations, hints,
// status queries). reference sched/src/protocol/{event,operation,hint,status}.cpp
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "xsched/utils/xassert.h"
#include "xsched/sched/protocol/event.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/protocol/operation.h"
#include "xsched/sched/protocol/status.h"

namespace xsched::sched
{

// ---- hints -----------------------------------------------------------------

std::shared_ptr<const Hint> Hint::CopyConstructor(const void *data)
{
    switch (((const HintMeta *)data)->type) {
    case kHintTypePriority:     return std::make_shared<PriorityHint>(data);
    case kHintTypeUtilization:  return std::make_shared<UtilizationHint>(data);
    case kHintTypeTimeslice:    return std::make_shared<TimesliceHint>(data);
    case kHintTypeDeadline:     return std::make_shared<DeadlineHint>(data);
    case kHintTypeKDeadline:    return std::make_shared<KDeadlineHint>(data);
    case kHintTypeLaxity:       return std::make_shared<LaxityHint>(data);
    case kHintTypeWindowActive: return std::make_shared<WindowActiveHint>(data);
    default:
        XERRO("unknown hint type: %d", ((const HintMeta *)data)->type);
        return nullptr;
    }
}

// ---- events ----------------------------------------------------------------

std::shared_ptr<const Event> Event::CopyConstructor(const void *data)
{
    switch (((const EventMeta *)data)->type) {
    case kEventHint:               return std::make_shared<HintEvent>(data);
    case kEventSchedulerTerminate: return std::make_shared<SchedulerTerminateEvent>(data);
    case kEventProcessCreate:      return std::make_shared<ProcessCreateEvent>(data);
    case kEventProcessDestroy:     return std::make_shared<ProcessDestroyEvent>(data);
    case kEventXQueueCreate:       return std::make_shared<XQueueCreateEvent>(data);
    case kEventXQueueDestroy:      return std::make_shared<XQueueDestroyEvent>(data);
    case kEventXQueueReady:        return std::make_shared<XQueueReadyEvent>(data);
    case kEventXQueueIdle:         return std::make_shared<XQueueIdleEvent>(data);
    case kEventXQueueConfigUpdate: return std::make_shared<XQueueConfigUpdateEvent>(data);
    case kEventXQueueQuery:        return std::make_shared<XQueueQueryEvent>(data);
    case kEventXQueueQueryAll:     return std::make_shared<XQueueQueryAllEvent>(data);
    case kEventOperationComplete:  return std::make_shared<OperationCompleteEvent>(data);
    default:
        XERRO("unknown event type: %d", ((const EventMeta *)data)->type);
        return nullptr;
    }
}

static size_t HintRecordSize(HintType type)
{
    switch (type) {
    case kHintTypePriority:     return sizeof(PriorityHintData);
    case kHintTypeUtilization:  return sizeof(UtilizationHintData);
    case kHintTypeTimeslice:    return sizeof(TimesliceHintData);
    case kHintTypeDeadline:     return sizeof(DeadlineHintData);
    case kHintTypeKDeadline:    return sizeof(KDeadlineHintData);
    case kHintTypeLaxity:       return sizeof(LaxityHintData);
    case kHintTypeWindowActive: return sizeof(WindowActiveHintData);
    default:                    return 0;
    }
}

bool Event::WireRecordOk(const void *data, size_t received)
{
    if (data == nullptr || received < sizeof(EventMeta)) return false;
    EventMeta meta;
    memcpy(&meta, data, sizeof(meta));
    switch (meta.type) {
    case kEventHint:
    {
        const size_t head = offsetof(HintEventData, hint_data);
        if (received < head + sizeof(HintMeta)) return false;
        HintEventData fixed;
        memcpy(&fixed, data, head);
        HintMeta hint;
        memcpy(&hint, (const char *)data + head, sizeof(hint));
        const size_t need = HintRecordSize(hint.type);
        return need != 0 && fixed.size <= received && fixed.size >= head + need;
    }
    case kEventSchedulerTerminate:
    case kEventProcessDestroy:     return received >= sizeof(MetaOnlyEventData);
    case kEventProcessCreate:      return received >= sizeof(ProcessCreateData);
    case kEventXQueueCreate:
    case kEventXQueueConfigUpdate: return received >= sizeof(XQueueConfigData);
    case kEventXQueueDestroy:
    case kEventXQueueIdle:         return received >= sizeof(XQueueHandleData);
    case kEventXQueueReady:        return received >= sizeof(XQueueReadyData);
    case kEventOperationComplete:  return received >= sizeof(OperationCompleteData);
    default:                       return false; // unknown, or a query (pointers inside)
    }
}

HintEvent::HintEvent(const void *data)
{
    const size_t size = ((const HintEventData *)data)->size;
    data_ = (HintEventData *)malloc(size);
    memcpy(data_, data, size);
}

HintEvent::HintEvent(std::shared_ptr<const Hint> hint)
{
    const size_t size = offsetof(HintEventData, hint_data) + hint->Size();
    data_ = (HintEventData *)calloc(1, size);
    data_->meta.type = kEventHint;
    data_->meta.pid = GetProcessId();
    data_->size = size;
    memcpy(data_->hint_data, hint->Data(), hint->Size());
}

HintEvent::~HintEvent() { free(data_); }

StatusQuery *XQueueQueryEvent::QueryData() const
{
    XASSERT(data_.query_data != nullptr, "query data should not be nullptr");
    XASSERT(data_.meta.pid == GetProcessId(), "a status query is only valid inside its process");
    return data_.query_data;
}

StatusQuery *XQueueQueryAllEvent::QueryData() const
{
    XASSERT(data_.query_data != nullptr, "query data should not be nullptr");
    XASSERT(data_.meta.pid == GetProcessId(), "a status query is only valid inside its process");
    return data_.query_data;
}

// ---- operations ------------------------------------------------------------

std::shared_ptr<const Operation> Operation::CopyConstructor(const void *data)
{
    switch (((const OperationMeta *)data)->type) {
    case kOperationTerminate: return std::make_shared<TerminateOperation>(data);
    case kOperationSched:     return std::make_shared<SchedOperation>(data);
    case kOperationConfig:    return std::make_shared<ConfigOperation>(data);
    default:
        XERRO("unsupported operation type: %d", ((const OperationMeta *)data)->type);
        return nullptr;
    }
}

bool Operation::WireRecordOk(const void *data, size_t received)
{
    if (data == nullptr || received < sizeof(OperationMeta)) return false;
    OperationMeta meta;
    memcpy(&meta, data, sizeof(meta));
    switch (meta.type) {
    case kOperationTerminate: return true;
    case kOperationConfig:    return received >= sizeof(ConfigOperationData);
    case kOperationSched:
    {
        const size_t head = offsetof(SchedOperationData, handles);
        if (received < head) return false;
        SchedOperationData fixed;
        memcpy(&fixed, data, head);
        const size_t room = (received - head) / sizeof(XQueueHandle);
        if (fixed.running_cnt > room || fixed.suspended_cnt > room - fixed.running_cnt) return false;
        return fixed.size <= received
            && fixed.size >= head + (fixed.running_cnt + fixed.suspended_cnt) * sizeof(XQueueHandle);
    }
    default: return false;
    }
}

TerminateOperation::TerminateOperation()
{
    memset(&meta_, 0, sizeof(meta_));
    meta_.type = kOperationTerminate;
    meta_.pid = GetProcessId();
}

TerminateOperation::TerminateOperation(const void *data) { memcpy(&meta_, data, sizeof(meta_)); }

SchedOperationData *SchedOperation::Alloc(OperationId id, PID pid, size_t running, size_t suspended)
{
    const size_t size = offsetof(SchedOperationData, handles)
                      + (running + suspended) * sizeof(XQueueHandle);
    auto *d = (SchedOperationData *)calloc(1, std::max(size, sizeof(SchedOperationData)));
    d->meta.id = id;
    d->meta.type = kOperationSched;
    d->meta.pid = pid;
    d->size = size;
    d->running_cnt = running;
    d->suspended_cnt = suspended;
    return d;
}

SchedOperation::SchedOperation(const void *data)
{
    const size_t size = ((const SchedOperationData *)data)->size;
    data_ = (SchedOperationData *)malloc(std::max(size, sizeof(SchedOperationData)));
    memcpy(data_, data, size);
}

SchedOperation::SchedOperation(OperationId id, const ProcessStatus &status)
{
    data_ = Alloc(id, status.info.pid, status.running_xqueues.size(),
                  status.suspended_xqueues.size());
    size_t n = 0;
    for (XQueueHandle h : status.running_xqueues)   data_->handles[n++] = h;
    for (XQueueHandle h : status.suspended_xqueues) data_->handles[n++] = h;
}

SchedOperation::SchedOperation(OperationId id, PID pid, SchedType type,
                               const std::vector<XQueueHandle> &xqs)
{
    const size_t n = xqs.size();
    data_ = Alloc(id, pid, type == kSchedTypeResumeAll ? n : 0, type == kSchedTypeSuspendAll ? n : 0);
    if (n) memcpy(data_->handles, xqs.data(), n * sizeof(XQueueHandle));
}

SchedOperation::~SchedOperation() { free(data_); }

ConfigOperation::ConfigOperation(const void *data) { memcpy(&data_, data, sizeof(data_)); }

ConfigOperation::ConfigOperation(OperationId id, PID pid, XQueueHandle handle,
                                 XPreemptLevel level, int64_t threshold, int64_t batch_size)
{
    memset(&data_, 0, sizeof(data_));
    data_.meta.id = id;
    data_.meta.type = kOperationConfig;
    data_.meta.pid = pid;
    data_.handle = handle;
    data_.level = level;
    data_.threshold = threshold;
    data_.batch_size = batch_size;
}

// ---- status query ----------------------------------------------------------

void StatusQuery::Wait()
{
    std::unique_lock<std::mutex> lock(mtx_);
    cv_.wait(lock, [this]() { return ready_; });
}

void StatusQuery::Notify()
{
    { std::lock_guard<std::mutex> lock(mtx_); ready_ = true; }
    cv_.notify_all();
}

void StatusQuery::Reset()
{
    ready_ = false;
    status_.clear();
    if (kQueryProcess) processes_.clear();
}

} // namespace xsched::sched
