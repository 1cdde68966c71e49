// Events: what XQueues, processes and the executor report to a scheduler.
// Record layouts and type codes equal reference
// sched/include/xsched/sched/protocol/event.h:18-433, so the byte stream is
// the same on a daemon channel.
#pragma once

#include <chrono>
#include <cstddef>
#include <cstring>
#include <memory>
#include <string>

#include "xsched/types.h"
#include "xsched/utils/common.h"
#include "xsched/sched/protocol/hint.h"
#include "xsched/sched/protocol/operation.h"
#include "xsched/sched/protocol/status.h"

namespace xsched::sched
{

enum EventType
{
    kEventHint               = 0,
    kEventSchedulerTerminate = 1,
    kEventProcessCreate      = 2,
    kEventProcessDestroy     = 3,
    kEventXQueueCreate       = 4,
    kEventXQueueDestroy      = 5,
    kEventXQueueReady        = 6,
    kEventXQueueIdle         = 7,
    kEventXQueueConfigUpdate = 8,
    kEventXQueueQuery        = 9,
    kEventXQueueQueryAll     = 10,
    kEventOperationComplete  = 11,
};

struct EventMeta { EventType type; PID pid; };

// ---- wire records (every record starts with EventMeta) ---------------------
struct MetaOnlyEventData     { EventMeta meta; };
/// Variable length: `size` bytes in total, the hint record starts at hint_data.
struct HintEventData         { EventMeta meta; size_t size; char hint_data[1]; };
struct ProcessCreateData     { EventMeta meta; char cmdline[256]; };
struct XQueueConfigData      { EventMeta meta; XQueueHandle handle; XDevice device;
                               XPreemptLevel level; int64_t threshold; int64_t batch_size; };
struct XQueueHandleData      { EventMeta meta; XQueueHandle handle; };
struct XQueueReadyData       { EventMeta meta; XQueueHandle handle; int64_t ready_time_us; };
struct XQueueQueryData       { EventMeta meta; XQueueHandle handle; StatusQuery *query_data; };
struct XQueueQueryAllData    { EventMeta meta; StatusQuery *query_data; };
struct OperationCompleteData { EventMeta meta; OperationId op_id; };

class Event
{
public:
    Event() = default;
    virtual ~Event() = default;

    /// The record; begins with EventMeta.
    virtual const void *Data() const = 0;
    virtual size_t      Size() const = 0;
    virtual EventType   Type() const = 0;
    /// The process that produced the event.
    virtual PID         Pid()  const = 0;

    static std::shared_ptr<const Event> CopyConstructor(const void *data);
    /// Whether `received` bytes that arrived from another process hold one complete event
    /// record of a known type whose embedded sizes stay inside those bytes. Records that
    /// carry pointers (status queries) are only valid inside their own process: false.
    static bool WireRecordOk(const void *data, size_t received);
};

/// Typed event over one fixed-size wire record; padding is zeroed.
template <typename Record, EventType kType>
class RecordEvent : public Event
{
public:
    explicit RecordEvent(const void *data) { memcpy(&data_, data, sizeof(Record)); }
    virtual const void *Data() const override { return &data_; }
    virtual size_t      Size() const override { return sizeof(Record); }
    virtual EventType   Type() const override { return kType; }
    virtual PID         Pid()  const override { return data_.meta.pid; }

protected:
    RecordEvent()
    {
        memset(&data_, 0, sizeof(Record));
        data_.meta.type = kType;
        data_.meta.pid = GetProcessId();
    }
    Record data_;
};

class HintEvent : public Event
{
public:
    explicit HintEvent(const void *data);
    explicit HintEvent(std::shared_ptr<const Hint> hint);
    virtual ~HintEvent();

    virtual const void *Data() const override { return data_; }
    virtual size_t      Size() const override { return data_->size; }
    virtual EventType   Type() const override { return kEventHint; }
    virtual PID         Pid()  const override { return data_->meta.pid; }
    std::shared_ptr<const Hint> GetHint() const { return Hint::CopyConstructor(data_->hint_data); }

private:
    HintEventData *data_ = nullptr;
};

/// Stops a scheduler's worker thread.
class SchedulerTerminateEvent : public RecordEvent<MetaOnlyEventData, kEventSchedulerTerminate>
{
public:
    using RecordEvent::RecordEvent;
    SchedulerTerminateEvent() = default;
};

class ProcessCreateEvent : public RecordEvent<ProcessCreateData, kEventProcessCreate>
{
public:
    using RecordEvent::RecordEvent;
    explicit ProcessCreateEvent(const std::string &cmdline)
    {
        strncpy(data_.cmdline, cmdline.c_str(), sizeof(data_.cmdline) - 1);
    }
    const char *Cmdline() const { return data_.cmdline; }
    static size_t CmdlineCapacity() { return sizeof(ProcessCreateData::cmdline); }
};

class ProcessDestroyEvent : public RecordEvent<MetaOnlyEventData, kEventProcessDestroy>
{
public:
    using RecordEvent::RecordEvent;
    ProcessDestroyEvent() = default;
    explicit ProcessDestroyEvent(PID pid) { data_.meta.pid = pid; }
};

template <EventType kType>
class XQueueConfigEventBase : public RecordEvent<XQueueConfigData, kType>
{
public:
    using RecordEvent<XQueueConfigData, kType>::RecordEvent;
    XQueueConfigEventBase(XQueueHandle handle, XDevice device, XPreemptLevel level,
                          int64_t threshold, int64_t batch_size)
    {
        this->data_.handle = handle;
        this->data_.device = device;
        this->data_.level = level;
        this->data_.threshold = threshold;
        this->data_.batch_size = batch_size;
    }
    XQueueHandle  Handle()    const { return this->data_.handle; }
    XDevice       Device()    const { return this->data_.device; }
    XPreemptLevel Level()     const { return this->data_.level; }
    int64_t       Threshold() const { return this->data_.threshold; }
    int64_t       BatchSize() const { return this->data_.batch_size; }
};
using XQueueCreateEvent       = XQueueConfigEventBase<kEventXQueueCreate>;
using XQueueConfigUpdateEvent = XQueueConfigEventBase<kEventXQueueConfigUpdate>;

template <EventType kType>
class XQueueHandleEventBase : public RecordEvent<XQueueHandleData, kType>
{
public:
    using RecordEvent<XQueueHandleData, kType>::RecordEvent;
    explicit XQueueHandleEventBase(XQueueHandle handle) { this->data_.handle = handle; }
    XQueueHandle Handle() const { return this->data_.handle; }
};
using XQueueDestroyEvent = XQueueHandleEventBase<kEventXQueueDestroy>;
using XQueueIdleEvent    = XQueueHandleEventBase<kEventXQueueIdle>;

class XQueueReadyEvent : public RecordEvent<XQueueReadyData, kEventXQueueReady>
{
public:
    using RecordEvent::RecordEvent;
    XQueueReadyEvent(XQueueHandle handle, std::chrono::system_clock::time_point ready_time)
    {
        data_.handle = handle;
        data_.ready_time_us = std::chrono::duration_cast<std::chrono::microseconds>(
            ready_time.time_since_epoch()).count();
    }
    XQueueHandle Handle() const { return data_.handle; }
    std::chrono::system_clock::time_point ReadyTime() const
    {
        return std::chrono::system_clock::time_point(std::chrono::microseconds(data_.ready_time_us));
    }
};

/// In-process only: carries a pointer to the asker's StatusQuery.
class XQueueQueryEvent : public RecordEvent<XQueueQueryData, kEventXQueueQuery>
{
public:
    using RecordEvent::RecordEvent;
    XQueueQueryEvent(XQueueHandle handle, StatusQuery *query)
    { data_.handle = handle; data_.query_data = query; }
    XQueueHandle Handle() const { return data_.handle; }
    StatusQuery *QueryData() const;
};

/// In-process only.
class XQueueQueryAllEvent : public RecordEvent<XQueueQueryAllData, kEventXQueueQueryAll>
{
public:
    using RecordEvent::RecordEvent;
    explicit XQueueQueryAllEvent(StatusQuery *query) { data_.query_data = query; }
    StatusQuery *QueryData() const;
};

/// Sent by the executor once an operation has been applied to the XQueues.
class OperationCompleteEvent : public RecordEvent<OperationCompleteData, kEventOperationComplete>
{
public:
    using RecordEvent::RecordEvent;
    explicit OperationCompleteEvent(OperationId op_id) { data_.op_id = op_id; }
    OperationId OpId() const { return data_.op_id; }
};

} // namespace xsched::sched
