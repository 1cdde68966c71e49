// Operations: what a scheduler tells a process to do with its XQueues. Record
// layouts and type codes equal reference
// sched/include/xsched/sched/protocol/operation.h:13-140.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <vector>

#include "xsched/types.h"
#include "xsched/sched/protocol/status.h"

namespace xsched::sched
{

typedef uint64_t OperationId;

enum OperationType
{
    kOperationNone      = 0,
    kOperationTerminate = 1,
    kOperationSched     = 2,
    kOperationConfig    = 4,
};

struct OperationMeta { OperationId id; OperationType type; PID pid; };

// ---- wire records ----------------------------------------------------------
/// Variable length: `size` bytes in total, `running_cnt` handles to resume
/// followed by `suspended_cnt` handles to suspend.
struct SchedOperationData
{
    OperationMeta meta;
    size_t        size;
    size_t        running_cnt;
    size_t        suspended_cnt;
    XQueueHandle  handles[1];
};

struct ConfigOperationData
{
    OperationMeta meta;
    XQueueHandle  handle;
    XPreemptLevel level;      // kPreemptLevelUnknown: keep
    int64_t       threshold;  // <= 0: keep
    int64_t       batch_size; // <= 0: keep
};

class Operation
{
public:
    Operation() = default;
    virtual ~Operation() = default;

    /// The record; begins with OperationMeta.
    virtual const void *  Data() const = 0;
    virtual size_t        Size() const = 0;
    virtual OperationId   Id()   const = 0;
    virtual OperationType Type() const = 0;
    /// The process that has to execute it.
    virtual PID           Pid()  const = 0;

    static std::shared_ptr<const Operation> CopyConstructor(const void *data);
    /// Whether `received` bytes from another process hold one complete operation record of a
    /// known type whose handle counts stay inside those bytes.
    static bool WireRecordOk(const void *data, size_t received);
};

/// Ends the receiving thread of a global-scheduler client.
class TerminateOperation : public Operation
{
public:
    TerminateOperation();
    explicit TerminateOperation(const void *data);
    virtual const void *  Data() const override { return &meta_; }
    virtual size_t        Size() const override { return sizeof(meta_); }
    virtual OperationId   Id()   const override { return meta_.id; }
    virtual OperationType Type() const override { return kOperationTerminate; }
    virtual PID           Pid()  const override { return meta_.pid; }
private:
    OperationMeta meta_;
};

class SchedOperation : public Operation
{
public:
    enum SchedType { kSchedTypeResumeAll = 0, kSchedTypeSuspendAll = 1 };

    explicit SchedOperation(const void *data);
    /// Running set first, then suspended set, both in ascending handle order.
    SchedOperation(OperationId id, const ProcessStatus &status);
    SchedOperation(OperationId id, PID pid, SchedType type, const std::vector<XQueueHandle> &xqs);
    virtual ~SchedOperation();

    virtual const void *  Data() const override { return data_; }
    virtual size_t        Size() const override { return data_->size; }
    virtual OperationId   Id()   const override { return data_->meta.id; }
    virtual OperationType Type() const override { return kOperationSched; }
    virtual PID           Pid()  const override { return data_->meta.pid; }

    size_t RunningCnt()   const { return data_->running_cnt; }
    size_t SuspendedCnt() const { return data_->suspended_cnt; }
    const XQueueHandle *Handles() const { return data_->handles; }

private:
    static SchedOperationData *Alloc(OperationId id, PID pid, size_t running, size_t suspended);
    SchedOperationData *data_ = nullptr;
};

class ConfigOperation : public Operation
{
public:
    explicit ConfigOperation(const void *data);
    ConfigOperation(OperationId id, PID pid, XQueueHandle handle,
                    XPreemptLevel level, int64_t threshold, int64_t batch_size);

    virtual const void *  Data() const override { return &data_; }
    virtual size_t        Size() const override { return sizeof(data_); }
    virtual OperationId   Id()   const override { return data_.meta.id; }
    virtual OperationType Type() const override { return kOperationConfig; }
    virtual PID           Pid()  const override { return data_.meta.pid; }

    XQueueHandle  Handle()    const { return data_.handle; }
    XPreemptLevel Level()     const { return data_.level; }
    int64_t       Threshold() const { return data_.threshold; }
    int64_t       BatchSize() const { return data_.batch_size; }

private:
    ConfigOperationData data_;
};

} // namespace xsched::sched
