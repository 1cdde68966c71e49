// Scheduling hints: fixed-layout records that travel from XHint*() calls to the
// policy, possibly across a process boundary. Record layouts and type codes
// equal reference sched/include/xsched/sched/protocol/hint.h:16-262.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <memory>

#include "xsched/types.h"
#include "xsched/utils/common.h"

namespace xsched::sched
{

enum HintType
{
    kHintTypeUnknown      = 0,
    kHintTypePriority     = 1,
    kHintTypeUtilization  = 2,
    kHintTypeTimeslice    = 3,
    kHintTypeDeadline     = 4,
    kHintTypeKDeadline    = 5,
    kHintTypeLaxity       = 6,
    kHintTypeWindowActive = 7,
    kHintTypeMax,
};

struct HintMeta { HintType type; };

// ---- wire records (every record starts with HintMeta) -----------------------
struct PriorityHintData     { HintMeta meta; XQueueHandle handle; Priority prio; };
struct UtilizationHintData  { HintMeta meta; PID pid; XQueueHandle handle; Utilization util; };
struct TimesliceHintData    { HintMeta meta; Timeslice ts_us; };
struct DeadlineHintData     { HintMeta meta; XQueueHandle handle; Deadline ddl; };
struct KDeadlineHintData    { HintMeta meta; size_t k; };
struct LaxityHintData       { HintMeta meta; XQueueHandle handle; Laxity lax;
                              Priority lax_prio; Priority crit_prio; };
struct WindowActiveHintData { HintMeta meta; PID pid; uint64_t display; };

class Hint
{
public:
    Hint() = default;
    virtual ~Hint() = default;

    /// The record; begins with HintMeta.
    virtual const void *Data() const = 0;
    virtual size_t      Size() const = 0;
    virtual HintType    Type() const = 0;

    /// Rebuild a typed hint from received bytes (nullptr + fatal on unknown type).
    static std::shared_ptr<const Hint> CopyConstructor(const void *data);
};

/// Typed hint over one wire record. Padding bytes are zero so that the byte
/// image is deterministic.
template <typename Record, HintType kType>
class RecordHint : public Hint
{
public:
    explicit RecordHint(const void *data) { memcpy(&data_, data, sizeof(Record)); }
    virtual const void *Data() const override { return &data_; }
    virtual size_t      Size() const override { return sizeof(Record); }
    virtual HintType    Type() const override { return kType; }

protected:
    RecordHint() { memset(&data_, 0, sizeof(Record)); data_.meta.type = kType; }
    Record data_;
};

class PriorityHint : public RecordHint<PriorityHintData, kHintTypePriority>
{
public:
    using RecordHint::RecordHint;
    PriorityHint(XQueueHandle handle, Priority prio) { data_.handle = handle; data_.prio = prio; }
    XQueueHandle Handle() const { return data_.handle; }
    Priority     Prio()   const { return data_.prio; }
};

class UtilizationHint : public RecordHint<UtilizationHintData, kHintTypeUtilization>
{
public:
    using RecordHint::RecordHint;
    /// pid == 0 / handle == 0 mean "not addressed to a process / queue".
    UtilizationHint(PID pid, XQueueHandle handle, Utilization util)
    { data_.pid = pid; data_.handle = handle; data_.util = util; }
    PID          Pid()    const { return data_.pid; }
    XQueueHandle Handle() const { return data_.handle; }
    Utilization  Util()   const { return data_.util; }
};

class TimesliceHint : public RecordHint<TimesliceHintData, kHintTypeTimeslice>
{
public:
    using RecordHint::RecordHint;
    explicit TimesliceHint(Timeslice ts_us) { data_.ts_us = ts_us; }
    Timeslice Ts() const { return data_.ts_us; }
};

class DeadlineHint : public RecordHint<DeadlineHintData, kHintTypeDeadline>
{
public:
    using RecordHint::RecordHint;
    DeadlineHint(XQueueHandle handle, Deadline ddl) { data_.handle = handle; data_.ddl = ddl; }
    XQueueHandle Handle() const { return data_.handle; }
    Deadline     Ddl()    const { return data_.ddl; }
};

class KDeadlineHint : public RecordHint<KDeadlineHintData, kHintTypeKDeadline>
{
public:
    using RecordHint::RecordHint;
    explicit KDeadlineHint(size_t k) { data_.k = k; }
    size_t K() const { return data_.k; }
};

class LaxityHint : public RecordHint<LaxityHintData, kHintTypeLaxity>
{
public:
    using RecordHint::RecordHint;
    LaxityHint(XQueueHandle handle, Laxity lax, Priority lax_prio, Priority crit_prio)
    { data_.handle = handle; data_.lax = lax; data_.lax_prio = lax_prio; data_.crit_prio = crit_prio; }
    XQueueHandle Handle()   const { return data_.handle; }
    Laxity       Lax()      const { return data_.lax; }
    Priority     LaxPrio()  const { return data_.lax_prio; }
    Priority     CritPrio() const { return data_.crit_prio; }
};

class WindowActiveHint : public RecordHint<WindowActiveHintData, kHintTypeWindowActive>
{
public:
    using RecordHint::RecordHint;
    WindowActiveHint(PID pid, uint64_t display) { data_.pid = pid; data_.display = display; }
    PID      Pid()     const { return data_.pid; }
    uint64_t Display() const { return data_.display; }
};

} // namespace xsched::sched
