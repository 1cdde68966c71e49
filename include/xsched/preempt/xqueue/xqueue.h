// XQueue: abstract preemptible queue plus its process-wide registry.
// Interface follows reference preempt/include/xsched/preempt/xqueue/xqueue.h:12-83.
#pragma once

#include <functional>
#include <memory>

#include "xsched/types.h"
#include "xsched/preempt/hal/hw_command.h"
#include "xsched/preempt/hal/hw_queue.h"

namespace xsched::preempt
{

enum XQueueImplType
{
    kXQueueImplTypeAsync    = 0,
    kXQueueImplTypeBlocking = 1,
};

typedef int64_t XQueueFeatures;

class XQueue : public std::enable_shared_from_this<XQueue>
{
public:
    XQueue(XQueueImplType impl_type, XQueueFeatures features, std::shared_ptr<HwQueue> hwq)
        : kImplType(impl_type), kFeatures(features), kDevice(hwq->GetDevice())
        , kHandle((uint64_t)this ^ ((uint64_t)GetProcessId() << 48)), kHwQueue(hwq) {}
    virtual ~XQueue() = default;

    virtual void Submit(std::shared_ptr<HwCommand> hw_cmd) = 0;
    virtual std::shared_ptr<XQueueWaitAllCommand> SubmitWaitAll() = 0;
    virtual void WaitAll() = 0;
    virtual void Wait(std::shared_ptr<HwCommand> hw_cmd) = 0;
    virtual XQueueState Query() = 0;
    virtual int64_t GetHwCommandCount() = 0;

    virtual void Suspend(int64_t flags) = 0;
    virtual void Resume(int64_t flags) = 0;

    /// Not thread-safe against Submit()/Wait() on the same queue.
    virtual void SetPreemptLevel(XPreemptLevel level) = 0;
    /// A value <= 0 keeps the current setting.
    virtual void SetLaunchConfig(int64_t threshold, int64_t batch_size) = 0;

    XQueueImplType           GetImplType() const { return kImplType; }
    XDevice                  GetDevice()   const { return kDevice;   }
    XQueueHandle             GetHandle()   const { return kHandle;   }
    std::shared_ptr<HwQueue> GetHwQueue()  const { return kHwQueue;  }
    XQueueFeatures GetFeatures(XQueueFeatures mask = kQueueFeatureMaskAll) const
    { return kFeatures & mask; }

protected:
    const XQueueImplType           kImplType;
    const XQueueFeatures           kFeatures;
    const XDevice                  kDevice;
    const XQueueHandle             kHandle;
    const std::shared_ptr<HwQueue> kHwQueue;
};

class XQueueManager
{
public:
    STATIC_CLASS(XQueueManager);

    static XResult Add(XQueueHandle *xq_hp, HwQueueHandle hwq_h, int64_t level, int64_t flags);
    static XResult Del(XQueueHandle xq_h);
    static XResult Exists(XQueueHandle xq_h);
    static std::shared_ptr<XQueue> Get(XQueueHandle xq_h);

    /// Enqueue a drain marker on every queue, then wait for all of them.
    static XResult ForEachWaitAll();
    static XResult ForEach(std::function<XResult(std::shared_ptr<XQueue>)> func);
    /// Shim helpers: create / destroy an XQueue configured from XSCHED_AUTO_XQUEUE*.
    static XResult AutoCreate(std::function<XResult(HwQueueHandle *)> create_hwq);
    static XResult AutoDestroy(HwQueueHandle hwq_h);
};

} // namespace xsched::preempt
