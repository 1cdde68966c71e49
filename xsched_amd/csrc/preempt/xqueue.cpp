// XQueue registry and the XQueue* C exports. reference preempt/src/xqueue/xqueue.cpp
#include <list>
#include <unordered_map>

#include "xsched/hint.h"
#include "xsched/xqueue.h"
#include "xsched/utils/env.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "ring_queue.h"
#include "xsched/preempt/xqueue/xqueue.h"

namespace xsched::preempt
{

namespace
{
std::mutex g_xq_mtx;
std::unordered_map<XQueueHandle, std::shared_ptr<XQueue>> g_xqs;
} // namespace

XResult XQueueManager::Add(XQueueHandle *xq_hp, HwQueueHandle hwq_h, int64_t level, int64_t flags)
{
    if (xq_hp == nullptr) return kXSchedErrorInvalidValue;
    if (level <= kPreemptLevelUnknown || level >= kPreemptLevelMax) return kXSchedErrorInvalidValue;
    // Only the asynchronous implementation exists.
    if (flags & kQueueCreateFlagBlockingSubmit) return kXSchedErrorNotSupported;

    auto hwq = HwQueueManager::Get(hwq_h);
    if (hwq == nullptr) {
        XWARN("HwQueue with handle 0x" FMT_64X " does not exist or is not registered", hwq_h);
        return kXSchedErrorNotFound;
    }

    // Creations take turns (two threads must not both build a queue for one hardware queue:
    // the loser's constructor and destructor would tell the scheduler about a handle that the
    // winner goes on using). A lock of its own, because the registry lock is not held while
    // the queue is built, see below.
    static std::mutex creation_mtx;
    std::lock_guard<std::mutex> one_at_a_time(creation_mtx);

    // One XQueue per hardware queue: hand out the one that is there.
    auto hand_out_existing = [&](const std::shared_ptr<XQueue> &existing) {
        XASSERT(g_xqs.count(existing->GetHandle()), "XQueue 0x" FMT_64X " is not registered",
                existing->GetHandle());
        XWARN("HwQueue 0x" FMT_64X " already has XQueue 0x" FMT_64X, hwq_h, existing->GetHandle());
        *xq_hp = existing->GetHandle();
        return kXSchedSuccess;
    };
    {
        std::lock_guard<std::mutex> lock(g_xq_mtx);
        if (auto existing = hwq->GetXQueue()) return hand_out_existing(existing);
    }
    // Built outside the registry lock: the constructor starts a thread and tells the scheduler,
    // and a scheduling round that runs on a submitter's thread looks queues up in this registry.
    auto xq = std::make_shared<RingXQueue>(hwq, (XPreemptLevel)level);
    std::lock_guard<std::mutex> lock(g_xq_mtx);
    hwq->SetXQueue(xq); // cycle, broken in Del()
    g_xqs[xq->GetHandle()] = xq;
    *xq_hp = xq->GetHandle();
    return kXSchedSuccess;
}

XResult XQueueManager::Del(XQueueHandle xq_h)
{
    std::shared_ptr<XQueue> xq;
    {
        std::lock_guard<std::mutex> lock(g_xq_mtx);
        auto it = g_xqs.find(xq_h);
        if (it == g_xqs.end()) {
            XWARN("XQueue with handle 0x" FMT_64X " does not exist", xq_h);
            return kXSchedErrorNotFound;
        }
        xq = std::move(it->second);
        if (auto hwq = xq->GetHwQueue()) hwq->SetXQueue(nullptr);
        g_xqs.erase(it);
    }
    // Outside the registry lock: let everything submitted finish so the launch
    // thread stops touching the hardware queue before the caller destroys it.
    xq->Resume(kQueueResumeFlagNone);
    xq->WaitAll();
    return kXSchedSuccess;
}

XResult XQueueManager::Exists(XQueueHandle xq_h)
{
    std::lock_guard<std::mutex> lock(g_xq_mtx);
    return g_xqs.count(xq_h) ? kXSchedSuccess : kXSchedErrorNotFound;
}

std::shared_ptr<XQueue> XQueueManager::Get(XQueueHandle xq_h)
{
    std::lock_guard<std::mutex> lock(g_xq_mtx);
    auto it = g_xqs.find(xq_h);
    return it == g_xqs.end() ? nullptr : it->second;
}

XResult XQueueManager::ForEachWaitAll()
{
    std::list<std::shared_ptr<XQueueWaitAllCommand>> drains;
    {
        std::lock_guard<std::mutex> lock(g_xq_mtx);
        for (auto &entry : g_xqs) {
            auto drain = entry.second->SubmitWaitAll();
            if (drain == nullptr) return kXSchedErrorUnknown;
            drains.push_back(std::move(drain));
        }
    }
    for (auto &drain : drains) drain->Wait();
    return kXSchedSuccess;
}

XResult XQueueManager::ForEach(std::function<XResult(std::shared_ptr<XQueue>)> func)
{
    std::lock_guard<std::mutex> lock(g_xq_mtx);
    for (auto &entry : g_xqs) {
        XResult res = func(entry.second);
        if (res != kXSchedSuccess) return res;
    }
    return kXSchedSuccess;
}

// Shim entry: build the hardware queue through `create_hwq`, attach an XQueue and
// apply every XSCHED_AUTO_XQUEUE_* setting present (xqueue.cpp:113-225). Failing
// to apply an optional setting only warns.
XResult XQueueManager::AutoCreate(std::function<XResult(HwQueueHandle *)> create_hwq)
{
    if (!GetEnvOption(XSCHED_AUTO_XQUEUE_ENV_NAME, false)) return kXSchedSuccess;

    HwQueueHandle hwq = 0;
    XResult res = create_hwq(&hwq);
    if (res != kXSchedSuccess) {
        XWARN("fail to auto-create HwQueue, err: %d", res);
        return res;
    }

    int64_t level = XSCHED_DEFAULT_PREEMPT_LEVEL;
    GetEnvInt64(XSCHED_AUTO_XQUEUE_LEVEL_ENV_NAME, level);

    XQueueHandle xq = 0;
    res = XQueueCreate(&xq, hwq, level, kQueueCreateFlagNone);
    if (res != kXSchedSuccess) {
        XWARN("fail to auto-create XQueue (level-" FMT_64D ") for HwQueue 0x" FMT_64X ", err: %d",
              level, hwq, res);
        return res;
    }

    auto warn_if = [&](XResult r, const char *what, int64_t v) {
        if (r != kXSchedSuccess) {
            XWARN("fail to auto-set %s " FMT_64D " for XQueue 0x" FMT_64X ", err: %d", what, v, xq, r);
        }
        return r;
    };

    int64_t threshold = -1, batch_size = -1;
    const bool has_threshold = GetEnvInt64(XSCHED_AUTO_XQUEUE_THRESHOLD_ENV_NAME, threshold);
    const bool has_batch = GetEnvInt64(XSCHED_AUTO_XQUEUE_BATCH_SIZE_ENV_NAME, batch_size);
    if (has_threshold || has_batch) {
        res = warn_if(XQueueSetLaunchConfig(xq, threshold, batch_size), "launch threshold", threshold);
    }

    int64_t v = 0;
    int64_t priority = PRIORITY_DEFAULT;
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_PRIORITY_ENV_NAME, priority)) {
        res = warn_if(XHintPriority(xq, (Priority)priority), "priority", priority);
    }
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_UTILIZATION_ENV_NAME, v)) {
        res = warn_if(XHintUtilization(xq, (Utilization)v), "utilization", v);
    }
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_TIMESLICE_ENV_NAME, v)) {
        res = warn_if(XHintTimeslice(v), "timeslice", v);
    }
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_DEADLINE_ENV_NAME, v)) {
        res = warn_if(XHintDeadline(xq, v), "deadline", v);
    }
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_KDEADLINE_ENV_NAME, v)) {
        res = warn_if(XHintKDeadline((size_t)v), "kdeadline", v);
    }
    if (GetEnvInt64(XSCHED_AUTO_XQUEUE_LAXITY_ENV_NAME, v)) {
        // Lax priority is the default one, critical priority the queue's own.
        res = warn_if(XHintLaxity(xq, v, PRIORITY_DEFAULT, (Priority)priority), "laxity", v);
    }
    return res;
}

XResult XQueueManager::AutoDestroy(HwQueueHandle hwq_h)
{
    if (!GetEnvOption(XSCHED_AUTO_XQUEUE_ENV_NAME, false)) return kXSchedSuccess;
    auto xq = HwQueueManager::GetXQueue(hwq_h);
    if (xq == nullptr) {
        XWARN("XQueue for HwQueue 0x" FMT_64X " does not exist", hwq_h);
        return kXSchedErrorNotFound;
    }
    XResult res = XQueueDestroy(xq->GetHandle());
    if (res != kXSchedSuccess) {
        XWARN("fail to auto-destroy XQueue 0x" FMT_64X ", err: %d", xq->GetHandle(), res);
        return res;
    }
    xq = nullptr;
    res = HwQueueDestroy(hwq_h);
    if (res != kXSchedSuccess) XWARN("fail to auto-destroy HwQueue 0x" FMT_64X ", err: %d", hwq_h, res);
    return res;
}

} // namespace xsched::preempt

using namespace xsched::preempt;

#define FIND_XQUEUE_OR_RETURN(var, handle) \
    std::shared_ptr<XQueue> var = XQueueManager::Get(handle); \
    if (var == nullptr) { \
        XWARN("XQueue with handle 0x" FMT_64X " does not exist", handle); \
        return kXSchedErrorNotFound; \
    }

EXPORT_C_FUNC XResult XQueueCreate(XQueueHandle *xq, HwQueueHandle hwq, int64_t level, int64_t flags)
{
    return XQueueManager::Add(xq, hwq, level, flags);
}

EXPORT_C_FUNC XResult XQueueDestroy(XQueueHandle xq) { return XQueueManager::Del(xq); }

EXPORT_C_FUNC XResult XQueueGet(XQueueHandle *xq, HwQueueHandle hwq)
{
    if (xq == nullptr) return kXSchedErrorInvalidValue;
    auto q = HwQueueManager::GetXQueue(hwq);
    if (q == nullptr) return kXSchedErrorNotFound;
    *xq = q->GetHandle();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueSetPreemptLevel(XQueueHandle xq, XPreemptLevel level)
{
    if (level <= kPreemptLevelUnknown || level >= kPreemptLevelMax) return kXSchedErrorInvalidValue;
    FIND_XQUEUE_OR_RETURN(q, xq);
    if (!q->GetFeatures(kQueueFeatureDynamicLevel)) {
        XWARN("XQueue with handle 0x" FMT_64X " does not support dynamic level", xq);
        return kXSchedErrorNotSupported;
    }
    q->SetPreemptLevel(level);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueSetLaunchConfig(XQueueHandle xq, int64_t threshold, int64_t batch_size)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    if (threshold <= 0 && batch_size <= 0) return kXSchedSuccess;
    if (threshold > 0 && !q->GetFeatures(kQueueFeatureDynamicThreshold)) return kXSchedErrorNotSupported;
    if (batch_size > 0 && !q->GetFeatures(kQueueFeatureDynamicBatchSize)) return kXSchedErrorNotSupported;
    q->SetLaunchConfig(threshold, batch_size);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueSubmit(XQueueHandle xq, HwCommandHandle hw_cmd)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    auto cmd = HwCommandManager::Del(hw_cmd); // ownership moves to the queue
    if (cmd == nullptr) {
        XWARN("HwCommand with handle 0x" FMT_64X " does not exist or is not registered", hw_cmd);
        return kXSchedErrorNotFound;
    }
    q->Submit(cmd);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueWait(XQueueHandle xq, HwCommandHandle hw_cmd)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    auto cmd = HwCommandManager::Get(hw_cmd);
    if (cmd == nullptr) {
        XWARN("HwCommand with handle 0x" FMT_64X " does not exist or is not registered", hw_cmd);
        return kXSchedErrorNotFound;
    }
    q->Wait(cmd);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueWaitAll(XQueueHandle xq)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    q->WaitAll();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueQuery(XQueueHandle xq, XQueueState *state)
{
    if (state == nullptr) return kXSchedErrorInvalidValue;
    FIND_XQUEUE_OR_RETURN(q, xq);
    *state = q->Query();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueSuspend(XQueueHandle xq, int64_t flags)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    q->Suspend(flags);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueResume(XQueueHandle xq, int64_t flags)
{
    FIND_XQUEUE_OR_RETURN(q, xq);
    q->Resume(flags);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueProfileHwCommandCount(XQueueHandle xq, int64_t *count)
{
    if (count == nullptr) return kXSchedErrorInvalidValue;
    FIND_XQUEUE_OR_RETURN(q, xq);
    *count = q->GetHwCommandCount();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult XQueueProfileDirectLaunchCount(XQueueHandle xq, int64_t *count)
{
    if (count == nullptr) return kXSchedErrorInvalidValue;
    FIND_XQUEUE_OR_RETURN(q, xq);
    auto *ring = dynamic_cast<RingXQueue *>(q.get());
    *count = ring != nullptr ? ring->GetDirectLaunchCount() : 0;
    return kXSchedSuccess;
}
