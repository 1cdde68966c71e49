// ORACLE - test infrastructure only. A recording hardware queue: an HwQueue whose
// "device" is a watermark the test advances by hand, and which writes down every call
// the XQueue core makes on it. It is compiled twice: against this repository's headers
// (libxqueue_probe.so, driving the shipped libpreempt.so) and against the reference's
// headers together with the reference's own XQueue sources (_ref/libxqueue_ref.so). Tests
// drive both through the public C API and compare the recorded traces with each other and
// with the launch-loop model in oracle/xqueue_model.py (same token vocabulary).
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "xsched/xqueue.h"
#include "xsched/utils/common.h"
#include "xsched/protocol/device.h"
#include "xsched/preempt/hal/hw_command.h"
#include "xsched/preempt/hal/hw_queue.h"

using namespace xsched::preempt;

namespace
{

class RecQueue;

class RecCommand : public HwCommand
{
public:
    RecCommand(XCommandProperties props, bool gate): HwCommand(props), gate_(gate) {}
    virtual void Synchronize() override;
    virtual bool Synchronizable() override { return marker_; }
    virtual bool EnableSynchronization() override { marker_ = true; return true; }
    virtual void BeforeLaunch() override;

    RecQueue *queue = nullptr;
private:
    const bool gate_;
    bool marker_ = false;
};

class RecQueue : public HwQueue
{
public:
    RecQueue(uint64_t handle, int max_level): handle_(handle), max_level_(max_level) {}

    virtual void Launch(std::shared_ptr<HwCommand> cmd) override
    {
        std::lock_guard<std::mutex> lock(mtx);
        last_launched = cmd->GetIdx();
        Add("L" + std::to_string(cmd->GetIdx()) + (cmd->Synchronizable() ? "*" : ""));
    }

    virtual void Synchronize() override
    {
        std::unique_lock<std::mutex> lock(mtx);
        Add("QS");
        const int64_t upto = last_launched;
        const uint64_t flush = flushes;
        cv.wait(lock, [&]() { return done >= upto || flushes != flush; });
    }

    virtual void Deactivate() override
    {
        { std::lock_guard<std::mutex> lock(mtx); Add("D"); flushes++; }
        cv.notify_all();
        if (on_deactivate) on_deactivate(on_deactivate_arg);   // on whichever thread runs the scheduling operation
    }

    virtual void Reactivate(const CommandLog &log) override
    {
        std::lock_guard<std::mutex> lock(mtx);
        std::string s = "R[";
        bool first = true;
        for (auto &c : log) { s += (first ? "" : ",") + std::to_string(c->GetIdx()); first = false; }
        Add(s + "]");
    }

    virtual XDevice GetDevice() override { return xsched::protocol::MakeDevice(kDeviceTypeCPU, 99); }
    virtual HwQueueHandle GetHandle() override { return handle_; }
    virtual bool SupportDynamicLevel() override { return true; }
    virtual XPreemptLevel GetMaxSupportedLevel() override { return (XPreemptLevel)max_level_; }
    virtual void OnHwCommandSubmit(std::shared_ptr<HwCommand> cmd) override
    {
        if (auto *rc = dynamic_cast<RecCommand *>(cmd.get())) rc->queue = this;
    }

    void Add(const std::string &tok) { trace.push_back(tok); }

    std::mutex mtx;
    std::condition_variable cv;
    std::vector<std::string> trace;
    int64_t done = 0;          // device watermark
    int64_t last_launched = 0;
    uint64_t flushes = 0;
    bool gate_open = false;
    void (*on_deactivate)(void *) = nullptr;
    void *on_deactivate_arg = nullptr;

private:
    const uint64_t handle_;
    const int max_level_;
};

void RecCommand::Synchronize()
{
    std::unique_lock<std::mutex> lock(queue->mtx);
    queue->Add("CS" + std::to_string(GetIdx()));
    const int64_t idx = GetIdx();
    const uint64_t flush = queue->flushes;
    queue->cv.wait(lock, [&]() { return queue->done >= idx || queue->flushes != flush; });
}

// A gate command holds the launch thread (outside its lock) until the test opens the
// gate, so that a whole burst can be submitted before the thread looks at it.
void RecCommand::BeforeLaunch()
{
    if (!gate_) return;
    std::unique_lock<std::mutex> lock(queue->mtx);
    queue->cv.wait(lock, [&]() { return queue->gate_open; });
}

std::shared_ptr<RecQueue> Find(HwQueueHandle h)
{
    return std::dynamic_pointer_cast<RecQueue>(HwQueueManager::Get(h));
}

} // namespace

extern "C" {

EXPORT_C_FUNC XResult RecQueueCreate(HwQueueHandle *hwq, int max_level)
{
    static uint64_t next = 0x5245430000000001ull; // "REC" | serial
    const uint64_t h = next++;
    XResult res = HwQueueManager::Add(h, [&]() { return std::make_shared<RecQueue>(h, max_level); });
    if (res == kXSchedSuccess) *hwq = h;
    return res;
}

EXPORT_C_FUNC XResult RecCommandCreate(HwCommandHandle *cmd, int64_t props, int gate)
{
    *cmd = HwCommandManager::Add(std::make_shared<RecCommand>(props, gate != 0));
    return kXSchedSuccess;
}

/// The device has finished everything launched up to and including idx.
EXPORT_C_FUNC XResult RecQueueComplete(HwQueueHandle hwq, int64_t idx)
{
    auto q = Find(hwq);
    if (!q) return kXSchedErrorNotFound;
    { std::lock_guard<std::mutex> lock(q->mtx); if (idx > q->done) q->done = idx; }
    q->cv.notify_all();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult RecQueueSetGate(HwQueueHandle hwq, int open)
{
    auto q = Find(hwq);
    if (!q) return kXSchedErrorNotFound;
    { std::lock_guard<std::mutex> lock(q->mtx); q->gate_open = open != 0; }
    q->cv.notify_all();
    return kXSchedSuccess;
}

/// `fn(arg)` is called at the end of every Deactivate() of this queue, on the thread that
/// executes the suspension (a test looks from there at what that thread holds).
EXPORT_C_FUNC XResult RecQueueOnDeactivate(HwQueueHandle hwq, void (*fn)(void *), void *arg)
{
    auto q = Find(hwq);
    if (!q) return kXSchedErrorNotFound;
    std::lock_guard<std::mutex> lock(q->mtx);
    q->on_deactivate = fn;
    q->on_deactivate_arg = arg;
    return kXSchedSuccess;
}

/// Space-separated trace so far; returns its length (truncated to cap - 1).
EXPORT_C_FUNC size_t RecQueueTrace(HwQueueHandle hwq, char *out, size_t cap)
{
    auto q = Find(hwq);
    if (!q || cap == 0) return 0;
    std::ostringstream os;
    {
        std::lock_guard<std::mutex> lock(q->mtx);
        for (size_t i = 0; i < q->trace.size(); ++i) os << (i ? " " : "") << q->trace[i];
    }
    const std::string s = os.str();
    const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
    memcpy(out, s.data(), n);
    out[n] = 0;
    return n;
}

} // extern "C"
