// ORACLE - test infrastructure only: the CPU baseline. A compact C++ restatement of
// XSched's host-side scheduling loop, driving CPU versions of the synthetic kernels
// (oracle/kernels.c) through a CPU hardware queue. It is what bench.py times as
// `cpu_baseline` (kind "port"); nothing shipped links it.
//
// Structure follows the reference, one class per reference class, with the reference's
// own data structures (std::list, mutex + condition variable per command):
//   Command        preempt/src/xqueue/xcommand.cpp:7-33       state + wait
//   Buffer         preempt/src/xqueue/command_buffer.cpp:39-155 FIFO, Idle/Ready, synthetic
//                                                              batch-sync and drain marker
//   Worker         preempt/src/xqueue/launch_worker.cpp:86-368 window / marker / pause logic
//   Queue          preempt/src/xqueue/async_xqueue.cpp:44-150  Submit / WaitAll / Suspend / Resume
//   Scheduler      sched/src/scheduler/local.cpp:142-206 + sched/src/policy/hpf.cpp:8-42
//                  event queue, worker thread, Highest-Priority-First, executor that
//                  resumes the running set and then suspends the rest
//                  (preempt/src/sched/executor.cpp:54-77)
//   CpuDevice      the CPU stand-in for a HIP stream: one executor thread per queue
//                  (level 1 only, as the reference's HIP adapter: hip_queue.h:25-26)
// Only what configuration "two XQueues, level 1, HPF" needs is restated.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <deque>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

extern "C" void oracle_axpy(float alpha, const float *x, float *y, size_t n);
extern "C" void oracle_vecadd(const float *a, const float *b, float *c, size_t n);
extern "C" void oracle_fill_uniform(float *dst, uint64_t first, uint64_t count, uint64_t key);
extern "C" uint64_t oracle_stream_key(uint64_t seed, uint64_t stream);

namespace port
{

using Clock = std::chrono::steady_clock;

enum Kind { kHardware, kWaitAll, kBatchSync, kDestroy };
enum State { kCreated, kPending, kInFlight, kCompleted };

struct Command
{
    Kind kind = kHardware;
    int64_t idx = -1;
    std::function<void()> body;      // the CPU kernel
    bool marker = false;             // completion marker enabled
    // device-side completion (the "event")
    std::mutex dev_mtx;
    std::condition_variable dev_cv;
    bool dev_done = false;
    // host-side state
    std::mutex mtx;
    std::condition_variable cv;
    State state = kCreated;

    void SetState(State s)
    {
        { std::lock_guard<std::mutex> l(mtx); if (s > state) state = s; }
        cv.notify_all();
    }
    void WaitUntil(State s)
    {
        std::unique_lock<std::mutex> l(mtx);
        cv.wait(l, [&] { return state >= s; });
    }
    void DeviceSynchronize()
    {
        std::unique_lock<std::mutex> l(dev_mtx);
        dev_cv.wait(l, [&] { return dev_done; });
    }
};
using Cmd = std::shared_ptr<Command>;

// One executor thread = one in-order device queue.
class CpuDevice
{
public:
    CpuDevice() { thread_ = std::thread([this] { Run(); }); }
    ~CpuDevice()
    {
        { std::lock_guard<std::mutex> l(mtx_); stop_ = true; }
        cv_.notify_all();
        thread_.join();
    }
    void Launch(Cmd c)
    {
        { std::lock_guard<std::mutex> l(mtx_); fifo_.push_back(std::move(c)); launched_++; }
        cv_.notify_one();
    }
    void Synchronize()
    {
        std::unique_lock<std::mutex> l(mtx_);
        const uint64_t target = launched_;
        drained_.wait(l, [&] { return retired_ >= target; });
    }
private:
    void Run()
    {
        while (true) {
            Cmd c;
            {
                std::unique_lock<std::mutex> l(mtx_);
                cv_.wait(l, [&] { return stop_ || !fifo_.empty(); });
                if (fifo_.empty()) return;
                c = std::move(fifo_.front());
                fifo_.pop_front();
            }
            c->body();
            { std::lock_guard<std::mutex> l(c->dev_mtx); c->dev_done = true; }
            c->dev_cv.notify_all();
            { std::lock_guard<std::mutex> l(mtx_); retired_++; }
            drained_.notify_all();
        }
    }
    std::mutex mtx_;
    std::condition_variable cv_, drained_;
    std::deque<Cmd> fifo_;
    uint64_t launched_ = 0, retired_ = 0;
    bool stop_ = false;
    std::thread thread_;
};

class Scheduler;

class Buffer
{
public:
    Buffer(uint64_t handle, Scheduler *sched): handle_(handle), sched_(sched)
    {
        auto first = std::make_shared<Command>();
        first->kind = kWaitAll;
        Enqueue(first);
    }
    void Enqueue(Cmd c);
    Cmd Dequeue();
    Cmd EnqueueWaitAll();
private:
    const uint64_t handle_;
    Scheduler *sched_;
    std::mutex mtx_;
    std::condition_variable cv_;
    bool ready_ = false;
    Cmd last_;
    std::list<Cmd> cmds_;
};

class Worker
{
public:
    Worker(CpuDevice *dev, Buffer *buf, int64_t threshold, int64_t batch)
        : dev_(dev), buf_(buf), threshold_(threshold), batch_(batch)
    {
        thread_ = std::thread([this] { Loop(); });
    }
    ~Worker() { thread_.join(); }
    void Pause() { std::lock_guard<std::mutex> l(mtx_); paused_ = true; pause_count_++; }
    void Resume() { { std::lock_guard<std::mutex> l(mtx_); paused_ = false; } cv_.notify_all(); }

private:
    using Lock = std::unique_lock<std::mutex>;

    void Loop()
    {
        while (true) {
            Cmd c = buf_->Dequeue();
            switch (c->kind) {
            case kHardware: Launch(c); break;
            case kWaitAll:
            { c->SetState(kInFlight); Lock l(mtx_); SyncAll(l); l.unlock(); c->SetState(kCompleted); break; }
            case kBatchSync:
            {
                c->SetState(kInFlight);
                Lock l(mtx_);
                if (!sync_log_.empty()) { Cmd m = sync_log_.front(); SyncCmd(l, m); }
                l.unlock();
                c->SetState(kCompleted);
                break;
            }
            case kDestroy:
            { c->SetState(kInFlight); Lock l(mtx_); SyncAll(l); l.unlock(); c->SetState(kCompleted); return; }
            }
        }
    }

    // launch_worker.cpp:164-263 (level 1: no deactivatable drain)
    void Launch(Cmd c)
    {
        Lock l(mtx_);
        if ((int64_t)log_.size() >= threshold_) {
            Cmd target;
            const int64_t front = log_.front()->idx;
            for (auto &m : sync_log_) if (m->idx >= front) { target = m; break; }
            if (target) SyncCmd(l, target); else SyncAll(l);
        } else {
            while (paused_) cv_.wait(l);
        }
        if (c->idx - last_marker_ >= batch_) c->marker = true;
        dev_->Launch(c);
        c->SetState(kInFlight);
        log_.push_back(c);
        if (c->marker) { sync_log_.push_back(c); last_marker_ = c->idx; }
    }

    void SyncAll(Lock &l)
    {
        while (true) {
            while (paused_) cv_.wait(l);
            if (log_.empty()) return;
            const int64_t cnt = pause_count_;
            l.unlock();
            dev_->Synchronize();
            l.lock();
            if (cnt == pause_count_) break;
        }
        sync_log_.clear();
        for (auto &c : log_) c->SetState(kCompleted);
        log_.clear();
    }

    void SyncCmd(Lock &l, Cmd m)
    {
        while (true) {
            while (paused_) cv_.wait(l);
            const int64_t cnt = pause_count_;
            l.unlock();
            m->DeviceSynchronize();
            l.lock();
            if (cnt == pause_count_) break;
        }
        while (!sync_log_.empty() && sync_log_.front()->idx <= m->idx) sync_log_.pop_front();
        while (!log_.empty() && log_.front()->idx <= m->idx) {
            log_.front()->SetState(kCompleted);
            log_.pop_front();
        }
    }

    CpuDevice *dev_;
    Buffer *buf_;
    const int64_t threshold_, batch_;
    std::list<Cmd> log_, sync_log_;
    int64_t last_marker_ = -1;
    std::mutex mtx_;
    std::condition_variable cv_;
    bool paused_ = false;
    int64_t pause_count_ = 0;
    std::thread thread_;
};

// local.cpp + hpf.cpp: one thread, events in, suspend/resume out.
class Scheduler
{
public:
    struct QueueInfo { int priority = 0; bool ready = false; bool suspended = false;
                       std::function<void()> suspend, resume; };

    Scheduler() { thread_ = std::thread([this] { Loop(); }); }
    ~Scheduler()
    {
        { std::lock_guard<std::mutex> l(mtx_); stop_ = true; }
        cv_.notify_all();
        thread_.join();
    }
    void AddQueue(uint64_t h, int prio, std::function<void()> s, std::function<void()> r)
    {
        std::lock_guard<std::mutex> l(mtx_);
        auto &q = queues_[h];
        q.priority = prio; q.suspend = std::move(s); q.resume = std::move(r);
    }
    void Event(uint64_t h, bool ready)
    {
        { std::lock_guard<std::mutex> l(mtx_); events_.push_back({ h, ready }); }
        cv_.notify_all();
    }
private:
    void Loop()
    {
        std::unique_lock<std::mutex> l(mtx_);
        while (true) {
            cv_.wait(l, [&] { return stop_ || !events_.empty(); });
            if (stop_ && events_.empty()) return;
            auto batch = std::move(events_);
            events_.clear();
            for (auto &e : batch) queues_[e.first].ready = e.second;
            // HPF: bar = highest priority among ready queues; below the bar -> suspend.
            int bar = -255;
            for (auto &q : queues_) if (q.second.ready && q.second.priority > bar) bar = q.second.priority;
            std::vector<std::function<void()>> ops;
            for (auto &q : queues_) if (!(q.second.priority < bar)) { q.second.suspended = false; ops.push_back(q.second.resume); }
            for (auto &q : queues_) if (q.second.priority < bar) { q.second.suspended = true; ops.push_back(q.second.suspend); }
            l.unlock();
            for (auto &op : ops) op();   // resume first, then suspend (executor.cpp:66-76)
            l.lock();
        }
    }
    std::mutex mtx_;
    std::condition_variable cv_;
    std::vector<std::pair<uint64_t, bool>> events_;
    std::map<uint64_t, QueueInfo> queues_;
    bool stop_ = false;
    std::thread thread_;
};

void Buffer::Enqueue(Cmd c)
{
    c->SetState(kPending);
    {
        std::lock_guard<std::mutex> l(mtx_);
        if (c->kind == kHardware && !ready_) { ready_ = true; if (sched_) sched_->Event(handle_, true); }
        last_ = c;
        cmds_.push_back(std::move(c));
    }
    cv_.notify_all();
}

Cmd Buffer::Dequeue()
{
    std::unique_lock<std::mutex> l(mtx_);
    if (!cmds_.empty()) { Cmd c = cmds_.front(); cmds_.pop_front(); return c; }
    if (last_->kind == kWaitAll) {
        if (ready_) { ready_ = false; if (sched_) sched_->Event(handle_, false); }
        cv_.wait(l, [&] { return !cmds_.empty(); });
        Cmd c = cmds_.front(); cmds_.pop_front(); return c;
    }
    auto c = std::make_shared<Command>();
    c->kind = last_->kind == kBatchSync ? kWaitAll : kBatchSync;
    c->SetState(kPending);
    last_ = c;
    return c;
}

Cmd Buffer::EnqueueWaitAll()
{
    std::unique_lock<std::mutex> l(mtx_);
    if (!ready_ || last_->kind == kWaitAll) return last_;
    auto c = std::make_shared<Command>();
    c->kind = kWaitAll;
    c->SetState(kPending);
    last_ = c;
    cmds_.push_back(c);
    l.unlock();
    cv_.notify_all();
    return c;
}

class Queue
{
public:
    Queue(uint64_t handle, Scheduler *sched, int prio, int64_t threshold, int64_t batch)
        : buf_(handle, sched), worker_(&dev_, &buf_, threshold, batch)
    {
        buf_.EnqueueWaitAll()->WaitUntil(kCompleted);
        if (sched) sched->AddQueue(handle, prio, [this] { Suspend(); }, [this] { Resume(); });
    }
    ~Queue()
    {
        Resume();
        auto d = std::make_shared<Command>();
        d->kind = kDestroy;
        buf_.Enqueue(d);
        d->WaitUntil(kCompleted);
    }
    void Submit(std::function<void()> body)
    {
        auto c = std::make_shared<Command>();
        c->body = std::move(body);
        c->idx = next_idx_++;
        buf_.Enqueue(c);
    }
    void WaitAll() { buf_.EnqueueWaitAll()->WaitUntil(kCompleted); }
    void Suspend() { bool e = false; if (suspended_.compare_exchange_strong(e, true)) worker_.Pause(); }
    void Resume() { bool e = true; if (suspended_.compare_exchange_strong(e, false)) worker_.Resume(); }
private:
    CpuDevice dev_;
    Buffer buf_;
    Worker worker_;
    std::atomic<bool> suspended_ { false };
    int64_t next_idx_ = 1;
};

} // namespace port

// Foreground latency under a streaming background, CPU edition.
//   bg: y = 0.5*x + y over bg_n elements, back to back, priority 1, threshold/batch as given
//   fg: the same over fg_n elements every period_us, priority 2, threshold 8 / batch 4
// Writes `samples` foreground latencies (submit -> WaitAll returns, microseconds) twice:
// alone and under contention. Returns the background commands completed while contended
// and the contended phase's wall time.
extern "C" __attribute__((visibility("default")))
int port_run_fg_bg_axpy(uint64_t bg_n, uint64_t fg_n, int64_t period_us, int samples,
                        int bg_threshold, int bg_batch, double *alone_us, double *contended_us,
                        uint64_t *bg_commands, double *contended_seconds, uint64_t *checksum)
{
    using namespace port;
    std::vector<float> bx(bg_n), by(bg_n), fx(fg_n), fy(fg_n);
    oracle_fill_uniform(bx.data(), 0, bg_n, oracle_stream_key(0, 4));
    oracle_fill_uniform(by.data(), 0, bg_n, oracle_stream_key(0, 5));
    oracle_fill_uniform(fx.data(), 0, fg_n, oracle_stream_key(0, 0));
    oracle_fill_uniform(fy.data(), 0, fg_n, oracle_stream_key(0, 1));

    Scheduler sched;
    Queue bg(1, &sched, 1, bg_threshold, bg_batch);
    Queue fg(2, &sched, 2, 8, 4);

    auto fg_once = [&]() {
        const auto t0 = Clock::now();
        fg.Submit([&] { oracle_axpy(0.5f, fx.data(), fy.data(), fg_n); });
        fg.WaitAll();
        return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
    };
    auto run_fg = [&](double *out) {
        auto next = Clock::now();
        for (int i = 0; i < samples; ++i) {
            std::this_thread::sleep_until(next);
            out[i] = fg_once();
            next += std::chrono::microseconds(period_us);
        }
    };

    run_fg(alone_us);

    std::atomic<bool> stop { false };
    std::atomic<uint64_t> done { 0 };
    std::thread bg_thread([&] {
        while (!stop.load()) {
            for (int i = 0; i < 8 && !stop.load(); ++i) {
                bg.Submit([&] { oracle_axpy(0.5f, bx.data(), by.data(), bg_n); done++; });
            }
            bg.WaitAll();
        }
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(50));
    const auto t0 = Clock::now();
    const uint64_t done0 = done.load();
    run_fg(contended_us);
    *bg_commands = done.load() - done0;
    *contended_seconds = std::chrono::duration<double>(Clock::now() - t0).count();
    stop.store(true);
    bg_thread.join();

    uint64_t sum = 0;
    for (uint64_t i = 0; i < fg_n; i += 97) { uint32_t u; memcpy(&u, &fy[i], 4); sum += u; }
    *checksum = sum;
    return 0;
}
