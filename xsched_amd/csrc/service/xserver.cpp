// xserver: the scheduler daemon for one machine. It owns a LocalScheduler with the
// chosen policy, receives the event records of every client process on the well-known
// channel (key 1), keeps one sending channel per client (key = client pid) and forwards
// the operations the scheduler emits to the process they are addressed to. Clients that
// disappear without saying so are detected by polling their pid and reported to the
// scheduler as destroyed. Role and flow follow reference
// service/server/src/server.cpp:47-202 (Run, RecvWorker, Execute, ProcessTerminate); the
// HTTP control plane of the reference (routes for xcli) is not part of this daemon.
//
//   usage: xserver <policy> [ignored-port]        e.g.  xserver HPF
#include <atomic>
#include <cerrno>
#include <chrono>
#include <csignal>
#include <cstdio>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "xsched/protocol/names.h"
#include "xsched/sched/ipc/channel.h"
#include "xsched/sched/policy/policy.h"
#include "xsched/sched/scheduler/local.h"

using namespace xsched::sched;
using namespace xsched::protocol;

namespace
{

std::atomic<bool> g_stop { false };
std::unique_ptr<ipc::Node> g_recv;

class Server
{
public:
    explicit Server(XPolicyType policy): scheduler_(std::make_unique<LocalScheduler>(policy)) {}

    void Run()
    {
        g_recv = std::make_unique<ipc::Node>((ipc::ChannelKey)XSCHED_SERVER_CHANNEL_KEY, ipc::NodeType::kReceiver);
        scheduler_->SetExecutor([this](std::shared_ptr<const Operation> op) { this->Execute(op); });
        scheduler_->Run();
        std::thread reaper([this]() { this->ReapLoop(); });
        XINFO("xserver: policy %s, listening on %s", GetPolicyTypeName(scheduler_->GetPolicy()).c_str(),
              ipc::Channel::Path(XSCHED_SERVER_CHANNEL_KEY).c_str());

        while (!g_stop.load()) {
            auto msg = g_recv->Receive();
            if (msg == nullptr) break;
            if (!Event::WireRecordOk(msg->Data(), msg->Size())) {
                XWARN("xserver: dropped a malformed or unknown event record of %zu bytes", msg->Size());
                continue;
            }
            auto e = Event::CopyConstructor(msg->Data());
            switch (e->Type()) {
            case kEventSchedulerTerminate:
                g_stop.store(true);
                break;
            case kEventProcessCreate:
            {
                const PID pid = e->Pid();
                // A recycled pid must not inherit a dead client's queues (server.cpp:123-126).
                scheduler_->RecvEvent(std::make_shared<ProcessDestroyEvent>(pid));
                Forget(pid);
                {
                    std::lock_guard<std::mutex> lock(mtx_);
                    clients_[pid] = std::make_shared<ipc::Node>((ipc::ChannelKey)pid, ipc::NodeType::kSender);
                }
                XINFO("xserver: client " FMT_PID " connected: %s", pid,
                      static_cast<const ProcessCreateEvent *>(e.get())->Cmdline());
                scheduler_->RecvEvent(e);
                break;
            }
            case kEventProcessDestroy:
                scheduler_->RecvEvent(e);
                Forget(e->Pid());
                break;
            case kEventXQueueQuery:
            case kEventXQueueQueryAll:
                break; // carry pointers: only valid inside the sender's process
            default:
                scheduler_->RecvEvent(e);
                break;
            }
        }
        g_stop.store(true);
        reaper.join();
        scheduler_->Stop();
        g_recv->Remove();
        XINFO("xserver: stopped");
    }

private:
    void Execute(std::shared_ptr<const Operation> op)
    {
        std::shared_ptr<ipc::Node> chan;
        {
            std::lock_guard<std::mutex> lock(mtx_);
            auto it = clients_.find(op->Pid());
            if (it == clients_.end()) return; // the client left while the round was running
            chan = it->second;
        }
        if (!chan->Send(op->Data(), op->Size())) {
            // The client is gone: purge its queues too, or they would stay "ready" in the
            // scheduler's mirror and keep lower-priority queues suspended for good.
            XWARN("xserver: cannot reach client " FMT_PID ", dropping it", op->Pid());
            Drop(op->Pid());
        }
    }

    void Forget(PID pid)
    {
        std::lock_guard<std::mutex> lock(mtx_);
        clients_.erase(pid);
    }

    /// A client died without a ProcessDestroy event.
    void Drop(PID pid)
    {
        Forget(pid);
        scheduler_->RecvEvent(std::make_shared<ProcessDestroyEvent>(pid));
        ipc::Channel::Remove((ipc::ChannelKey)pid);
    }

    // Clients that died without a ProcessDestroy event (reference: pidfd/epoll waiter,
    // utils/include/xsched/utils/waitpid.h:27-87).
    void ReapLoop()
    {
        while (!g_stop.load()) {
            std::this_thread::sleep_for(std::chrono::milliseconds(100));
            std::vector<PID> dead;
            {
                std::lock_guard<std::mutex> lock(mtx_);
                for (auto &c : clients_) if (kill(c.first, 0) != 0 && errno == ESRCH) dead.push_back(c.first);
            }
            for (PID pid : dead) {
                XINFO("xserver: client " FMT_PID " is gone", pid);
                Drop(pid);
            }
        }
    }

    std::unique_ptr<LocalScheduler> scheduler_;
    std::mutex mtx_;
    std::map<PID, std::shared_ptr<ipc::Node>> clients_;
};

void OnSignal(int)
{
    g_stop.store(true);
    if (g_recv) g_recv->Remove();
}

} // namespace

int main(int argc, char **argv)
{
    if (argc < 2) {
        fprintf(stderr, "usage: %s <policy: HPF | HHPF | CHPF | UP | PUP | KEDF | LAX | AWF | CFS | MLFQ> [port, unused]\n", argv[0]);
        return 2;
    }
    const XPolicyType policy = GetPolicyType(argv[1]);
    if (!xsched::sched::PolicyAvailable(policy)) {
        fprintf(stderr, "xserver: policy '%s' is not available\n", argv[1]);
        return 2;
    }
    signal(SIGINT, OnSignal);
    signal(SIGTERM, OnSignal);
    Server server(policy);
    server.Run();
    return 0;
}
