// xserver: the scheduler daemon for one machine. It owns a LocalScheduler with the
// chosen policy, receives the event records of every client process on the well-known
// channel (key 1), keeps one sending channel per client (key = client pid) and forwards
// the operations the scheduler emits to the process they are addressed to. Clients that
// disappear without saying so are detected by polling their pid and reported to the
// scheduler as destroyed. Role and flow follow reference
// service/server/src/server.cpp:47-202 (Run, RecvWorker, Execute, ProcessTerminate). With a
// port it also serves the reference daemon's control plane over HTTP, route for route and
// field for field (service/server/src/server.cpp:28-39,270-543; status fields as
// service/common/src/convert.cpp:7-17), so that its command-line client can talk to it:
//   GET  /xqueues            {"xqueues":[{handle,device,level,pid,threshold,batch_size,ready,suspended}...],
//                             "processes":[{pid,cmdline}...]}
//   GET  /xqueue/<hex>       {"xqueue":{...},"process":{...}}            404 for an unknown handle
//   POST /config/<hex>?level=&threshold=&batch_size=    a configuration operation for the owner
//   GET  /policy             {"policy":<XPolicyType>}
//   POST /policy?policy=<n>  switches the policy
//   POST /hint               body {"hint_type":..,...}: priority, utilization, timeslice, window-active
//
//   usage: xserver <policy> [port]        e.g.  xserver HPF 50000
// Without a port nothing listens on the network. XSCHED_SERVER_ADDR (default 127.0.0.1) is
// the address to bind; the reference binds every interface.
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

#include "http.h"
#include "xsched/utils/env.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "xsched/protocol/names.h"
#include "xsched/sched/ipc/channel.h"
#include "xsched/sched/policy/policy.h"
#include "xsched/sched/scheduler/local.h"

using namespace xsched::sched;
using namespace xsched::protocol;
using namespace xsched::service;

namespace
{

std::atomic<bool> g_stop { false };
std::unique_ptr<ipc::Node> g_recv;

class Server
{
public:
    Server(XPolicyType policy, int port): scheduler_(std::make_unique<LocalScheduler>(policy)), port_(port) {}

    void Run()
    {
        g_recv = std::make_unique<ipc::Node>((ipc::ChannelKey)XSCHED_SERVER_CHANNEL_KEY, ipc::NodeType::kReceiver);
        scheduler_->SetExecutor([this](std::shared_ptr<const Operation> op) { this->Execute(op); });
        // Events come in on this process's own threads, which hold nothing an operation could
        // need: they run the scheduling rounds themselves (one wake-up less per preemption).
        scheduler_->RunRoundsOnCallers(GetEnvOption("XSCHED_SERVER_INLINE_ROUNDS", true) ? LocalScheduler::kRoundsOnCallersAll
                                                                                          : LocalScheduler::kRoundsOnCallersOff);
        scheduler_->Run();
        std::thread reaper([this]() { this->ReapLoop(); });
        if (port_ > 0) {
            std::string addr = GetEnv("XSCHED_SERVER_ADDR");
            if (addr.empty()) addr = "127.0.0.1";
            if (http_.Start(addr, port_, [this](const HttpRequest &req, HttpResponse &res) { this->Serve(req, res); })) {
                XINFO("xserver: control plane on http://%s:%d", addr.c_str(), http_.Port());
            }
        }
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
        http_.Stop();
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

    // ---- control plane (reference server.cpp:204-543) -----------------------------------------

    static void Fail(HttpResponse &res, int status, const char *error = nullptr)
    {
        res.status = status;
        res.body = error ? JsonWriter().BeginObject().Key("error").String(error).EndObject().Text() : "";
    }

    static void Say(HttpResponse &res, const char *key, const char *text)
    {
        res.body = JsonWriter().BeginObject().Key(key).String(text).EndObject().Text();
    }

    static void WriteStatus(JsonWriter &w, const XQueueStatus &s)
    {
        w.BeginObject().Key("handle").UInt(s.handle).Key("device").UInt(s.device).Key("level").Int(s.level)
         .Key("pid").Int(s.pid).Key("threshold").Int(s.threshold).Key("batch_size").Int(s.batch_size)
         .Key("ready").Bool(s.ready).Key("suspended").Bool(s.suspended).EndObject();
    }

    static void WriteProcess(JsonWriter &w, const ProcessInfo &p)
    {
        w.BeginObject().Key("pid").Int(p.pid).Key("cmdline").String(p.cmdline).EndObject();
    }

    /// The scheduler thread fills the query in its next round (queries are events).
    void Ask(StatusQuery &query, XQueueHandle handle)
    {
        if (handle != 0) scheduler_->RecvEvent(std::make_shared<XQueueQueryEvent>(handle, &query));
        else scheduler_->RecvEvent(std::make_shared<XQueueQueryAllEvent>(&query));
        query.Wait();
    }

    /// "/prefix/<hex handle>" -> handle; 0 when the rest is no non-zero hexadecimal number.
    static XQueueHandle HandleIn(const std::string &path, const std::string &prefix)
    {
        uint64_t h = 0;
        std::string hex = path.substr(prefix.size());
        if (hex.rfind("0x", 0) == 0 || hex.rfind("0X", 0) == 0) hex = hex.substr(2);
        return ParseUInt64(hex, 16, &h) ? h : 0;
    }

    void Serve(const HttpRequest &req, HttpResponse &res)
    {
        const bool get = req.method == "GET", post = req.method == "POST";
        if (get && req.path == "/xqueues") return GetXQueues(res);
        if (get && req.path.rfind("/xqueue/", 0) == 0) return GetXQueue(HandleIn(req.path, "/xqueue/"), res);
        if (post && req.path.rfind("/config/", 0) == 0) return PostConfig(HandleIn(req.path, "/config/"), req, res);
        if (get && req.path == "/policy") {
            res.body = JsonWriter().BeginObject().Key("policy").Int(scheduler_->GetPolicy()).EndObject().Text();
            return;
        }
        if (post && req.path == "/policy") return PostPolicy(req, res);
        if (post && req.path == "/hint") return PostHint(req, res);
        Fail(res, 404);
    }

    void GetXQueues(HttpResponse &res)
    {
        StatusQuery query(true);
        Ask(query, 0);
        JsonWriter w;
        w.BeginObject().Key("xqueues").BeginArray();
        for (auto &s : query.status_) WriteStatus(w, *s);
        w.EndArray().Key("processes").BeginArray();
        for (auto &p : query.processes_) WriteProcess(w, *p);
        w.EndArray().EndObject();
        res.body = w.Text();
    }

    void GetXQueue(XQueueHandle handle, HttpResponse &res)
    {
        if (handle == 0) return Fail(res, 400);
        StatusQuery query(true);
        Ask(query, handle);
        if (query.status_.empty() || query.processes_.empty()) return Fail(res, 404);
        JsonWriter w;
        w.BeginObject().Key("xqueue");
        WriteStatus(w, *query.status_[0]);
        w.Key("process");
        WriteProcess(w, *query.processes_[0]);
        w.EndObject();
        res.body = w.Text();
    }

    void PostConfig(XQueueHandle handle, const HttpRequest &req, HttpResponse &res)
    {
        if (handle == 0) return Fail(res, 400);
        int64_t level = kPreemptLevelUnknown, threshold = -1, batch = -1;
        auto it = req.query.find("level");
        if (it != req.query.end() && (!ParseInt64(it->second, &level) || level <= kPreemptLevelUnknown || level >= kPreemptLevelMax)) {
            return Fail(res, 400, "invalid level");
        }
        it = req.query.find("threshold");
        if (it != req.query.end() && (!ParseInt64(it->second, &threshold) || threshold <= 0)) {
            return Fail(res, 400, "invalid command threshold");
        }
        it = req.query.find("batch_size");
        if (it != req.query.end() && (!ParseInt64(it->second, &batch) || batch <= 0)) {
            return Fail(res, 400, "invalid command batch size");
        }
        StatusQuery query(false);
        Ask(query, handle);
        if (query.status_.empty()) return Fail(res, 404, "XQueue not found");
        const XQueueStatus &now = *query.status_[0];
        const int64_t new_threshold = threshold > 0 ? threshold : now.threshold;
        const int64_t new_batch = batch > 0 ? batch : now.batch_size;
        // the reference's daemon asks for strictly less (server.cpp:366-370), stricter than the queue itself
        if (new_batch >= new_threshold) return Fail(res, 400, "batch size must be less than threshold");
        if (level == kPreemptLevelUnknown && threshold == -1 && batch == -1) return Say(res, "warning", "no change");
        Execute(std::make_shared<ConfigOperation>(scheduler_->NextOperationId(now.pid), now.pid, handle,
                                                  (XPreemptLevel)level, threshold, batch));
        Say(res, "info", "success");
    }

    void PostPolicy(const HttpRequest &req, HttpResponse &res)
    {
        auto it = req.query.find("policy");
        int64_t type = 0;
        if (it == req.query.end() || !ParseInt64(it->second, &type) || type <= kPolicyUnknown || type >= kPolicyMax) {
            return Fail(res, 400);
        }
        if (!PolicyAvailable((XPolicyType)type)) return Fail(res, 400, "policy has no implementation");
        scheduler_->SetPolicy((XPolicyType)type);
        Say(res, "info", "success");
    }

    void Hint(std::shared_ptr<const xsched::sched::Hint> hint) { scheduler_->RecvEvent(std::make_shared<HintEvent>(hint)); }

    void PostHint(const HttpRequest &req, HttpResponse &res)
    {
        std::map<std::string, std::string> body;
        if (!ParseFlatJsonObject(req.body, &body)) return Fail(res, 400);
        auto number = [&](const char *key, int64_t *out) {
            auto it = body.find(key);
            return it != body.end() && ParseInt64(it->second, out);
        };
        auto handle_of = [&]() {
            uint64_t h = 0;
            auto it = body.find("handle");
            return it != body.end() && ParseUInt64(it->second, 10, &h) ? h : 0;
        };
        int64_t type = 0;
        if (body.find("hint_type") == body.end()) return Fail(res, 400, "missing hint type");
        if (!number("hint_type", &type) || type <= kHintTypeUnknown || type >= kHintTypeMax) return Fail(res, 400, "invalid hint type");
        switch ((HintType)type) {
        case kHintTypePriority:
        {
            const XQueueHandle handle = handle_of();
            int64_t prio = 0;
            if (handle == 0) return Fail(res, 400, "invalid handle");
            if (body.find("priority") == body.end()) return Fail(res, 400, "missing priority");
            if (!number("priority", &prio) || prio < PRIORITY_MIN || prio > PRIORITY_MAX) return Fail(res, 400, "invalid priority");
            Hint(std::make_shared<PriorityHint>(handle, (Priority)prio));
            return Say(res, "info", "success");
        }
        case kHintTypeUtilization:
        {
            const XQueueHandle handle = handle_of();
            int64_t pid = 0, util = 0;
            (void)number("pid", &pid);
            if (handle == 0 && pid == 0) return Fail(res, 400, "handle or pid is required");
            if (body.find("utilization") == body.end()) return Fail(res, 400, "missing utilization");
            if (!number("utilization", &util) || util < UTILIZATION_MIN || util > UTILIZATION_MAX) return Fail(res, 400, "invalid utilization");
            Hint(std::make_shared<UtilizationHint>((PID)pid, handle, (Utilization)util));
            return Say(res, "info", "success");
        }
        case kHintTypeTimeslice:
        {
            int64_t ts = 0;
            if (body.find("timeslice") == body.end()) return Fail(res, 400, "missing timeslice");
            if (!number("timeslice", &ts) || ts <= 0) return Fail(res, 400, "invalid timeslice");
            Hint(std::make_shared<TimesliceHint>((Timeslice)ts));
            return Say(res, "info", "success");
        }
        case kHintTypeWindowActive:
        {
            int64_t pid = 0;
            uint64_t display = 0;
            if (!number("pid", &pid)) return Fail(res, 400, "missing pid");
            auto it = body.find("display");
            if (it == body.end() || !ParseUInt64(it->second, 10, &display)) return Fail(res, 400, "missing display");
            Hint(std::make_shared<WindowActiveHint>((PID)pid, display));
            return Say(res, "info", "success");
        }
        default:
            return Fail(res, 400, "invalid hint type");
        }
    }

    std::unique_ptr<LocalScheduler> scheduler_;
    const int port_;
    HttpServer http_;
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
        fprintf(stderr, "usage: %s <policy: HPF | HHPF | CHPF | UP | PUP | KEDF | LAX | AWF | CFS | MLFQ> [port of the HTTP control plane; none when left out]\n", argv[0]);
        return 2;
    }
    const XPolicyType policy = GetPolicyType(argv[1]);
    if (!xsched::sched::PolicyAvailable(policy)) {
        fprintf(stderr, "xserver: policy '%s' is not available\n", argv[1]);
        return 2;
    }
    signal(SIGINT, OnSignal);
    signal(SIGTERM, OnSignal);
    int64_t port = 0;
    if (argc >= 3) {
        if (!ParseInt64(argv[2], &port) || port < 0 || port > 65535) {
            fprintf(stderr, "xserver: '%s' is not a port\n", argv[2]);
            return 2;
        }
    }
    Server server(policy, (int)port);
    server.Run();
    return 0;
}
