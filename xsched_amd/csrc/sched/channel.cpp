// Datagram channel over Unix-domain sockets.
#include <cerrno>
#include <cstring>
#include <algorithm>
#include <poll.h>
#include <sys/prctl.h>
#include <sys/eventfd.h>
#include <sys/socket.h>
#include <sys/stat.h>
#include <sys/un.h>
#include <unistd.h>

#include "xsched/utils/env.h"
#include "xsched/utils/xassert.h"
#include "xsched/protocol/def.h"
#include "xsched/sched/ipc/channel.h"
#include "spin.h"

namespace xsched::sched::ipc
{

std::string Channel::Dir()
{
    std::string dir = GetEnv(XSCHED_SOCKET_DIR_ENV_NAME);
    const bool own_default = dir.empty();
    if (own_default) dir = "/tmp/xsched-" + std::to_string((long)getuid());
    if (mkdir(dir.c_str(), 0700) != 0 && errno != EEXIST) {
        XERRO("cannot create the socket directory %s: %s", dir.c_str(), strerror(errno));
    }
    // A directory somebody else made (or a link to one) would hand them the sockets: it must
    // be a real directory of this user. The default one must also be closed to others; a
    // directory named through the environment is the operator's to open up (several users
    // sharing one daemon).
    struct stat st {};
    if (lstat(dir.c_str(), &st) != 0 || !S_ISDIR(st.st_mode) || st.st_uid != getuid()
        || (own_default && (st.st_mode & 077) != 0)) {
        XERRO("socket directory %s is not a directory owned by uid %ld%s; set %s to a safe one", dir.c_str(),
              (long)getuid(), own_default ? " with mode 0700" : "", XSCHED_SOCKET_DIR_ENV_NAME);
    }
    return dir;
}

std::string Channel::Path(ChannelKey key)
{
    return Dir() + "/xsched-" + std::to_string((long long)key) + ".sock";
}

void Channel::Remove(ChannelKey key) { unlink(Path(key).c_str()); }

static bool FillAddr(const std::string &path, sockaddr_un &addr)
{
    memset(&addr, 0, sizeof(addr));
    addr.sun_family = AF_UNIX;
    if (path.size() >= sizeof(addr.sun_path)) return false;
    memcpy(addr.sun_path, path.c_str(), path.size() + 1);
    return true;
}

Node::Node(ChannelKey key, NodeType type): key_(key), type_(type), path_(Channel::Path(key))
{
    fd_ = socket(AF_UNIX, SOCK_DGRAM | SOCK_CLOEXEC, 0);
    XASSERT(fd_ >= 0, "socket() failed: %s", strerror(errno));
    if (type_ != NodeType::kReceiver) return;

    sockaddr_un addr;
    XASSERT(FillAddr(path_, addr), "socket path too long: %s", path_.c_str());
    unlink(path_.c_str()); // a stale socket of a dead process with the same key
    XASSERT(bind(fd_, (sockaddr *)&addr, sizeof(addr)) == 0,
            "bind(%s) failed: %s", path_.c_str(), strerror(errno));
    wake_fd_ = eventfd(0, EFD_CLOEXEC);
    XASSERT(wake_fd_ >= 0, "eventfd() failed: %s", strerror(errno));
}

Node::~Node()
{
    Remove();
    if (fd_ >= 0) close(fd_);
    if (wake_fd_ >= 0) close(wake_fd_);
}

bool Node::Send(const void *data, size_t size)
{
    if (fd_ < 0 || size > kMaxMessageSize) return false;
    sockaddr_un addr;
    if (!FillAddr(path_, addr)) return false;
    while (true) {
        ssize_t n = sendto(fd_, data, size, MSG_NOSIGNAL, (sockaddr *)&addr, sizeof(addr));
        if (n == (ssize_t)size) return true;
        if (n < 0 && errno == EINTR) continue;
        return false;
    }
}

// One datagram if one is there, without blocking; nullptr otherwise (errno tells which).
std::unique_ptr<Message> Node::TryReceive()
{
    ssize_t n = recv(fd_, rx_, sizeof(rx_), MSG_DONTWAIT);
    if (n < 0) return nullptr;
    return std::make_unique<Message>(std::vector<char>(rx_, rx_ + n));
}

// Bookkeeping for every message. A message after a pause starts a burst. Without a rhythm,
// the times between the last four burst starts become the period when they agree within an
// eighth. With one, a burst that starts a whole number of periods after the last beat (within
// an eighth of the period) is the next beat and corrects the period; any other burst is
// somebody else's (another client's queue going idle, a hint) and changes nothing: the rhythm
// is only given up when its own beats stop coming (Receive counts those).
std::unique_ptr<Message> Node::Arrived(std::unique_ptr<Message> msg)
{
    const auto now = Clock::now();
    if (now - last_message_ > kBurstWindow) {
        if (period_ > Clock::duration::zero()) {
            const auto since = now - burst_start_;
            const int64_t beats = (since + period_ / 2) / period_;
            const auto expected = period_ * beats;
            const auto off = since > expected ? since - expected : expected - since;
            if (beats >= 1 && off * kLatenessDivisor <= period_) {
                if (beats == 1) period_ = (period_ * 3 + since) / 4;
                burst_start_ = now;
                missed_ = 0;
            }
        } else {
            if (burst_start_ != Clock::time_point {}) {
                intervals_[0] = intervals_[1];
                intervals_[1] = intervals_[2];
                intervals_[2] = now - burst_start_;
                const auto mean = (intervals_[0] + intervals_[1] + intervals_[2]) / 3;
                bool steady = intervals_[0] > Clock::duration::zero() && mean >= kShortestPeriod && mean <= kLongestPeriod;
                for (const auto &i : intervals_) {
                    const auto off = i > mean ? i - mean : mean - i;
                    steady = steady && off * kLatenessDivisor <= mean;
                }
                if (steady) { period_ = mean; missed_ = 0; }
            }
            burst_start_ = now;
        }
    }
    last_message_ = now;
    return msg;
}

std::unique_ptr<Message> Node::Receive()
{
    if (type_ != NodeType::kReceiver || removed_.load()) return nullptr;
    const bool ahead = WakeAhead();
    if (ahead && !slack_set_) {
        // the timed sleep below is meant to end on time (the default slack of a thread's timers is 50 us)
        (void)prctl(PR_SET_TIMERSLACK, 1000UL, 0, 0, 0);
        slack_set_ = true;
    }
    // 1. Poll for a while after the last message before blocking: XSCHED_SPIN_US when it is
    //    set, else the length of a burst.
    const auto window = SpinWindow().count() > 0 ? Clock::duration(SpinWindow()) : (ahead ? Clock::duration(kBurstWindow) : Clock::duration::zero());
    auto poll_until = [this](Clock::time_point give_up) -> std::unique_ptr<Message> {
        while (Clock::now() < give_up && !removed_.load(std::memory_order_relaxed)) {
            if (auto msg = TryReceive()) return msg;
            if (errno != EAGAIN && errno != EWOULDBLOCK && errno != EINTR) return nullptr;
            __builtin_ia32_pause();
        }
        return nullptr;
    };
    if (window > Clock::duration::zero()) {
        auto until = last_message_ + window;
        // No rhythm yet, but the last two bursts came close together: the next one is
        // expected as soon, and learning a rhythm takes four of them. Polling through
        // that one pause makes the second and third burst of a periodic sender find the
        // receiver awake already (and a sender that is not periodic but this busy, always).
        if (ahead && period_ == Clock::duration::zero() && intervals_[2] > Clock::duration::zero() &&
            intervals_[2] <= kDensePause && last_message_ - burst_start_ <= kBurstWindow) {
            until = std::max(until, burst_start_ + intervals_[2] + intervals_[2] / 4);
        }
        if (auto msg = poll_until(until)) return Arrived(std::move(msg));
    }
    // 2. A steady rhythm: sleep until shortly before the next burst is due, then poll until
    //    it comes or is clearly late. kBeatsToGiveUp beats in a row that do not come and the
    //    rhythm is forgotten.
    Clock::time_point sleep_until {};
    if (ahead && period_ > Clock::duration::zero() && missed_ < kBeatsToGiveUp) {
        const auto due = burst_start_ + period_ * (missed_ + 1);
        const auto late = std::max<Clock::duration>(period_ / kLatenessDivisor, Clock::duration(WakeAheadMargin()));
        if (Clock::now() < due + late) sleep_until = due - WakeAheadMargin();
    }
    while (true) {
        pollfd fds[2] = { { fd_, POLLIN, 0 }, { wake_fd_, POLLIN, 0 } };
        int rc;
        if (sleep_until != Clock::time_point {}) {
            const auto left = sleep_until - Clock::now();
            const auto ns = std::chrono::duration_cast<std::chrono::nanoseconds>(left).count();
            timespec ts { (time_t)(ns > 0 ? ns / 1000000000 : 0), (long)(ns > 0 ? ns % 1000000000 : 0) };
            rc = ppoll(fds, 2, &ts, nullptr);
        } else {
            rc = poll(fds, 2, -1);
        }
        if (rc < 0) { if (errno == EINTR) continue; return nullptr; }
        if (fds[1].revents != 0 || removed_.load()) return nullptr;
        if (rc == 0) {
            // up ahead of the burst
            const auto due = burst_start_ + period_ * (missed_ + 1);
            const auto late = std::max<Clock::duration>(period_ / kLatenessDivisor, Clock::duration(WakeAheadMargin()));
            sleep_until = Clock::time_point {};
            if (auto msg = poll_until(due + late)) return Arrived(std::move(msg));
            missed_++;
            if (missed_ < kBeatsToGiveUp && !removed_.load()) sleep_until = burst_start_ + period_ * (missed_ + 1) - WakeAheadMargin();
            else { period_ = Clock::duration::zero(); intervals_[0] = intervals_[1] = intervals_[2] = Clock::duration::zero(); }
            continue;
        }
        if (!(fds[0].revents & POLLIN)) continue;
        if (auto msg = TryReceive()) return Arrived(std::move(msg));
        if (errno == EINTR || errno == EAGAIN || errno == EWOULDBLOCK) continue;
        return nullptr;
    }
}

void Node::Remove()
{
    if (removed_.exchange(true)) return;
    if (type_ == NodeType::kReceiver) {
        unlink(path_.c_str());
        uint64_t one = 1;
        if (wake_fd_ >= 0) { ssize_t r = write(wake_fd_, &one, sizeof(one)); (void)r; }
    }
}

} // namespace xsched::sched::ipc
