// Datagram channel over Unix-domain sockets.
#include <cerrno>
#include <cstring>
#include <poll.h>
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

std::unique_ptr<Message> Node::Receive()
{
    if (type_ != NodeType::kReceiver || removed_.load()) return nullptr;
    std::vector<char> buf(kMaxMessageSize);
    // Poll for a while after the last message before blocking (off unless XSCHED_SPIN_US is set).
    const auto window = SpinWindow();
    if (window.count() > 0) {
        const auto give_up = last_message_ + window;
        while (std::chrono::steady_clock::now() < give_up && !removed_.load(std::memory_order_relaxed)) {
            ssize_t n = recv(fd_, buf.data(), buf.size(), MSG_DONTWAIT);
            if (n >= 0) {
                last_message_ = std::chrono::steady_clock::now();
                buf.resize((size_t)n);
                return std::make_unique<Message>(std::move(buf));
            }
            if (errno != EAGAIN && errno != EWOULDBLOCK && errno != EINTR) return nullptr;
            __builtin_ia32_pause();
        }
    }
    while (true) {
        pollfd fds[2] = { { fd_, POLLIN, 0 }, { wake_fd_, POLLIN, 0 } };
        int rc = poll(fds, 2, -1);
        if (rc < 0) { if (errno == EINTR) continue; return nullptr; }
        if (fds[1].revents != 0 || removed_.load()) return nullptr;
        if (!(fds[0].revents & POLLIN)) continue;
        ssize_t n = recv(fd_, buf.data(), buf.size(), 0);
        if (n < 0) { if (errno == EINTR || errno == EAGAIN) continue; return nullptr; }
        last_message_ = std::chrono::steady_clock::now();
        buf.resize((size_t)n);
        return std::make_unique<Message>(std::move(buf));
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
