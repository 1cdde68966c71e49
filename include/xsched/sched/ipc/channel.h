// Host-side message channel between application processes and the scheduler
// daemon. A channel is named by an integer key (the daemon listens on key 1,
// each client on its pid) and carries whole records, one per datagram, over a
// Unix-domain socket "<dir>/xsched-<key>.sock". Plays the role of the
// ipc::Node objects used at reference sched/src/scheduler/global.cpp:17-69 and
// service/server/src/server.cpp:47-202.
#pragma once

#include <atomic>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

namespace xsched::sched::ipc
{

typedef int64_t ChannelKey;

enum class NodeType { kSender, kReceiver };

class Message
{
public:
    explicit Message(std::vector<char> bytes): bytes_(std::move(bytes)) {}
    const void *Data() const { return bytes_.data(); }
    size_t Size() const { return bytes_.size(); }
private:
    std::vector<char> bytes_;
};

class Node
{
public:
    Node(ChannelKey key, NodeType type);
    ~Node();

    /// False when the receiver does not exist (any more) or the record is too big.
    bool Send(const void *data, size_t size);
    /// Blocks; nullptr once the node has been removed.
    std::unique_ptr<Message> Receive();
    /// Close the node; a blocked Receive() returns nullptr. A receiver also
    /// unlinks its socket path.
    void Remove();

    static constexpr size_t kMaxMessageSize = 4096;

private:
    const ChannelKey key_;
    const NodeType type_;
    std::string path_;
    int fd_ = -1;
    int wake_fd_ = -1;
    std::atomic_bool removed_ { false };

    // Receiver thread only: when messages came, to be awake when the next one does.
    using Clock = std::chrono::steady_clock;
    std::unique_ptr<Message> TryReceive();
    std::unique_ptr<Message> Arrived(std::unique_ptr<Message> msg);
    Clock::time_point last_message_ {};
    Clock::time_point burst_start_ {};       // first message after a pause; with a rhythm: the last beat
    Clock::duration intervals_[3] {};        // between the last four such moments
    Clock::duration period_ {};              // their common value when they agree, else zero
    int missed_ = 0;                         // predictions in a row that nothing came of
    bool slack_set_ = false;
    char rx_[kMaxMessageSize];
};

class Channel
{
public:
    /// Socket directory: $XSCHED_SOCKET_DIR or /tmp/xsched-<uid>.
    static std::string Dir();
    static std::string Path(ChannelKey key);
    /// Unlink the socket of a dead peer.
    static void Remove(ChannelKey key);
};

} // namespace xsched::sched::ipc
