// XSCHED_SPIN_US: how long a thread that waits for scheduler traffic (the daemon's receiver,
// a client's receiver of operations, the scheduler's round thread) keeps polling after its
// last message before it blocks in the kernel. 0 (the default) blocks at once. A blocked
// thread costs 10-50 us to wake (futex or poll wake-up of an idle core); with events every few
// milliseconds a window of a few milliseconds keeps the three hops of a cross-process
// preemption (client -> daemon -> round thread -> other client) at a few microseconds each,
// at the price of one busy core per waiting thread.
//
// Without the variable a receiver of the daemon channel (Node::Receive) still does two
// bounded things, both switched off by XSCHED_WAKE_AHEAD=OFF: it polls for kBurstWindow after
// each message (the messages of one scheduling decision follow each other within tens of
// microseconds), and when the pauses between such bursts have been equal three times in a row
// (a client that submits every few milliseconds) it sleeps until shortly before the next
// burst is due and polls from there, so the message that starts a preemption finds it awake.
#pragma once

#include <chrono>
#include <cstdint>

#include "xsched/utils/env.h"

namespace xsched::sched
{

inline std::chrono::microseconds SpinWindow()
{
    static const int64_t us = []() {
        int64_t v = 0;
        return GetEnvInt64("XSCHED_SPIN_US", v) && v > 0 ? v : (int64_t)0;
    }();
    return std::chrono::microseconds(us);
}

/// A pause longer than this ends a burst of messages; also how long a receiver polls after a
/// message when XSCHED_SPIN_US does not say otherwise.
inline constexpr std::chrono::microseconds kBurstWindow { 250 };
/// Periods a receiver is prepared to follow, how early it is up before a burst is due, and
/// how far past the due time it keeps polling, as a fraction of the period (at least the wake-ahead margin).
inline constexpr std::chrono::microseconds kShortestPeriod { 400 }, kLongestPeriod { 100000 };
inline constexpr int kLatenessDivisor = 8;
/// Beats in a row that fail to come before a receiver stops following the rhythm.
inline constexpr int kBeatsToGiveUp = 3;
/// Without a rhythm: a pause between two bursts up to this long makes the receiver poll through the next one.
inline constexpr std::chrono::microseconds kDensePause { 3000 };

inline bool WakeAhead()
{
    static const bool on = GetEnvOption("XSCHED_WAKE_AHEAD", true);
    return on;
}

/// How long before a burst is due the receiver is up and polling (XSCHED_WAKE_AHEAD_US).
inline std::chrono::microseconds WakeAheadMargin()
{
    static const int64_t us = []() {
        int64_t v = 400;
        return GetEnvInt64("XSCHED_WAKE_AHEAD_US", v) && v > 0 ? v : (int64_t)400;
    }();
    return std::chrono::microseconds(us);
}

} // namespace xsched::sched
