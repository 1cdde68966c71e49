// XSCHED_SPIN_US: how long a thread that waits for scheduler traffic (the daemon's receiver,
// a client's receiver of operations, the scheduler's round thread) keeps polling after its
// last message before it blocks in the kernel. 0 (the default) blocks at once. A blocked
// thread costs 10-50 us to wake (futex or poll wake-up of an idle core); with events every few
// milliseconds a window of a few milliseconds keeps the three hops of a cross-process
// preemption (client -> daemon -> round thread -> other client) at a few microseconds each,
// at the price of one busy core per waiting thread.
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

} // namespace xsched::sched
