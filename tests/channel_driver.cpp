// Test driver for the daemon channel's receiver (include/xsched/sched/ipc/channel.h): a sender
// thread sends bursts of two records at a fixed period, the receiver thread notes how long each
// first record of a burst was on its way and how much CPU time receiving cost, during the
// periodic phase and during a silent phase after it.
//   channel_driver PERIOD_US BURSTS SILENT_MS [NOISE_US]   (NOISE_US: a second sender's record every so often, off the beat)
// prints: median_us=<first-record delivery> cpu_frac_periodic=<..> cpu_ms_silent=<..> received=<n>
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <time.h>
#include <unistd.h>
#include <vector>

#include "xsched/sched/ipc/channel.h"

using namespace xsched::sched::ipc;
using Clock = std::chrono::steady_clock;

static double ThreadCpuMs()
{
    timespec ts;
    clock_gettime(CLOCK_THREAD_CPUTIME_ID, &ts);
    return ts.tv_sec * 1e3 + ts.tv_nsec / 1e6;
}

struct Record { int64_t sent_ns; int32_t first; int32_t stop; };

int main(int argc, char **argv)
{
    const int period_us = argc > 1 ? atoi(argv[1]) : 4000, bursts = argc > 2 ? atoi(argv[2]) : 150, silent_ms = argc > 3 ? atoi(argv[3]) : 200, noise_us = argc > 4 ? atoi(argv[4]) : 0;
    const ChannelKey key = (ChannelKey)getpid();
    Node rx(key, NodeType::kReceiver);
    std::vector<double> latency_us;
    std::atomic<double> cpu_periodic { 0 }, cpu_silent { 0 };
    std::atomic<int> received { 0 };
    std::atomic<bool> periodic_over { false };

    std::thread receiver([&]() {
        const double c0 = ThreadCpuMs();
        double c1 = c0;
        while (auto msg = rx.Receive()) {
            Record r;
            if (msg->Size() != sizeof r) continue;
            memcpy(&r, msg->Data(), sizeof r);
            const int64_t now = std::chrono::duration_cast<std::chrono::nanoseconds>(Clock::now().time_since_epoch()).count();
            if (r.stop == 1) { c1 = ThreadCpuMs(); cpu_periodic = c1 - c0; continue; }   // end of the periodic phase
            if (r.stop == 2) break;                                                       // end of the silent phase
            if (r.first) latency_us.push_back((now - r.sent_ns) / 1e3);
            received++;
        }
        cpu_silent = ThreadCpuMs() - c1;
    });

    Node tx(key, NodeType::kSender);
    auto send = [&](int first, int stop) {
        Record r { std::chrono::duration_cast<std::chrono::nanoseconds>(Clock::now().time_since_epoch()).count(), first, stop };
        if (!tx.Send(&r, sizeof r)) { fprintf(stderr, "send failed\n"); exit(2); }
    };
    std::atomic<bool> noise_stop { false };
    std::thread noise([&]() {
        if (noise_us <= 0) return;
        Node other(key, NodeType::kSender);
        while (!noise_stop.load()) {
            std::this_thread::sleep_for(std::chrono::microseconds(noise_us));
            Record r { 0, 0, 0 };
            (void)other.Send(&r, sizeof r);
        }
    });
    const auto t0 = Clock::now();
    auto next = t0;
    for (int b = 0; b < bursts; ++b) {
        while (Clock::now() < next) {}      // the sender is on time to the microsecond: the test is about the receiver
        send(1, 0);
        const auto gap = Clock::now() + std::chrono::microseconds(30);
        while (Clock::now() < gap) {}
        send(0, 0);
        next += std::chrono::microseconds(period_us);
    }
    const double wall_ms = std::chrono::duration<double, std::milli>(Clock::now() - t0).count();
    noise_stop = true;
    noise.join();
    send(0, 1);
    std::this_thread::sleep_for(std::chrono::milliseconds(silent_ms));
    send(0, 2);
    receiver.join();
    std::sort(latency_us.begin(), latency_us.end());
    // the first bursts teach the receiver the rhythm: the median is over the second half
    std::vector<double> tail(latency_us.begin() + latency_us.size() / 2, latency_us.end());
    if (getenv("CHANNEL_DRIVER_VERBOSE") && !latency_us.empty()) {
        for (double q : { 0.1, 0.25, 0.5, 0.75, 0.9, 0.99 }) fprintf(stderr, "p%.0f=%.1f ", q * 100, latency_us[(size_t)(q * latency_us.size())]);
        fprintf(stderr, "\n");
    }
    printf("median_us=%.1f late_half_median_us=%.1f cpu_frac_periodic=%.3f cpu_ms_silent=%.2f received=%d\n",
           latency_us.empty() ? -1.0 : latency_us[latency_us.size() / 2], tail.empty() ? -1.0 : tail[tail.size() / 2],
           cpu_periodic.load() / wall_ms, cpu_silent.load(), received.load());
    return 0;
}
