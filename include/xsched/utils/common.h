// Small portable helpers shared by every layer (Linux only).
// Covers the parts of reference utils/include/xsched/utils/common.h:28-175 that
// the command-queue path uses: branch hints, class-shape macros, symbol export,
// printf formats and process / thread ids.
#pragma once

#include <cerrno>
#include <cinttypes>
#include <cstdint>
#include <cstring>
#include <string>
#include <sys/syscall.h>
#include <unistd.h>

#define LIKELY(x)   __builtin_expect(!!(x), 1)
#define UNLIKELY(x) __builtin_expect(!!(x), 0)

#define NO_COPY_CLASS(T) T(const T &) = delete; T &operator=(const T &) = delete;
#define NO_MOVE_CLASS(T) T(T &&) = delete; T &operator=(T &&) = delete;
#define STATIC_CLASS(T)  T() = delete; ~T() = delete; NO_COPY_CLASS(T) NO_MOVE_CLASS(T)

#define UNUSED(expr) do { (void)(expr); } while (0)
#define ROUND_UP(x, a)   ((((x) + (a) - 1) / (a)) * (a))
#define ROUND_DOWN(x, a) ((x) / (a) * (a))

#ifdef __cplusplus
#define EXPORT_C_FUNC   extern "C" __attribute__((visibility("default")))
#define EXPORT_CXX_FUNC __attribute__((visibility("default")))
#else
#define EXPORT_C_FUNC   __attribute__((visibility("default")))
#endif

#define FMT_32D "%" PRId32
#define FMT_32U "%" PRIu32
#define FMT_64D "%" PRId64
#define FMT_64U "%" PRIu64
#define FMT_64X "%" PRIx64
#define FMT_TID FMT_32D
#define FMT_PID FMT_32D

typedef pid_t TID;
typedef pid_t PID;

inline TID GetThreadId()
{
    static const thread_local TID tid = (TID)syscall(SYS_gettid);
    return tid;
}

// Not cached: a forked child must see its own pid.
inline PID GetProcessId() { return getpid(); }
