#include <cstdarg>

#include "xsched/utils/log.h"

namespace xsched::utils
{

// One fprintf per line so that lines of different threads do not interleave.
// Shape: "[XSCHED LEVEL @ T tid @ hh:mm:ss.us] message @ file:line"
// (reference utils/include/xsched/utils/log.h:79-96).
void LogLine(int level, const char *tag, const char *file, int line, const char *fmt, ...)
{
    static const bool tty = isatty(fileno(stderr)) != 0;
    static const char *colors[] = { "\x1b[31m", "\x1b[33m", "\x1b[32m", "\x1b[36m" };

    char msg[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(msg, sizeof(msg), fmt, ap);
    va_end(ap);

    const auto now = std::chrono::system_clock::now();
    const time_t tt = std::chrono::system_clock::to_time_t(now);
    std::tm lt{};
    localtime_r(&tt, &lt);
    const long us = (long)(std::chrono::duration_cast<std::chrono::microseconds>(
        now.time_since_epoch()).count() % 1000000);

    fprintf(stderr, "[XSCHED %s%s%s @ T " FMT_TID " @ %02d:%02d:%02d.%06ld] %s @ %s:%d\n",
            tty ? colors[level & 3] : "", tag, tty ? "\x1b[0m" : "",
            GetThreadId(), lt.tm_hour, lt.tm_min, lt.tm_sec, us, msg, file, line);
    if (level == XLOG_LEVEL_DEBG) fflush(stderr);
}

} // namespace xsched::utils
