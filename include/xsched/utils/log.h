// Leveled stderr logging. Line shape and XLOG_LEVEL handling follow reference
// utils/include/xsched/utils/log.h:40-126; XERRO terminates the process, which
// is the library's convention for internal failures.
#pragma once

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <ctime>

#include "xsched/utils/common.h"
#include "xsched/utils/env.h"

#define XLOG_LEVEL_ERRO 0
#define XLOG_LEVEL_WARN 1
#define XLOG_LEVEL_INFO 2
#define XLOG_LEVEL_DEBG 3

namespace xsched::utils
{

inline int LogLevel()
{
    static const int level = []() {
        const std::string s = GetEnv("XLOG_LEVEL");
        if (s.empty())   return XLOG_LEVEL_DEBG;
        if (s == "ERRO") return XLOG_LEVEL_ERRO;
        if (s == "WARN") return XLOG_LEVEL_WARN;
        if (s == "DEBG") return XLOG_LEVEL_DEBG;
        return XLOG_LEVEL_INFO;
    }();
    return level;
}

__attribute__((format(printf, 5, 6)))
void LogLine(int level, const char *tag, const char *file, int line, const char *fmt, ...);

} // namespace xsched::utils

#define XLOG_AT(lv, tag, ...) \
    do { if ((lv) <= xsched::utils::LogLevel()) \
        xsched::utils::LogLine((lv), tag, __FILE__, __LINE__, __VA_ARGS__); } while (0)

#ifdef XSCHED_DEBUG_LOG
#define XDEBG(...) XLOG_AT(XLOG_LEVEL_DEBG, "DEBG", __VA_ARGS__)
#else
#define XDEBG(...) do {} while (0)
#endif
#define XINFO(...) XLOG_AT(XLOG_LEVEL_INFO, "INFO", __VA_ARGS__)
#define XWARN(...) XLOG_AT(XLOG_LEVEL_WARN, "WARN", __VA_ARGS__)
#define XERRO(...) \
    do { XLOG_AT(XLOG_LEVEL_ERRO, "ERRO", __VA_ARGS__); fflush(stderr); exit(EXIT_FAILURE); } while (0)
