// Environment-variable access with the reference's parsing rules
// (utils/include/xsched/utils/env.h:8-43): ON/OFF/1/0 case-insensitive options,
// stoll integers, empty string when unset.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <string>
#include <strings.h>

inline std::string GetEnv(const std::string &name)
{
    const char *v = std::getenv(name.c_str());
    return v ? std::string(v) : std::string();
}

inline bool GetEnvInt64(const std::string &name, int64_t &val)
{
    std::string v = GetEnv(name);
    if (v.empty()) return false;
    try { val = std::stoll(v); } catch (...) { return false; }
    return true;
}

inline bool GetEnvOption(const std::string &name, bool dflt = false)
{
    std::string v = GetEnv(name);
    if (v == "0" || strcasecmp(v.c_str(), "off") == 0) return false;
    if (v == "1" || strcasecmp(v.c_str(), "on") == 0) return true;
    return dflt;
}
