// Fatal assertion: a false condition logs and exits (reference
// utils/include/xsched/utils/xassert.h:9-15).
#pragma once

#include "xsched/utils/log.h"

#define XASSERT(cond, ...) \
    do { if (UNLIKELY(!(cond))) { XERRO(__VA_ARGS__); } } while (0)
