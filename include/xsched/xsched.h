/* Umbrella header of the C API. reference include/xsched/xsched.h */
#ifndef XSCHED_XSCHED_H_
#define XSCHED_XSCHED_H_
#include "xsched/types.h"
#include "xsched/xqueue.h"
#include "xsched/hint.h"
#endif
