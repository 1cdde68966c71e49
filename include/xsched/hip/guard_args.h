// The arguments of the work-group entry guard (xsched/hip/guard.h), as a plain struct that
// host code can include without the HIP device headers: the last parameter of every guarded
// kernel, filled in by the queue at each launch. All zeroes switches the guard off.
#pragma once

#include <stdint.h>

struct XGuardArgs
{
    const uint32_t *flag;      // the queue's preempt word, copy 0 (deactivation count)
    uint8_t        *done;      // progress map: done[w] == gen once work-group w has committed; may be null
    uint32_t        epoch;     // deactivation count this launch was enqueued under
    uint32_t        resume;    // nonzero: skip work-groups that have already committed
    uint32_t        flag_mask; // number of copies of the preempt word minus one (2^k - 1)
    uint32_t        gen;       // generation tag of this command in its progress map (1..255)
    uint32_t       *flushed;   // the queue's "a work-group of this epoch was flushed" word; may be null
};
