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

// ---- the guard's decisions as plain functions --------------------------------------------
// Device code (xsched/hip/guard.h) reads the words and calls these; a CPU test calls the same
// functions from a simulation in which the copies of the preempt word change one at a time.
// What a work-group may do with the values it has read:
//   copy          its copy of the preempt word, read after the launch started
//   flushed_word  the queue's `flushed` word, read after the launch started
//   my_tag        its byte of the progress map (only looked at for replays)
#if defined(__HIPCC__)
#define XGUARD_FN __host__ __device__ static inline
#else
#define XGUARD_FN static inline
#endif

struct XGuardVerdict
{
    uint32_t run;         // nonzero: the work-group may start (or go on)
    uint32_t note_flush;  // nonzero: it must store its epoch into the `flushed` word before it leaves
};

/// At work-group entry. The work-group leaves when its copy no longer shows its launch's epoch
/// (a deactivation has reached it: later launches of the epoch must hear of it), when an
/// EARLIER launch of the same epoch was flushed (its copy may simply not have been rewritten
/// yet), or when a replay finds its own tag in the progress map (it ran before the flush).
XGUARD_FN struct XGuardVerdict xguard_entry_verdict(uint32_t copy, uint32_t flushed_word, uint32_t epoch,
                                                    uint32_t resume, uint32_t has_map, uint32_t my_tag, uint32_t gen)
{
    struct XGuardVerdict v;
    v.note_flush = copy != epoch;
    v.run = copy == epoch && flushed_word != epoch && !(resume && has_map && my_tag == gen);
    return v;
}

/// At a later look of a work-group that has no side effect yet (it abandons itself when told
/// not to go on, its progress byte stays untagged).
XGUARD_FN struct XGuardVerdict xguard_recheck_verdict(uint32_t copy, uint32_t epoch)
{
    struct XGuardVerdict v;
    v.note_flush = copy != epoch;
    v.run = copy == epoch;
    return v;
}
