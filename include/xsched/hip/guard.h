// Device-side preemption guard for Level-2 (deactivate / reactivate) on gfx950.
//
// A kernel that wants to be flushable takes one extra by-value argument, an
// XGuardArgs, and brackets the work of each work-group with the calls below:
//
//     XGuardWave guard(g, wg);      // or XGuardBlock for multi-wave work-groups
//     if (!guard.Enter()) return;   // flushed (or already done): touch nothing
//     ... compute, store ...
//     guard.Commit();               // mark the work-group done
//
// Protocol. The queue owns one 32-bit preempt word that counts deactivations.
// Every launch carries the count that was current when it was enqueued
// (`epoch`). A work-group may run only while word == epoch: Deactivate() bumps
// the word, so every work-group that has not yet passed Enter() returns at once
// and the device drains in about the time of one work-group. Work-groups that did
// pass Enter() run to their end and record themselves in the progress map `done`
// (one byte per work-group, holding the generation tag of the command).
// Reactivate() enqueues the same kernel again with the new epoch and `resume`
// set; the work-groups already recorded return immediately, the others run. Each
// work-group therefore executes exactly once, which makes in-place and atomic
// kernels safe to flush. Stream order guarantees that a replay starts only after
// the flushed launch has left the device, so the progress map it reads is final.
// The generation tag makes a recycled map valid without clearing it: bytes left by
// an earlier command carry another tag.
//
// This is the role of the guardian prologue that XSched injects into CUDA kernels
// by binary instrumentation (reference platforms/cuda/hal/inject/inject.cu:43-83
// check_preempt, :124-140 restore_exec; preempt buffer layout
// platforms/cuda/hal/src/level2/instrument.cpp:177-180). Differences: it is
// compiled into hand-written kernels instead of injected; the flag is an epoch
// counter, so nothing has to be cleared or read back on resume; one byte per
// work-group instead of two words.
//
// Cost: one uncached and one cached scalar load per work-group (hidden by the other
// resident waves), two compares, and one byte store per work-group.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "xsched/hip/guard_args.h"

// The preempt word is replicated: copy c lives at flag[c * kXGuardFlagStrideWords],
// c in [0, flag_mask]. Uncached reads of ONE address are served one after the other by
// a single memory channel (about 27 ns each on MI355X), which would cap a kernel at
// some 37 M work-groups per second; work-group w reads copy (w & flag_mask), so the
// reads spread over many channels. The host rewrites all copies on a deactivation, one
// after the other: for the microseconds that takes, work-groups that read different
// copies disagree. Within one launch that is harmless, each work-group decides for
// itself. Across launches it would let a work-group of a LATER launch run (its copy still
// old) although a work-group of an EARLIER launch has been flushed (its copy already
// new), and read what the flushed one has not written yet. The queue's `flushed` word
// closes that: a work-group that finds its copy changed stores the epoch of its launch
// there before it leaves, and every work-group also refuses to run when it finds its own
// epoch in that word. The word lives in ordinary cached memory: what a launch stored is
// visible to every later launch of the stream (kernel boundary), which is all that is
// needed, and reading it costs a cache hit. A kernel that needs ALL work-groups of an
// earlier launch (not just "none flushed") still has to check their progress bytes.
#define kXGuardFlagStrideWords 64u /* 256 bytes between copies */


__device__ __forceinline__ const uint32_t *xguard_flag_copy(const XGuardArgs &g, uint32_t wg)
{
    return g.flag + (size_t)(wg & g.flag_mask) * kXGuardFlagStrideWords;
}

#ifndef XGUARD_SCALAR_LOAD
#define XGUARD_SCALAR_LOAD 1
#endif

// The preempt word is written by the host while kernels run, so the load must not
// be served from the scalar data cache or a non-coherent L2 line: a scalar load
// with the GLC bit always fetches memory-side data (the word lives in fine-grained
// memory). Load and wait form one asm statement so the compiler never touches the
// destination register while the load is in flight. Vector loads issued before
// this call stay in flight across it (it waits on the scalar counter only).
__device__ __forceinline__ uint32_t xguard_read_flag(const uint32_t *flag)
{
    uint32_t v;
#if XGUARD_SCALAR_LOAD
    asm volatile("s_load_dword %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(v) : "s"(flag) : "memory");
#else
    v = __builtin_amdgcn_readfirstlane(
        __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM));
#endif
    return v;
}

// The same read in two halves, for a loop that has other work to do while the word is
// on its way: Begin() issues the load, End() hands out the value. This one is a VECTOR
// load (every lane reads the same word, one memory request): vector loads return in
// order and are counted apart from LDS operations, so the wait the compiler places in
// front of End()'s use covers this load and older ones only. The scalar load above
// shares its counter with LDS operations and returns out of order, so waiting for it
// means waiting for every LDS atomic the wave has issued - which stalls a loop that
// lives on having many of them in flight.
__device__ __forceinline__ uint32_t xguard_read_flag_begin(const uint32_t *flag)
{
    return __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ uint32_t xguard_read_flag_end(uint32_t v)
{
    return __builtin_amdgcn_readfirstlane(v);
}

__device__ __forceinline__ bool xguard_committed(const XGuardArgs &g, uint32_t wg)
{
    const uint32_t tag = __builtin_amdgcn_readfirstlane((uint32_t)__builtin_nontemporal_load(&g.done[wg]));
    return tag == g.gen;
}

// A plain (cached) byte store: the L2 merges the bytes of neighbouring work-groups
// into whole lines. A non-temporal store or an atomic OR here costs 3-4 % of a
// streaming kernel's bandwidth on MI355X, the cached store well under 1 %.
__device__ __forceinline__ void xguard_commit(const XGuardArgs &g, uint32_t wg)
{
    g.done[wg] = (uint8_t)g.gen;
}

/// Called by ONE lane of a work-group that leaves because its copy of the preempt word
/// has changed (at entry or at a later look): later launches of this epoch must not run.
__device__ __forceinline__ void xguard_note_flush(const XGuardArgs &g)
{
    if (g.flushed) *g.flushed = g.epoch;
}

/// The `flushed` word (wave-uniform); a value no launch carries when the queue has none.
__device__ __forceinline__ uint32_t xguard_read_flushed(const XGuardArgs &g)
{
    return g.flushed != nullptr ? (uint32_t)__builtin_amdgcn_readfirstlane((int)*g.flushed) : ~g.epoch;
}

/// The work-group's byte of the progress map (wave-uniform).
__device__ __forceinline__ uint32_t xguard_read_tag(const XGuardArgs &g, uint32_t wg)
{
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)__builtin_nontemporal_load(&g.done[wg]));
}

/// True when an earlier launch of this epoch has been flushed (wave-uniform).
__device__ __forceinline__ bool xguard_epoch_flushed(const XGuardArgs &g)
{
    return g.flushed != nullptr && (uint32_t)__builtin_amdgcn_readfirstlane((int)*g.flushed) == g.epoch;
}

/// An XGuardArgs of all zeroes switches the guard off: every work-group runs and nothing is
/// recorded. It is what a program passes that launches a guarded kernel itself, with no
/// queue behind the launch (`kernel<<<grid, block, 0, stream>>>(..., XGuardArgs{})`).
__device__ __forceinline__ bool xguard_inert(const XGuardArgs &g) { return g.flag == nullptr; }

/// Guard of a work-group that is ONE wavefront (blockDim == 64): the decision is
/// wave-uniform by construction, no LDS or barrier is needed.
class XGuardWave
{
public:
    __device__ __forceinline__ XGuardWave(const XGuardArgs &g, uint32_t wg): g_(g), wg_(wg) {}

    /// False: this work-group must not run (flushed, or finished by an earlier launch).
    __device__ __forceinline__ bool Enter() const
    {
        if (xguard_inert(g_)) return true;
        const uint32_t flushed_word = xguard_read_flushed(g_);
        const uint32_t copy = xguard_read_flag(xguard_flag_copy(g_, wg_));
        const bool replay_with_map = g_.resume && g_.done;
        const uint32_t tag = replay_with_map && copy == g_.epoch ? xguard_read_tag(g_, wg_) : 0u;
        const XGuardVerdict v = xguard_entry_verdict(copy, flushed_word, g_.epoch, g_.resume, g_.done != nullptr, tag, g_.gen);
        if (v.note_flush && (threadIdx.x & 63) == 0) xguard_note_flush(g_);
        return v.run != 0;
    }

    /// Call after the last store of the work-group.
    __device__ __forceinline__ void Commit() const
    {
        if (g_.done && (threadIdx.x & 63) == 0) xguard_commit(g_, wg_);
    }

private:
    const XGuardArgs &g_;
    const uint32_t wg_;
};

/// Guard of a multi-wave work-group: wave 0 decides, the decision is shared through
/// one LDS word and a barrier so that all waves of the group agree.
class XGuardBlock
{
public:
    __device__ __forceinline__ XGuardBlock(const XGuardArgs &g, uint32_t wg, uint32_t *lds_word)
        : g_(g), wg_(wg), lds_(lds_word) {}

    __device__ __forceinline__ bool Enter() const
    {
        if (xguard_inert(g_)) return true;
        if (threadIdx.x < 64) {
            const uint32_t flushed_word = xguard_read_flushed(g_);
            const uint32_t copy = xguard_read_flag(xguard_flag_copy(g_, wg_));
            const bool replay_with_map = g_.resume && g_.done;
            const uint32_t tag = replay_with_map && copy == g_.epoch ? xguard_read_tag(g_, wg_) : 0u;
            const XGuardVerdict v = xguard_entry_verdict(copy, flushed_word, g_.epoch, g_.resume, g_.done != nullptr, tag, g_.gen);
            if (threadIdx.x == 0) {
                if (v.note_flush) xguard_note_flush(g_);
                *lds_ = v.run;
            }
        }
        __syncthreads();
        return *lds_ != 0;
    }

    /// Mid-work re-check for a work-group whose results so far live only in
    /// registers / LDS: when it returns false the work-group abandons itself (its
    /// byte stays untagged, a replay redoes it). Every wave of the group must call it
    /// at the same point; it contains two barriers.
    __device__ __forceinline__ bool StillCurrent() const
    {
        if (xguard_inert(g_)) return true;
        __syncthreads();
        if (threadIdx.x == 0) {
            const XGuardVerdict v = xguard_recheck_verdict(xguard_read_flag(xguard_flag_copy(g_, wg_)), g_.epoch);
            if (v.note_flush) xguard_note_flush(g_);
            *lds_ = v.run;
        }
        __syncthreads();
        return *lds_ != 0;
    }

    /// Barrier-free variant of the re-check for the calling wave alone (the result is
    /// wave-uniform). The kernel has to make the waves of the group agree before any of
    /// them produces a side effect, e.g. through an LDS word and the barrier it already
    /// has in front of its write-out.
    __device__ __forceinline__ bool WaveStillCurrent() const
    {
        if (xguard_inert(g_)) return true;
        const XGuardVerdict v = xguard_recheck_verdict(xguard_read_flag(xguard_flag_copy(g_, wg_)), g_.epoch);
        if (v.note_flush && (threadIdx.x & 63) == 0) xguard_note_flush(g_);
        return v.run != 0;
    }

    /// WaveStillCurrent() split in two so that the read of the preempt word overlaps the
    /// work between the calls: `pending = WavePollBegin(); ...; if (!WavePollEnd(pending))`.
    __device__ __forceinline__ uint32_t WavePollBegin() const
    {
        if (xguard_inert(g_)) return g_.epoch;
        return xguard_read_flag_begin(xguard_flag_copy(g_, wg_));
    }

    __device__ __forceinline__ bool WavePollEnd(uint32_t pending) const
    {
        const XGuardVerdict v = xguard_recheck_verdict(xguard_read_flag_end(pending), g_.epoch);
        if (v.note_flush && (threadIdx.x & 63) == 0) xguard_note_flush(g_);
        return v.run != 0;
    }

    /// Call after the last store of the work-group (all waves; one barrier inside).
    __device__ __forceinline__ void Commit() const
    {
        __syncthreads();
        if (g_.done && threadIdx.x == 0) xguard_commit(g_, wg_);
    }

private:
    const XGuardArgs &g_;
    const uint32_t wg_;
    uint32_t *lds_;
};
