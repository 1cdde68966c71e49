// Device-side preemption guard for Level-2 (deactivate / reactivate) on gfx950.
//
// A kernel that wants to be flushable takes one extra by-value argument, an
// XGuardArgs, and brackets the work of each work-group with the calls below:
//
//     XGuardWave guard(g, wg);      // or XGuardBlock for multi-wave work-groups
//     ... issue the loads of the work-group's inputs ...
//     if (!guard.Enter()) return;   // flushed (or already done): store nothing
//     ... compute, store ...
//     guard.Commit();               // mark the work-group done
//
// Protocol. The queue owns one 32-bit preempt word that counts deactivations.
// Every launch carries the count that was current when it was enqueued
// (`epoch`). A work-group may run only while word == epoch: Deactivate() bumps
// the word, so every work-group that has not yet passed Enter() returns at once
// and the device drains in about the time of one work-group. Work-groups that did
// pass Enter() run to their end and set their bit in `bitmap`. Reactivate()
// enqueues the same kernel again with the new epoch and `resume` set; the
// work-groups whose bit is set return immediately, the others run. Each
// work-group therefore executes exactly once, which makes in-place and atomic
// kernels safe to flush. Stream order guarantees that a replay starts only after
// the flushed launch has left the device, so the bitmap it reads is final.
//
// This is the role of the guardian prologue that XSched injects into CUDA kernels
// by binary instrumentation (reference platforms/cuda/hal/inject/inject.cu:43-83
// check_preempt, :124-140 restore_exec; preempt buffer layout
// platforms/cuda/hal/src/level2/instrument.cpp:177-180). Differences: it is
// compiled into hand-written kernels instead of injected; the flag is an epoch
// counter, so nothing has to be cleared or read back on resume; one bit per
// work-group instead of two words.
//
// Cost: one scalar load per work-group whose latency hides behind the first
// input loads, one compare, and one atomic OR per work-group.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

struct XGuardArgs
{
    const uint32_t *flag;   // the queue's preempt word (deactivation count)
    uint32_t       *bitmap; // 1 bit per work-group, set at Commit(); may be null
    uint32_t        epoch;  // deactivation count this launch was enqueued under
    uint32_t        resume; // nonzero: skip work-groups whose bit is already set
};

#ifndef XGUARD_SCALAR_LOAD
#define XGUARD_SCALAR_LOAD 1
#endif

// The preempt word is written by the host while kernels run, so the load must not
// be served from the scalar data cache or a non-coherent L2 line: a scalar load
// with the GLC bit always fetches memory-side data (the word lives in fine-grained
// memory). Load and wait form one asm statement so the compiler never touches the
// destination register while the load is in flight. Vector loads issued before
// this call stay in flight across it (it waits on the scalar counter only), which
// is how a kernel hides the latency of the word: inputs first, then Enter().
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

__device__ __forceinline__ bool xguard_bit_set(const uint32_t *bitmap, uint32_t wg)
{
    const uint32_t word = __builtin_amdgcn_readfirstlane(__builtin_nontemporal_load(&bitmap[wg >> 5]));
    return ((word >> (wg & 31)) & 1u) != 0;
}

/// Guard of a work-group that is ONE wavefront (blockDim == 64): the decision is
/// wave-uniform by construction, no LDS or barrier is needed.
class XGuardWave
{
public:
    __device__ __forceinline__ XGuardWave(const XGuardArgs &g, uint32_t wg): g_(g), wg_(wg) {}

    /// False: this work-group must not run (flushed, or finished by an earlier launch).
    __device__ __forceinline__ bool Enter() const
    {
        if (xguard_read_flag(g_.flag) != g_.epoch) return false;
        if (g_.resume && g_.bitmap && xguard_bit_set(g_.bitmap, wg_)) return false;
        return true;
    }

    /// Call after the last store of the work-group.
    __device__ __forceinline__ void Commit() const
    {
        if (g_.bitmap && (threadIdx.x & 63) == 0) {
            __hip_atomic_fetch_or(&g_.bitmap[wg_ >> 5], 1u << (wg_ & 31),
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
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
        if (threadIdx.x < 64) {
            bool go = xguard_read_flag(g_.flag) == g_.epoch;
            if (go && g_.resume && g_.bitmap && xguard_bit_set(g_.bitmap, wg_)) go = false;
            if (threadIdx.x == 0) *lds_ = go ? 1u : 0u;
        }
        __syncthreads();
        return *lds_ != 0;
    }

    /// Mid-work re-check for a work-group whose results so far live only in
    /// registers / LDS: when it returns false the work-group abandons itself (its
    /// bit stays clear, a replay redoes it). Every wave of the group must call it
    /// at the same point; it contains two barriers.
    __device__ __forceinline__ bool StillCurrent() const
    {
        __syncthreads();
        if (threadIdx.x == 0) *lds_ = xguard_read_flag(g_.flag) == g_.epoch ? 1u : 0u;
        __syncthreads();
        return *lds_ != 0;
    }

    /// Call after the last store of the work-group (all waves; one barrier inside).
    __device__ __forceinline__ void Commit() const
    {
        __syncthreads();
        if (g_.bitmap && threadIdx.x == 0) {
            __hip_atomic_fetch_or(&g_.bitmap[wg_ >> 5], 1u << (wg_ & 31),
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

private:
    const XGuardArgs &g_;
    const uint32_t wg_;
    uint32_t *lds_;
};
