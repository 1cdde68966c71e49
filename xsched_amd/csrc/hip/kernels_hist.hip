// Guarded integer histogram for gfx950: bins[keys[i]] += 1, keys int32 in
// [0, n_bins), n_bins <= 65536, bins uint32.
//
// HBM-bound on the keys (4 bytes per key) as long as the counting keeps up. A
// work-group of 512 threads owns a contiguous chunk of kChunkKeys keys and counts
// in three tiers, chosen for skewed (Zipf-like) keys where a handful of bins take
// a third of all keys:
//   tier 0  keys < kBallotBins: wave ballot. Per key value one ballot + popcount,
//           accumulated in a scalar register per wave - no memory traffic at all.
//   tier 1  keys < kLdsBins: LDS-privatised 32-bit counters (64 KiB per group),
//           LDS atomics without return.
//   tier 2  the cold tail: atomics straight to the global bins.
// At the end the group flushes its non-zero private counters to the global bins
// with atomic adds. Integer adds commute, so the result does not depend on the
// order in which work-groups (or replays) run.
//
// Guard: work-group entry. Tier-2 atomics go to global memory while the group is
// running, so a group that has started must finish (exactly-once); it commits its
// byte in the progress map after the flush.
#include "hip_hal.h"
#include "xsched/hip/hal.h"

using namespace xsched::preempt;

namespace xsched::hip
{

namespace hist
{

constexpr uint32_t kThreads = 512;
constexpr uint32_t kChunkKeys = 1u << 16;   // keys per work-group
constexpr uint32_t kBallotBins = 8;
constexpr uint32_t kLdsBins = 1u << 14;     // 64 KiB of LDS

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

template <bool kGuard>
__global__ __launch_bounds__(kThreads)
void HistogramKernel(const int32_t *__restrict__ keys, uint64_t n, uint32_t *__restrict__ bins,
                     uint32_t n_bins, XGuardArgs g)
{
    __shared__ uint32_t lds_bins[kLdsBins];
    __shared__ uint32_t guard_word;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t lds_used = n_bins < kLdsBins ? n_bins : kLdsBins;

    for (uint32_t i = tid; i < lds_used; i += kThreads) lds_bins[i] = 0;

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        if (!guard.Enter()) return; // Enter() contains the barrier that also publishes the zeroed bins
    } else {
        __syncthreads();
    }

    const uint64_t begin = (uint64_t)blockIdx.x * kChunkKeys;
    const uint64_t end = begin + kChunkKeys < n ? begin + kChunkKeys : n;

    uint32_t hot[kBallotBins];
#pragma unroll
    for (uint32_t b = 0; b < kBallotBins; ++b) hot[b] = 0;

    auto count = [&](int32_t key, bool valid) {
        const uint32_t k = (uint32_t)key;
#pragma unroll
        for (uint32_t b = 0; b < kBallotBins; ++b) {
            const uint64_t m = __ballot(valid && k == b);
            hot[b] += (uint32_t)__popcll(m);
        }
        if (valid && k >= kBallotBins) {
            if (k < lds_used) __hip_atomic_fetch_add(&lds_bins[k], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            else if (k < n_bins) __hip_atomic_fetch_add(&bins[k], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    // 128-bit loads over the aligned body of the chunk, scalars for the ragged ends.
    const bool aligned = (((uintptr_t)keys) & 15) == 0;
    uint64_t i = begin;
    if (aligned && (begin & 3) == 0) {
        const uint64_t vec_end = begin + ((end - begin) & ~(uint64_t)3);
        // Uniform trip count per group so that the ballots see all lanes.
        for (uint64_t base = begin; base < vec_end; base += (uint64_t)kThreads * 4) {
            const uint64_t idx = base + (uint64_t)tid * 4;
            const bool valid = idx < vec_end;
            i32x4 v = { 0, 0, 0, 0 };
            if (valid) v = __builtin_nontemporal_load((const i32x4 *)(keys + idx));
            count(v.x, valid);
            count(v.y, valid);
            count(v.z, valid);
            count(v.w, valid);
        }
        i = vec_end;
    }
    for (uint64_t base = i; base < end; base += kThreads) {
        const uint64_t idx = base + tid;
        const bool valid = idx < end;
        const int32_t key = valid ? keys[idx] : 0;
        count(key, valid);
    }

    __syncthreads();

    // Flush. Ballot counters are per wave: lane 0 of each wave adds them.
    if (lane == 0) {
#pragma unroll
        for (uint32_t b = 0; b < kBallotBins; ++b) {
            if (hot[b] != 0 && b < n_bins) {
                __hip_atomic_fetch_add(&bins[b], hot[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    for (uint32_t b = tid; b < lds_used; b += kThreads) {
        const uint32_t c = lds_bins[b];
        if (c != 0) __hip_atomic_fetch_add(&bins[b], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        guard.Commit();
    }
}

class HipHistogramCommand final : public HipGuardedCommand
{
public:
    HipHistogramCommand(const void *keys, size_t n, void *bins, uint32_t n_bins, uint32_t n_wg,
                        int guard_mode)
        : HipGuardedCommand(n_wg, guard_mode)
        , keys_((const int32_t *)keys), n_(n), bins_((uint32_t *)bins), n_bins_(n_bins) {}

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        if (n_ == 0) return hipSuccess;
        const dim3 grid(n_wg_), block(kThreads);
        if (guarded) hipLaunchKernelGGL(HistogramKernel<true>, grid, block, 0, stream, keys_, (uint64_t)n_, bins_, n_bins_, g);
        else         hipLaunchKernelGGL(HistogramKernel<false>, grid, block, 0, stream, keys_, (uint64_t)n_, bins_, n_bins_, g);
        return hipGetLastError();
    }

private:
    const int32_t *keys_;
    const size_t n_;
    uint32_t *bins_;
    const uint32_t n_bins_;
};

} // namespace hist

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipHistogramCommandCreate(HwCommandHandle *cmd, const void *keys, size_t n,
                                                void *bins, uint32_t n_bins, int guard)
{
    if (cmd == nullptr || bins == nullptr || (n != 0 && keys == nullptr) || guard < 0 || guard > 2) {
        return kXSchedErrorInvalidValue;
    }
    if (n_bins == 0 || n_bins > 65536) return kXSchedErrorInvalidValue;
    const uint64_t n_wg = n == 0 ? 1 : (n + hist::kChunkKeys - 1) / hist::kChunkKeys;
    if (n_wg > GuardState::kMaxWorkGroups) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<hist::HipHistogramCommand>(
        keys, n, bins, n_bins, (uint32_t)n_wg, guard));
    return kXSchedSuccess;
}
