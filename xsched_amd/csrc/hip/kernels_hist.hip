// Guarded integer histogram for gfx950: bins[keys[i]] += 1, keys int32 in
// [0, n_bins), n_bins <= 65536, bins uint32.
//
// The keys are read once (4 bytes per key); what bounds the kernel on MI355X is the
// LDS atomic unit (a 64-lane ds_add on random addresses retires in ~38 cycles per
// CU) and, before this layout, VALU issue: a wave64 vector instruction occupies its
// SIMD for four cycles, so every compare per key counts.
//
// One work-group of 1024 threads per compute unit owns a contiguous chunk of keys
// (sized so that a launch has about one work-group per CU) and keeps everything it
// counts on chip until the end:
//   hot    keys < kHotBins: wave ballot + popcount into scalar registers. For skewed
//          (Zipf-like) keys these few bins take a quarter of all keys and would
//          otherwise serialise the LDS atomics of a wave on one address.
//   main   keys < kLdsBins (32768): LDS-privatised 32-bit counters, 128 KiB.
//   tail   keys >= kLdsBins: appended as 16-bit values to an LDS list (28 KiB), one
//          list reservation per wave and iteration.
// Only then does it touch global memory: a sweep of atomic adds over its non-zero
// counters (a wave covers 256 consecutive bins, so the adds arrive line by line; each
// group starts its sweep at a different segment because atomics on ONE cache line
// retire at only ~0.1 G/s); then the same 128 KiB are cleared, the listed tail keys
// are counted into them and swept out the same way (scattered global atomics, one per
// tail key, retire at ~25 G/s device-wide: too slow). If the list overflows (an
// adversarial distribution), the group re-reads its chunk for the tail keys instead.
//
// Guard: entry check, and because a group has no side effects before its write-out,
// every wave re-reads the preempt word every second iteration and the group abandons
// itself (its progress byte stays untagged, a replay redoes the chunk). The write-out
// runs to completion and commits. Integer adds commute, so the result does not depend
// on the order in which work-groups (or replays) run.
#include "hip_hal.h"
#include "xsched/hip/hal.h"

using namespace xsched::preempt;

namespace xsched::hip
{

namespace hist
{

constexpr uint32_t kThreads = 1024;
constexpr uint32_t kWaves = kThreads / 64;
#ifndef XSCHED_HIST_HOT_BINS
#define XSCHED_HIST_HOT_BINS 2
#endif
constexpr uint32_t kHotBins = XSCHED_HIST_HOT_BINS;
constexpr uint32_t kLdsBins = 1u << 15;       // 128 KiB of counters
constexpr uint32_t kTailCap = 14336;          // 16-bit entries, 28 KiB
#ifndef XSCHED_HIST_UNITS
#define XSCHED_HIST_UNITS 4
#endif
constexpr uint32_t kUnits = XSCHED_HIST_UNITS;  // 128-bit loads per thread and iteration
constexpr uint32_t kUnitKeys = kThreads * 4;
constexpr uint32_t kIterKeys = kUnitKeys * kUnits;
constexpr uint32_t kMinChunk = kUnitKeys;
constexpr uint32_t kMaxChunk = 1u << 18;
constexpr uint32_t kTargetGroups = 256;       // compute units of an MI355X
constexpr uint32_t kSegBins = 256;            // bins one wave sweeps per step
constexpr uint32_t kSegs = kLdsBins / kSegBins;

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

/// Keys per work-group for a histogram of n keys: a multiple of kMinChunk.
inline uint32_t ChunkFor(uint64_t n)
{
    uint64_t c = (n + kTargetGroups - 1) / kTargetGroups;
    c = (c + kMinChunk - 1) / kMinChunk * kMinChunk;
    if (c < kMinChunk) c = kMinChunk;
    if (c > kMaxChunk) c = kMaxChunk;
    return (uint32_t)c;
}

struct Shared
{
    uint32_t bins[kLdsBins];
    uint16_t tail[kTailCap];
    uint32_t tail_count;
    uint32_t bailed;
    uint32_t guard_word;
};

__device__ __forceinline__ void LdsAdd(uint32_t *p, uint32_t v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

__device__ __forceinline__ void GlobalAdd(uint32_t *p, uint32_t v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/// dst[0] += lo, dst[1] += hi with ONE 64-bit atomic (dst is 8-byte aligned): the
/// write-out is bound by the number of atomic operations, and this halves it. The two
/// counters stay independent 32-bit values: should the low one wrap, the returned old
/// value shows it and the carry that leaked into the high one is taken back (PairFix).
/// Issue and check are separate calls so that a sweep has all its atomics in flight
/// before it looks at the first returned value.
__device__ __forceinline__ uint32_t PairAdd(uint32_t *dst, uint32_t lo, uint32_t hi)
{
    return (uint32_t)__hip_atomic_fetch_add((unsigned long long *)dst, ((unsigned long long)hi << 32) | lo,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void PairFix(uint32_t *dst, uint32_t old_lo, uint32_t lo)
{
    if ((uint32_t)(old_lo + lo) < lo) GlobalAdd(dst + 1, 0xFFFFFFFFu);
}

/// acc += popcount(mask), issued where it is written. Left to the compiler, the
/// popcounts of a whole iteration sink below the per-key branches and their 64-bit
/// lane masks are spilled and reloaded.
__device__ __forceinline__ void AddPopcount(uint32_t &acc, uint64_t mask)
{
    uint32_t tmp;
    asm volatile("s_bcnt1_i32_b64 %1, %2\n\ts_add_u32 %0, %0, %1" : "+s"(acc), "=&s"(tmp) : "s"(mask) : "scc");
}

/// Adds the non-zero counters of sh.bins[0, count) to dst[0, count), never touching
/// memory at or beyond dst + count. Wave q of the group sweeps segments rot + q,
/// rot + q + 16, ... (mod kSegs), so groups that write out at the same time start on
/// different cache lines.
__device__ __forceinline__ void SweepOut(Shared &sh, uint32_t *dst, uint32_t count, uint32_t rot)
{
    constexpr uint32_t kSteps = kSegs / kWaves;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool pair_ok = (((uintptr_t)dst) & 7) == 0; // segment starts are even indices
    uint32_t low[kSteps][2], old[kSteps][2];
#pragma unroll
    for (uint32_t step = 0; step < kSteps; ++step) {
        const uint32_t seg = (rot + step * kWaves + wave) & (kSegs - 1);
        const uint32_t b4 = seg * kSegBins + lane * 4;
        // counters at or beyond `count` are never incremented, so they read zero
        const u32x4 c = b4 < count ? *(const u32x4 *)&sh.bins[b4] : u32x4 { 0, 0, 0, 0 };
        const uint32_t v[4] = { c.x, c.y, c.z, c.w };
#pragma unroll
        for (uint32_t p = 0; p < 2; ++p) {
            const uint32_t i = b4 + p * 2, lo = v[p * 2], hi = v[p * 2 + 1];
            low[step][p] = 0;
            old[step][p] = 0;
            if ((lo | hi) == 0) continue;
            if (pair_ok && i + 1 < count) {
                low[step][p] = lo;
                old[step][p] = PairAdd(dst + i, lo, hi);
            } else {
                if (lo != 0 && i < count) GlobalAdd(dst + i, lo);
                if (hi != 0 && i + 1 < count) GlobalAdd(dst + i + 1, hi);
            }
        }
    }
#pragma unroll
    for (uint32_t step = 0; step < kSteps; ++step) {
        const uint32_t seg = (rot + step * kWaves + wave) & (kSegs - 1);
        const uint32_t b4 = seg * kSegBins + lane * 4;
#pragma unroll
        for (uint32_t p = 0; p < 2; ++p) PairFix(dst + b4 + p * 2, old[step][p], low[step][p]);
    }
}

__device__ __forceinline__ void ClearBins(Shared &sh)
{
    for (uint32_t i = threadIdx.x * 4; i < kLdsBins; i += kThreads * 4) *(u32x4 *)&sh.bins[i] = u32x4 { 0, 0, 0, 0 };
}

template <bool kGuard>
__global__ __launch_bounds__(kThreads)
void HistogramKernel(const int32_t *__restrict__ keys, uint64_t n, uint32_t *__restrict__ bins,
                     uint32_t n_bins, uint32_t chunk, XGuardArgs g)
{
    __shared__ __attribute__((aligned(16))) Shared sh;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t lds_used = n_bins < kLdsBins ? n_bins : kLdsBins;
    // unsigned "k - lo < range" tests: one subtract and one compare per tier, and the
    // sentinel 0xFFFFFFFF of an absent key fails all of them
    const uint32_t main_range = lds_used > kHotBins ? lds_used - kHotBins : 0;
    const uint32_t tail_range = n_bins > kLdsBins ? n_bins - kLdsBins : 0;
    XGuardBlock guard(g, blockIdx.x, &sh.guard_word);

    ClearBins(sh);
    if (tid == 0) { sh.tail_count = 0; sh.bailed = 0; }

    if (kGuard) {
        if (!guard.Enter()) return; // Enter() contains the barrier that also publishes the cleared counters
    } else {
        __syncthreads();
    }

    const uint64_t begin = (uint64_t)blockIdx.x * chunk;
    const uint64_t end = begin + chunk < n ? begin + chunk : n;
    const bool vec_ok = (((uintptr_t)keys) & 15) == 0; // chunk starts are multiples of 4 keys

    uint32_t hot[kHotBins];
#pragma unroll
    for (uint32_t b = 0; b < kHotBins; ++b) hot[b] = 0;

    // Lists the tail keys among k[0, count) one key vector at a time: one reservation for
    // the wave, each key placed by its rank among the wave's tail lanes of that vector.
    // Used when some thread holds more than four tail keys in one iteration.
    auto list_tail_per_key = [&](const uint32_t *k, uint32_t count) {
        uint32_t total = 0;
        for (uint32_t j = 0; j < count; ++j) AddPopcount(total, __ballot(k[j] - kLdsBins < tail_range));
        uint32_t slot = 0;
        if (lane == 0) slot = __hip_atomic_fetch_add(&sh.tail_count, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        slot = __builtin_amdgcn_readfirstlane(slot);
        for (uint32_t j = 0; j < count; ++j) {
            const bool is_tail = k[j] - kLdsBins < tail_range;
            const uint64_t m = __ballot(is_tail);
            if (is_tail) {
                const uint32_t at = slot + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                           __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                if (at < kTailCap) sh.tail[at] = (uint16_t)k[j];
            }
            AddPopcount(slot, m);
        }
    };

    // Counts kUnitsNow * 4 keys per thread.
    auto process = [&](const i32x4 *v, auto units_tag) {
        constexpr uint32_t kN = decltype(units_tag)::value * 4;
        uint32_t k[kN];
#pragma unroll
        for (uint32_t u = 0; u < kN / 4; ++u) {
            k[u * 4 + 0] = (uint32_t)v[u].x; k[u * 4 + 1] = (uint32_t)v[u].y;
            k[u * 4 + 2] = (uint32_t)v[u].z; k[u * 4 + 3] = (uint32_t)v[u].w;
        }
#pragma unroll
        for (uint32_t j = 0; j < kN; ++j) {
#pragma unroll
            for (uint32_t b = 0; b < kHotBins; ++b) AddPopcount(hot[b], __ballot(k[j] == b));
            if (k[j] - kHotBins < main_range) LdsAdd(&sh.bins[k[j]], 1u);
        }
        if (tail_range != 0) {
            // Tail keys are rare for skewed inputs, and VALU issue is what bounds this loop:
            // each thread first gathers its own tail keys (up to four 16-bit values in two
            // registers, newest in the low half of `lo`), then the wave places them with at
            // most four list writes per iteration instead of one per key.
            uint32_t cnt = 0, lo = 0, hi = 0;
#pragma unroll
            for (uint32_t j = 0; j < kN; ++j) {
                if (k[j] - kLdsBins < tail_range) {
                    // asm so that the body stays under the branch (three instructions that
                    // run only for key vectors with a tail lane) instead of becoming selects
                    asm volatile("v_alignbit_b32 %0, %0, %1, 16\n\t"
                                 "v_lshl_or_b32 %1, %1, 16, %3\n\t"
                                 "v_add_u32 %2, 1, %2"
                                 : "+v"(hi), "+v"(lo), "+v"(cnt) : "v"(k[j]));
                }
            }
            if (kN > 4 && __ballot(cnt > 4) != 0) {
                list_tail_per_key(k, kN);
            } else {
                const uint64_t l1 = __ballot(cnt >= 1);
                if (l1 != 0) {
                    const uint64_t l2 = __ballot(cnt >= 2), l3 = __ballot(cnt >= 3), l4 = __ballot(cnt >= 4);
                    const uint32_t n1 = (uint32_t)__popcll(l1), n2 = (uint32_t)__popcll(l2);
                    const uint32_t n3 = (uint32_t)__popcll(l3), n4 = (uint32_t)__popcll(l4);
                    const uint32_t total = n1 + n2 + n3 + n4;
                    uint32_t slot = 0;
                    if (lane == 0) slot = __hip_atomic_fetch_add(&sh.tail_count, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    slot = __builtin_amdgcn_readfirstlane(slot);
                    if (slot + total <= kTailCap) {
                        auto rank = [](uint64_t m) {
                            return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                        };
                        if (cnt >= 1) sh.tail[slot + rank(l1)] = (uint16_t)lo;
                        if (cnt >= 2) sh.tail[slot + n1 + rank(l2)] = (uint16_t)(lo >> 16);
                        if (l3 != 0) {
                            if (cnt >= 3) sh.tail[slot + n1 + n2 + rank(l3)] = (uint16_t)hi;
                            if (cnt >= 4) sh.tail[slot + n1 + n2 + n3 + rank(l4)] = (uint16_t)(hi >> 16);
                        }
                    }
                    // else: tail_count has passed the capacity, the write-out re-reads the chunk
                }
            }
        }
    };
    using Units = std::integral_constant<uint32_t, kUnits>;
    using OneUnit = std::integral_constant<uint32_t, 1>;

    auto load_iter = [&](i32x4 *v, uint64_t base) {
#pragma unroll
        for (uint32_t u = 0; u < kUnits; ++u) {
            v[u] = __builtin_nontemporal_load((const i32x4 *)(keys + base + ((uint64_t)u * kThreads + tid) * 4));
        }
    };

    // Full iterations: plain 128-bit loads, two register sets so that the next
    // iteration's keys are in flight while this one's are counted.
    uint64_t base = begin;
    bool quit = false;
    if (vec_ok) {
        const uint64_t full_end = begin + (end - begin) / kIterKeys * kIterKeys;
        i32x4 a[kUnits], b[kUnits];
        if (base < full_end) load_iter(a, base);
        while (base < full_end) {
            const bool has_b = base + kIterKeys < full_end;
            if (has_b) load_iter(b, base + kIterKeys);
            process(a, Units {});
            base += kIterKeys;
            if (!has_b) break;
            const bool has_a = base + kIterKeys < full_end;
            if (has_a) load_iter(a, base + kIterKeys);
            process(b, Units {});
            base += kIterKeys;
            if (kGuard && !guard.WaveStillCurrent()) {
                if (lane == 0) sh.bailed = 1;
                quit = true;
                break;
            }
        }
    }
    // Ragged remainder (and unaligned key arrays): one unit at a time, absent keys read
    // as the sentinel.
    for (; !quit && base < end; base += kUnitKeys) {
        const uint64_t idx = base + (uint64_t)tid * 4;
        i32x4 v = { -1, -1, -1, -1 };
        if (vec_ok && idx + 3 < end) {
            v = __builtin_nontemporal_load((const i32x4 *)(keys + idx));
        } else {
            if (idx + 0 < end) v.x = keys[idx + 0];
            if (idx + 1 < end) v.y = keys[idx + 1];
            if (idx + 2 < end) v.z = keys[idx + 2];
            if (idx + 3 < end) v.w = keys[idx + 3];
        }
        process(&v, OneUnit {});
    }

    // Ballot counters are per wave: lane 0 of each wave folds them into the LDS counters.
    if (lane == 0) {
#pragma unroll
        for (uint32_t b = 0; b < kHotBins; ++b) {
            if (hot[b] != 0 && b < lds_used) LdsAdd(&sh.bins[b], hot[b]);
        }
    }
    __syncthreads();

    if (kGuard) {
        // Last point without side effects: all waves agree on writing out or abandoning.
        if (tid == 0) sh.guard_word = (sh.bailed == 0 && guard.WaveStillCurrent()) ? 1u : 0u;
        __syncthreads();
        if (sh.guard_word == 0) return;
    }

    const uint32_t rot = (blockIdx.x * 37u) & (kSegs - 1);
    SweepOut(sh, bins, lds_used, rot);

    if (tail_range != 0) {
        const uint32_t listed = sh.tail_count;
        __syncthreads();
        ClearBins(sh);
        __syncthreads();
        if (listed <= kTailCap) {
            for (uint32_t i = tid; i < listed; i += kThreads) LdsAdd(&sh.bins[sh.tail[i] - kLdsBins], 1u);
        } else {
            // The list overflowed: count the chunk's tail keys from memory instead.
            for (uint64_t idx = begin + tid; idx < end; idx += kThreads) {
                const uint32_t key = (uint32_t)keys[idx];
                if (key - kLdsBins < tail_range) LdsAdd(&sh.bins[key - kLdsBins], 1u);
            }
        }
        __syncthreads();
        SweepOut(sh, bins + kLdsBins, tail_range, rot);
    }

    if (kGuard) guard.Commit();
}

class HipHistogramCommand final : public HipGuardedCommand
{
public:
    HipHistogramCommand(const void *keys, size_t n, void *bins, uint32_t n_bins, uint32_t chunk,
                        uint32_t n_wg, int guard_mode)
        : HipGuardedCommand(n_wg, guard_mode)
        , keys_((const int32_t *)keys), n_(n), bins_((uint32_t *)bins), n_bins_(n_bins), chunk_(chunk) {}

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        if (n_ == 0) return hipSuccess;
        const dim3 grid(n_wg_), block(kThreads);
        if (guarded) hipLaunchKernelGGL(HistogramKernel<true>, grid, block, 0, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, g);
        else         hipLaunchKernelGGL(HistogramKernel<false>, grid, block, 0, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, g);
        return hipGetLastError();
    }

private:
    const int32_t *keys_;
    const size_t n_;
    uint32_t *bins_;
    const uint32_t n_bins_;
    const uint32_t chunk_;
};

} // namespace hist

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipHistogramCommandCreate(HwCommandHandle *cmd, const void *keys, size_t n,
                                                void *bins, uint32_t n_bins, int guard)
{
    if (cmd == nullptr || bins == nullptr || (n != 0 && keys == nullptr) || guard < 0 || guard > 3) {
        return kXSchedErrorInvalidValue;
    }
    if (n_bins == 0 || n_bins > 65536) return kXSchedErrorInvalidValue;
    const uint32_t chunk = hist::ChunkFor(n);
    const uint64_t n_wg = n == 0 ? 1 : (n + chunk - 1) / chunk;
    if (n_wg > GuardState::kMaxWorkGroups) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<hist::HipHistogramCommand>(
        keys, n, bins, n_bins, chunk, (uint32_t)n_wg, guard));
    return kXSchedSuccess;
}
