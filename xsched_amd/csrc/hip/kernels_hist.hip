// Guarded integer histogram for gfx950: bins[keys[i]] += 1, keys int32 in
// [0, n_bins), n_bins <= 65536, bins uint32.
//
// The keys are read once (4 bytes per key). Two things used to cost more than that read
// on MI355X: the LDS atomics when many lanes of a wave add to ONE address (the hottest bins of
// a skewed distribution; spread over addresses they are cheap: with 16 waves issuing, a CU
// retires a 64-lane ds_add every 1.7 ns on per-lane words and every 2.2 ns on random words,
// five times what this kernel asks of it) and the merge of the
// per-group counts into the one result array (device-wide atomic adds retire at
// ~90-110 G/s however they are arranged, and 256 groups times 65536 bins is a lot of
// them; hence the second kernel below).
//
// One work-group of 1024 threads per compute unit owns a contiguous chunk of keys
// (sized so that a launch has about one work-group per CU) and keeps everything it
// counts on chip until the end. Keys < kHotBins are counted by wave ballot + popcount
// into scalar registers: for skewed (Zipf-like) keys these few bins take a quarter of
// all keys and would otherwise serialise the LDS atomics of a wave on one address.
// The other keys go to LDS counters, in one of two layouts:
//
// Two kernels (kMerge; the layout in use up to 2^28 keys). The group's 128 KiB of LDS
// counters are split in two. Bins below 256 (two thirds of all Zipf(1.1) keys, a fifth of
// them in bins 0 and 1) have one 32-bit counter PER LANE: 256 bins x 64 lanes, so the lanes of
// a wave never add to the same address for them, no vote and no popcount is needed, and they
// cannot overflow. Every other bin is a BYTE: 16384 words shared by the group, word w counts
// bins w, w + 16384, w + 32768, w + 49152 in its bytes 0..3, one ds_add of
// 1 << 8 * (key >> 14) per key. One vote per iteration tells whether every key of the wave is
// below n_bins, so the add needs no branch. The group then stores a partial histogram of
// 65 KiB (the byte words as they are, the per-lane counters summed) into a scratch buffer,
// and a second kernel sums the partials column by column and adds the totals to the result
// with one 64-bit atomic per pair of bins. A byte overflows only when one bin outside the
// first 256 takes 256 keys of a chunk (0.1 % of it; the hottest such bin of a Zipf(1.1)
// chunk takes 80). Every overflow lowers the sum of all counters by at least 255 and nothing
// raises it, so "sum of counters == keys that must be in them" (all key slots of the chunk
// minus the invalid ones) proves there was none; a group that fails the test stores an
// all-zero partial and recounts its chunk the slow way (32-bit counters, two passes over its
// keys, atomic sweep into the result). The first version of this layout kept 16-bit halves
// for every bin and ballot counters for bins 0 and 1: partials of 128 KiB (32 MiB written
// and read back per 2^26 keys, now 16.25 MiB), 14 vector instructions per key (now 10), and
// LDS adds that serialised on the hot bins.
//
// One kernel (above 2^28 keys, where the partials would need more than 128 MiB of
// scratch, when the scratch buffer cannot be allocated, or on request through
// XSCHED_HIP_HIST_MERGE_MIN_KEYS). The group keeps 32-bit counters for bins < 32768,
// appends the rarer keys above that as 16-bit values to an LDS list (one list
// reservation per wave and iteration), and merges by itself: a sweep of atomic adds
// over its non-zero counters (a wave covers 256 consecutive bins, so the adds arrive
// line by line; each group starts its sweep at a different segment because atomics on
// ONE cache line retire at only ~0.1 G/s); then the same 128 KiB are cleared, the
// listed keys are counted into them and swept out the same way. If the list
// overflows (an adversarial distribution), the group re-reads its chunk for those
// keys instead.
//
// Guard: entry check, and because a group has no side effects before its write-out,
// every wave re-reads the preempt word every 32768 keys of the group and the group abandons
// itself (its progress byte stays untagged, a replay redoes the chunk). The write-out
// runs to completion and commits. The groups of the merge kernel have progress bytes
// of their own behind those of the counting groups, and run only when every counting
// group has committed; the scratch buffer is the command's own from its first launch
// until it is destroyed, so the partials of a flushed launch are still there for the
// replay (a later command of the queue must not write into them: its groups may pass
// their entry check on a copy of the preempt word that has not been rewritten yet while
// this command is already flushed). Integer adds commute, so the result does not depend on the order in which work-groups (or
// replays) run.
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
#define XSCHED_HIST_UNITS 1
#endif
constexpr uint32_t kUnits = XSCHED_HIST_UNITS;  // 128-bit loads per thread and iteration
#ifndef XSCHED_HIST_DEPTH
#define XSCHED_HIST_DEPTH 2
#endif
constexpr uint32_t kDepth = XSCHED_HIST_DEPTH;  // iterations of keys in flight or being counted
#ifndef XSCHED_HIST_POLL_TURNS
#define XSCHED_HIST_POLL_TURNS 2
#endif
constexpr uint32_t kPollTurns = XSCHED_HIST_POLL_TURNS; // turns of the ring per look at the preempt word
constexpr uint32_t kUnitKeys = kThreads * 4;
constexpr uint32_t kIterKeys = kUnitKeys * kUnits;
constexpr uint32_t kMinChunk = kUnitKeys;
constexpr uint32_t kMaxChunk = 1u << 18;
constexpr uint32_t kTargetGroups = 256;       // compute units of an MI355X
constexpr uint32_t kSegBins = 256;            // bins one wave sweeps per step
constexpr uint32_t kSegs = kLdsBins / kSegBins;
// merge layout
constexpr uint32_t kColdWords = 1u << 14;           // byte counters: word w, byte b = bin w + b * 16384
constexpr uint32_t kWarmBins = 256;                 // bins below this have 32-bit counters of their own
constexpr uint32_t kCountWords = kColdWords + kWarmBins * 64;   // LDS words in use: byte words, then a counter per warm bin and lane
static_assert(kCountWords <= kLdsBins, "the merge layout's counters fit the group's LDS array");
// The partial histograms of a launch in memory, n_part of them (one per counting group): the
// byte words column by column, one column per merge group, and within a column partial by
// partial: column c of partial p is the 64 words (256 bytes, two whole cache lines) at
// ((c * n_part) + p) * 64. A merge group therefore reads ONE contiguous run of n_part * 256
// bytes, and a counting group stores its partial as 256 pieces of two lines each. (Partial by
// partial, column by column inside, a merge group read 272 bytes out of every 68 KiB: three
// lines touched for two and a bit used, 1.41 times its bytes in traffic.) Behind the byte
// words: the counts of bins 0..255, which are kept outside the bytes, partial by partial
// (1 KiB each).
constexpr uint32_t kMergeGroups = 256;
constexpr uint32_t kMergeThreads = 256;             // threads of a merge group
constexpr uint32_t kMergeWords = kColdWords / kMergeGroups;          // byte words per column (64)
constexpr uint32_t kPartialWords = kColdWords + kWarmBins;           // 65 KiB of scratch per counting group

/// Where column `column` of partial `p` lies, and where that partial's 256 outside counts do.
__host__ __device__ inline size_t ColumnAt(uint32_t column, uint32_t p, uint32_t n_part)
{
    return ((size_t)column * n_part + p) * kMergeWords;
}
__host__ __device__ inline size_t OutsideAt(uint32_t p, uint32_t n_part)
{
    return (size_t)n_part * kColdWords + (size_t)p * kWarmBins;
}
constexpr uint32_t kMaxPartials = 1024;
static_assert(kWarmBins == kMergeGroups && kHotBins <= kWarmBins, "column j carries the outside count of bin j");
constexpr uint64_t kMergeMinKeys = 1;             // the two-kernel layout wins at every size measured
constexpr uint32_t kMergeMinChunk = 16384;        // fewer, fuller partials for small inputs

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

/// Keys per work-group for a histogram of n keys: a multiple of kMinChunk, at least
/// `floor` (rounded up to one).
inline uint32_t ChunkFor(uint64_t n, uint64_t floor = kMinChunk)
{
    uint64_t c = (n + kTargetGroups - 1) / kTargetGroups;
    if (c < floor) c = floor;
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
    uint32_t invalid;       // merge layout: keys outside [0, n_bins), absent ones included
    uint32_t sum;           // merge layout: sum of all packed counters
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

__device__ __forceinline__ void ClearBins(Shared &sh, uint32_t words = kLdsBins)
{
    for (uint32_t i = threadIdx.x * 4; i < words; i += kThreads * 4) *(u32x4 *)&sh.bins[i] = u32x4 { 0, 0, 0, 0 };
}

/// Merge layout: where a valid key is counted, and by how much. Bins below kWarmBins (two
/// thirds of all Zipf(1.1) keys) have one 32-bit counter PER LANE, so the lanes of a wave never
/// add to the same address for them; every other bin is a byte of a word shared by the group.
__device__ __forceinline__ void PackedSlot(uint32_t key, uint32_t lane, uint32_t &word, uint32_t &inc)
{
    const bool warm = key < kWarmBins;
    word = warm ? kColdWords + key * 64 + lane : key & (kColdWords - 1);
    inc = warm ? 1u : 1u << ((key >> 11) & 24u);
}

/// Sum of the four byte counters of each of four packed words.
__device__ __forceinline__ uint32_t ByteSum(const u32x4 &w)
{
    const uint32_t even = (w.x & 0x00FF00FFu) + (w.y & 0x00FF00FFu) + (w.z & 0x00FF00FFu) + (w.w & 0x00FF00FFu);
    const uint32_t odd = ((w.x >> 8) & 0x00FF00FFu) + ((w.y >> 8) & 0x00FF00FFu) + ((w.z >> 8) & 0x00FF00FFu) +
                         ((w.w >> 8) & 0x00FF00FFu);
    return (even & 0xFFFFu) + (even >> 16) + (odd & 0xFFFFu) + (odd >> 16);
}

/// kMerge: the group stores a packed partial histogram at partials + blockIdx.x *
/// kPartialWords instead of adding its counts to bins itself (HistogramMergeKernel does).
template <bool kGuard, bool kMerge>
__global__ __launch_bounds__(kThreads)
void HistogramKernel(const int32_t *__restrict__ keys, uint64_t n, uint32_t *__restrict__ bins,
                     uint32_t n_bins, uint32_t chunk, uint32_t *__restrict__ partials, XGuardArgs g)
{
    __shared__ __attribute__((aligned(16))) Shared sh;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t lds_used = n_bins < kLdsBins ? n_bins : kLdsBins;
    // unsigned "k - lo < range" tests: one subtract and one compare per tier, and the
    // sentinel 0xFFFFFFFF of an absent key fails all of them
    const uint32_t main_range = kMerge ? (n_bins > kHotBins ? n_bins - kHotBins : 0)
                                       : (lds_used > kHotBins ? lds_used - kHotBins : 0);
    const uint32_t tail_range = !kMerge && n_bins > kLdsBins ? n_bins - kLdsBins : 0;
    XGuardBlock guard(g, blockIdx.x, &sh.guard_word);

    ClearBins(sh, kMerge ? kCountWords : kLdsBins);   // the same number today; the layouts differ
    if (tid == 0) { sh.tail_count = 0; sh.bailed = 0; sh.invalid = 0; sh.sum = 0; }

    const uint64_t begin = (uint64_t)blockIdx.x * chunk;
    const uint64_t end = begin + chunk < n ? begin + chunk : n;
    const bool vec_ok = (((uintptr_t)keys) & 15) == 0; // chunk starts are multiples of 4 keys
    const uint64_t full_end = vec_ok ? begin + (end - begin) / kIterKeys * kIterKeys : begin;

    auto load_iter = [&](i32x4 *v, uint64_t base) {
#pragma unroll
        for (uint32_t u = 0; u < kUnits; ++u) {
            v[u] = __builtin_nontemporal_load((const i32x4 *)(keys + base + ((uint64_t)u * kThreads + tid) * 4));
            if (u + 1 < kUnits) asm volatile("" ::: "memory");
        }
    };
    // A ring of kDepth register sets: the set just counted is refilled with the keys of
    // kDepth iterations ahead. The first sets are requested before the guard's uncached
    // read of the preempt word, so that the memory round trips overlap (reading keys has
    // no side effect).
    constexpr uint64_t kTurnKeys = (uint64_t)kDepth * kIterKeys;
    constexpr uint64_t kLoopKeys = kTurnKeys * kPollTurns; // one trip of the main loop
    const uint64_t turns_end = begin + (full_end - begin) / kLoopKeys * kLoopKeys;
    i32x4 ring[kDepth][kUnits];
    if (begin < turns_end) {
        // Every set is loaded, no branch per set, and in the order in which the loop
        // refills them (the empty statements keep the scheduler from permuting the loads:
        // the loop's waits count on that order). A chunk shorter than one trip of the loop
        // does not use it at all, so that these registers are written on this path only.
#pragma unroll
        for (uint32_t d = 0; d < kDepth; ++d) {
            load_iter(ring[d], begin + (uint64_t)d * kIterKeys);
            asm volatile("" ::: "memory");
        }
    }

    if (kGuard) {
        if (!guard.Enter()) return; // Enter() contains the barrier that also publishes the cleared counters
    } else {
        __syncthreads();
    }

    uint32_t hot[kHotBins];
#pragma unroll
    for (uint32_t b = 0; b < kHotBins; ++b) hot[b] = 0;
    uint32_t invalid = 0; // merge layout: keys of this thread outside [0, n_bins), absent ones included

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
        if (kMerge) {
            // Are all keys of the wave below n_bins (the usual case)? One max per key and one
            // vote per iteration decide it; then nothing has to be tallied per key and the
            // LDS add needs no branch.
            uint32_t largest = k[0];
#pragma unroll
            for (uint32_t j = 1; j < kN; ++j) largest = largest > k[j] ? largest : k[j];
            if (__ballot(largest >= n_bins) == 0) {
#pragma unroll
                for (uint32_t j = 0; j < kN; ++j) {
                    uint32_t word, inc;
                    PackedSlot(k[j], lane, word, inc);
                    LdsAdd(&sh.bins[word], inc);
                }
            } else {
#pragma unroll
                for (uint32_t j = 0; j < kN; ++j) {
                    if (k[j] >= n_bins) {
                        invalid += 1;
                    } else {
                        uint32_t word, inc;
                        PackedSlot(k[j], lane, word, inc);
                        LdsAdd(&sh.bins[word], inc);
                    }
                }
            }
        } else {
#pragma unroll
            for (uint32_t j = 0; j < kN; ++j) {
#pragma unroll
                for (uint32_t b = 0; b < kHotBins; ++b) AddPopcount(hot[b], __ballot(k[j] == b));
                if (k[j] - kHotBins < main_range) LdsAdd(&sh.bins[k[j]], 1u);
            }
        }
        if (!kMerge && tail_range != 0) {
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

    // Counts the chunk; false when the wave saw a deactivation and gave up.
    //
    // Full iterations go through the ring. Whole turns of it run without a branch around
    // their loads (a refill that would start beyond the last full iteration re-reads that
    // one instead, unused), so the compiler can count exactly how many loads may still be
    // in flight where it needs one of them. The preempt word is requested at the start of
    // a trip of the loop (kPollTurns turns) and looked at at its end: by then the refills
    // issued behind it are the only loads it does not wait for.
    auto count_chunk = [&]() -> bool {
        uint64_t base = begin;
        if (base < turns_end) {
            do {
                const uint32_t polled = kGuard ? guard.WavePollBegin() : 0u;
#pragma unroll
                for (uint32_t t = 0; t < kPollTurns; ++t) {
#pragma unroll
                    for (uint32_t d = 0; d < kDepth; ++d) {
                        process(ring[d], Units {});
                        const uint64_t next = base + (uint64_t)d * kIterKeys + kTurnKeys;
                        load_iter(ring[d], next < full_end ? next : full_end - kIterKeys);
                    }
                    base += kTurnKeys;
                }
                if (kGuard && !guard.WavePollEnd(polled)) return false;
            } while (base < turns_end);
            // fewer than kDepth full iterations are left, and their keys are in the ring already
#pragma unroll
            for (uint32_t d = 0; d < kDepth; ++d) {
                if (base < full_end) {
                    process(ring[d], Units {});
                    base += kIterKeys;
                }
            }
        }
        // what a chunk has beyond whole trips of the loop and the ring: one iteration at a time
        for (; base < full_end; base += kIterKeys) {
            i32x4 v[kUnits];
            load_iter(v, base);
            process(v, Units {});
        }
        // Ragged remainder (and unaligned key arrays): one unit at a time, absent keys read
        // as the sentinel.
        for (; base < end; base += kUnitKeys) {
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
        return true;
    };
    if (!count_chunk() && lane == 0) sh.bailed = 1;

    // Ballot counters are per wave: lane 0 of each wave folds them into the group's.
    if (!kMerge && lane == 0) {
#pragma unroll
        for (uint32_t b = 0; b < kHotBins; ++b) {
            if (hot[b] != 0 && b < lds_used) LdsAdd(&sh.bins[b], hot[b]);
        }
    }
    if (kMerge && invalid != 0) LdsAdd(&sh.invalid, invalid);
    __syncthreads();

    if (kGuard) {
        // Last point without side effects: the group abandons if any of its waves saw a
        // deactivation (the barrier above published their verdicts). The preempt word is
        // not read again here: that round trip would sit exposed in front of every
        // write-out, and a group that writes out just after a deactivation is no different
        // from one that was a little further along.
        if (sh.bailed != 0) return;
    }

    const uint32_t rot = (blockIdx.x * 37u) & (kSegs - 1);
    if (kMerge) {
        const uint32_t me = blockIdx.x, n_part = gridDim.x;
        uint32_t *const outside = partials + OutsideAt(me, n_part);
        uint32_t counted = 0;
        // Every group starts at a column of its own: column c of all partials is one run of
        // n_part * 256 bytes, and groups that all wrote column 0 first, then column 1, would
        // all be storing into the same few DRAM pages at any moment.
        const uint32_t turn = ((me * 37u) & (kMergeGroups - 1)) * kMergeWords;
        for (uint32_t k = tid * 4; k < kColdWords; k += kThreads * 4) {
            const uint32_t i = (k + turn) & (kColdWords - 1);
            const u32x4 w = *(const u32x4 *)&sh.bins[i];
            // (a plain store: non-temporal ones make the command 1.5 us slower, the counting
            // kernel and the merge kernel's reads both)
            *(u32x4 *)&partials[ColumnAt(i / kMergeWords, me, n_part) + i % kMergeWords] = w;
            counted += ByteSum(w);
        }
        {
            // the 64 per-lane counters of warm bin tid / 4: four threads sum 16 each
            const uint32_t *mine = &sh.bins[kColdWords + (tid / 4) * 64 + (tid % 4) * 16];
            uint32_t warm = 0;
#pragma unroll
            for (uint32_t q = 0; q < 4; ++q) {
                const u32x4 w = *(const u32x4 *)&mine[q * 4];
                warm += w.x + w.y + w.z + w.w;
            }
            counted += warm;
            warm += __shfl_xor(warm, 1);
            warm += __shfl_xor(warm, 2);
            if (tid % 4 == 0) outside[tid / 4] = warm;
        }
        LdsAdd(&sh.sum, counted);
        __syncthreads();
        // every key slot the group went through (absent keys of the ragged end included) is
        // an invalid key or in the counters
        const uint32_t expected = (uint32_t)(full_end - begin)
                                + (uint32_t)((end - full_end + kUnitKeys - 1) / kUnitKeys) * kUnitKeys - sh.invalid;
        if (__builtin_amdgcn_readfirstlane(sh.sum) != __builtin_amdgcn_readfirstlane(expected)) {
            // A byte counter overflowed: this group's partial counts nothing, and the chunk
            // is counted again with 32-bit counters, one half of the bins at a time.
            __syncthreads();
            for (uint32_t i = tid * 4; i < kColdWords; i += kThreads * 4) {
                *(u32x4 *)&partials[ColumnAt(i / kMergeWords, me, n_part) + i % kMergeWords] = u32x4 { 0, 0, 0, 0 };
            }
            if (tid < kWarmBins) outside[tid] = 0;
            for (uint32_t first = 0; first < n_bins; first += kLdsBins) {
                const uint32_t count = n_bins - first < kLdsBins ? n_bins - first : kLdsBins;
                ClearBins(sh);
                __syncthreads();
                for (uint64_t idx = begin + tid; idx < end; idx += kThreads) {
                    const uint32_t key = (uint32_t)keys[idx];
                    if (key - first < count) LdsAdd(&sh.bins[key - first], 1u);
                }
                __syncthreads();
                SweepOut(sh, bins + first, count, rot);
                __syncthreads();
            }
        }
    } else {
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
    }

    if (kGuard) guard.Commit();
}

/// Sums the partial histograms of the counting groups and adds the totals to bins. Group j
/// owns column j of every partial: 64 words of byte counters (word w, byte b = bin
/// w + b * 16384) and the count of bin j, which is kept outside the bytes. Thread (row, col)
/// reads four byte words of its column from partials row, row + 16, ... (the sixteen threads
/// of a row one partial's 256 bytes, the four rows of a wave four neighbouring partials: one
/// KiB in a piece); the threads of col 0 also read the outside count. The group's progress
/// byte is first_wg + j. Four waves per group: the kernel is one round trip to its partials,
/// a reduction through 16 KiB of LDS and 256 atomics.
template <bool kGuard>
__global__ __launch_bounds__(kMergeThreads)
void HistogramMergeKernel(const uint32_t *__restrict__ partials, uint32_t n_part, uint32_t *__restrict__ bins,
                          uint32_t n_bins, uint32_t first_wg, XGuardArgs g)
{
    constexpr uint32_t kCols = kMergeWords / 4, kRows = kMergeThreads / kCols; // 16 x 16
    constexpr uint32_t kAhead = 16;                                      // rows requested before the guard's reads
    __shared__ uint32_t red[kRows][16][kCols];   // per row: the 16 byte counters of each of the 16 word quads
    __shared__ uint32_t total[16][kCols];
    __shared__ uint32_t outside_total;
    __shared__ uint32_t guard_word;

    const uint32_t tid = threadIdx.x;
    const uint32_t col = tid % kCols, row = tid / kCols;
    const uint32_t column = blockIdx.x;
    auto load_words = [&](uint32_t p) {
        return p < n_part ? *(const u32x4 *)(partials + ColumnAt(column, p, n_part) + col * 4) : u32x4 { 0, 0, 0, 0 };
    };
    auto load_outside = [&](uint32_t p) {
        return col == 0 && p < n_part ? partials[OutsideAt(p, n_part) + column] : 0u;
    };
    // even[i] holds bytes 0 and 2 of word i in its halves, odd[i] bytes 1 and 3; a thread adds
    // at most kMaxPartials / kRows = 64 values of 255 into a half.
    uint32_t even[4] = { 0, 0, 0, 0 }, odd[4] = { 0, 0, 0, 0 }, outside = 0;
    auto add_words = [&](const u32x4 &w) {
        const uint32_t v[4] = { w.x, w.y, w.z, w.w };
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) { even[i] += v[i] & 0x00FF00FFu; odd[i] += (v[i] >> 8) & 0x00FF00FFu; }
    };
    // The first rows are requested before the guard's reads: the kernel is short, and the
    // round trips overlap. Reading has no side effect (after a flushed counting launch the
    // words are stale, and nothing is done with them).
    u32x4 first[kAhead];
    uint32_t first_outside[kAhead];
#pragma unroll
    for (uint32_t i = 0; i < kAhead; ++i) {
        first[i] = load_words(row + i * kRows);
        first_outside[i] = load_outside(row + i * kRows);
    }
    if (tid == 0) {
        outside_total = 0;
        // This kernel does not look at the preempt word itself: it runs for a few
        // microseconds, and what it must not do is run after a counting launch that was
        // flushed, whose partials are incomplete. Every counting group that leaves because of
        // a deactivation puts the epoch of its launch into the `flushed` word before it does
        // (and every group that starts later finds the word and leaves the same way): the
        // word differs from this launch's epoch exactly when every counting group has run to
        // its end, now or in an earlier launch. The group's own tag says whether it has added
        // its column already, before a flush that made this launch a replay.
        bool go = true;
        if (kGuard) {
            go = !xguard_epoch_flushed(g);
            if (go && g.resume && g.done && xguard_committed(g, first_wg + blockIdx.x)) go = false;
        }
        guard_word = go ? 1u : 0u;
    }
    __syncthreads();
    if (kGuard && guard_word == 0) return;

#pragma unroll
    for (uint32_t i = 0; i < kAhead; ++i) { add_words(first[i]); outside += first_outside[i]; }
#pragma unroll 4
    for (uint32_t p = row + kAhead * kRows; p < n_part; p += kRows) { add_words(load_words(p)); outside += load_outside(p); }
    // counter b * 4 + i of a thread: byte b of its word i
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        red[row][0 + i][col] = even[i] & 0xFFFFu;
        red[row][4 + i][col] = odd[i] & 0xFFFFu;
        red[row][8 + i][col] = even[i] >> 16;
        red[row][12 + i][col] = odd[i] >> 16;
    }
    if (outside != 0) LdsAdd(&outside_total, outside);
    __syncthreads();
    static_assert(kMergeThreads == 16 * kCols, "one thread per counter of the column");
    {
        const uint32_t v = tid / kCols, c = tid % kCols;
        uint32_t t = 0;
#pragma unroll 16
        for (uint32_t r = 0; r < kRows; ++r) t += red[r][v][c];
        total[v][c] = t;
    }
    __syncthreads();

    // 256 counters: counter (b, i) of quad c is bin column * 64 + c * 4 + i + b * 16384. One
    // 32-bit add each, nothing returned, so no wave waits for the round trip; the 64 lanes of a
    // wave add to 64 neighbouring bins.
    {
        const uint32_t b = tid / 64, c = (tid % 64) / 4, i = tid % 4;
        const uint32_t count = total[b * 4 + i][c];
        const uint32_t bin = column * kMergeWords + c * 4 + i + b * kColdWords;
        if (count != 0 && bin < n_bins) GlobalAdd(bins + bin, count);
    }
    if (tid == 0) {
        // bin <column>, counted outside the bytes (which hold nothing for bins below 256)
        if (outside_total != 0 && column < n_bins) GlobalAdd(bins + column, outside_total);
    }
    if (kGuard) {
        XGuardBlock guard(g, first_wg + blockIdx.x, &guard_word);
        guard.Commit();
    }
}

class HipHistogramCommand final : public HipGuardedCommand
{
public:
    /// n_count_wg counting groups; with `merge`, kMergeGroups merge groups follow them in
    /// the progress map.
    HipHistogramCommand(const void *keys, size_t n, void *bins, uint32_t n_bins, uint32_t chunk,
                        uint32_t n_count_wg, bool merge, int guard_mode)
        : HipGuardedCommand(n_count_wg + (merge ? kMergeGroups : 0), guard_mode)
        , keys_((const int32_t *)keys), n_(n), bins_((uint32_t *)bins), n_bins_(n_bins), chunk_(chunk)
        , n_count_wg_(n_count_wg), merge_(merge) {}
    virtual ~HipHistogramCommand() { if (partials_ != nullptr) pool_->Release(partials_); }

protected:
    size_t ScratchBytes() const { return (size_t)n_count_wg_ * kPartialWords * sizeof(uint32_t); }

    virtual void ReserveOnSubmit(HipQueue &q) override
    {
        if (merge_ && n_ != 0 && partials_ == nullptr) q.Scratch()->Reserve(ScratchBytes());
    }

    virtual hipError_t PrepareLaunch(HipQueue &q) override
    {
        // A replay must find the partials of the flushed launch: the buffer taken at the
        // first launch is kept until the command is destroyed.
        if (!merge_ || n_ == 0 || partials_ != nullptr) return hipSuccess;
        pool_ = q.Scratch();
        partials_ = (uint32_t *)pool_->Acquire(ScratchBytes());
        // No scratch: the one-kernel layout works on the same chunks (decided before the
        // first launch, so every replay takes the same path).
        if (partials_ == nullptr) merge_ = false;
        return hipSuccess;
    }

    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        if (n_ == 0) return hipSuccess;
        const dim3 grid(n_count_wg_), block(kThreads);
        if (!merge_) {
            const hipEvent_t stop = TakeStopEvent();
            if (guarded) LaunchWithStop(stop, (HistogramKernel<true, false>), grid, block, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, (uint32_t *)nullptr, g);
            else         LaunchWithStop(stop, (HistogramKernel<false, false>), grid, block, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, (uint32_t *)nullptr, g);
            return hipGetLastError();
        }
        hipEvent_t stop = nullptr;    // the merge kernel is the command's last
        if (guarded) LaunchWithStop(stop, (HistogramKernel<true, true>), grid, block, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, partials_, g);
        else         LaunchWithStop(stop, (HistogramKernel<false, true>), grid, block, stream, keys_, (uint64_t)n_, bins_, n_bins_, chunk_, partials_, g);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
        const dim3 merge_grid(kMergeGroups), merge_block(kMergeThreads);
        stop = TakeStopEvent();
        if (guarded) LaunchWithStop(stop, HistogramMergeKernel<true>, merge_grid, merge_block, stream, (const uint32_t *)partials_, n_count_wg_, bins_, n_bins_, n_count_wg_, g);
        else         LaunchWithStop(stop, HistogramMergeKernel<false>, merge_grid, merge_block, stream, (const uint32_t *)partials_, n_count_wg_, bins_, n_bins_, n_count_wg_, g);
        return hipGetLastError();
    }

private:
    const int32_t *keys_;
    const size_t n_;
    uint32_t *bins_;
    const uint32_t n_bins_;
    const uint32_t chunk_;
    const uint32_t n_count_wg_;
    bool merge_;
    std::shared_ptr<ScratchPool> pool_;
    uint32_t *partials_ = nullptr;
};

/// Keys from which the two-kernel layout is used (XSCHED_HIP_HIST_MERGE_MIN_KEYS).
inline uint64_t MergeMinKeys()
{
    const char *env = getenv("XSCHED_HIP_HIST_MERGE_MIN_KEYS");
    if (env == nullptr || *env == 0) return kMergeMinKeys;
    return strtoull(env, nullptr, 0);
}

} // namespace hist

} // namespace xsched::hip

using namespace xsched::hip;

// ---- the entry point that allocates nothing -------------------------------------------
//
// The partial histograms of HipHistogramLaunchNoAlloc() live in this array instead of a
// buffer from a queue's pool. Every GPU the library runs on holds its own copy at its own
// address for the life of the process; in host code the array's NAME is only a handle for
// hipGetSymbolAddress(), never a device pointer.
namespace
{
constexpr uint32_t kNoAllocMaxGroups = 256;                       // counting work-groups
constexpr uint64_t kNoAllocMaxKeys = (uint64_t)kNoAllocMaxGroups * hist::kMaxChunk; // 2^26
constexpr size_t kNoAllocScratchWords = (size_t)kNoAllocMaxGroups * hist::kPartialWords;

static __device__ __align__(256) uint32_t scratch[kNoAllocScratchWords];          // 16.25 MiB

constexpr int kNoAllocMaxDevices = 64;
std::mutex g_scratch_mtx;
uint32_t *g_scratch_ptr[kNoAllocMaxDevices] = {};

/// Device address of `scratch` on `device`, which must be the calling thread's current device.
/// Looked up once per device (when a hardware queue is created there, else at the entry
/// point's first call on it); nullptr (and a warning) if the runtime refuses. The first
/// lookup may load the code object, which allocates: it runs with the thread's capture mode
/// relaxed, so a capture under way on ANOTHER stream is not invalidated by it, but it cannot
/// be part of a capture itself: the first call on a device comes before the capture begins.
uint32_t *ScratchOnCurrentDevice(int device)
{
    if (device < 0 || device >= kNoAllocMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mtx);
    if (g_scratch_ptr[device] != nullptr) return g_scratch_ptr[device];
    RelaxedCaptureScope relaxed;
    uint32_t *ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
        XWARN("hipGetSymbolAddress(scratch) on device %d failed: %d (%s)", device, (int)err, hipGetErrorString(err));
        (void)hipGetLastError();
        return nullptr;
    }
    g_scratch_ptr[device] = ptr;
    return ptr;
}
} // namespace

namespace xsched::hip
{
bool ResolveNoAllocScratch(int device) { return ScratchOnCurrentDevice(device) != nullptr; }
} // namespace xsched::hip

EXPORT_C_FUNC XResult HipHistogramLaunchNoAlloc(void *stream_ptr, const void *keys, size_t n, void *bins,
                                                uint32_t n_bins)
{
    if (bins == nullptr || (n != 0 && keys == nullptr)) return kXSchedErrorInvalidValue;
    if (n_bins == 0 || n_bins > 65536) return kXSchedErrorInvalidValue;
    if (n > kNoAllocMaxKeys) {
        XWARN("HipHistogramLaunchNoAlloc: %zu keys exceed the limit of %llu keys that the static "
              "scratch array holds partial histograms for", n, (unsigned long long)kNoAllocMaxKeys);
        return kXSchedErrorInvalidValue;
    }
    if (n == 0) return kXSchedSuccess;

    hipStream_t stream = (hipStream_t)stream_ptr;
    int device = -1, current = -1;
    if (hipGetDevice(&current) != hipSuccess) return kXSchedErrorHardware;
    if (stream == nullptr) device = current;
    else if (hipStreamGetDevice(stream, &device) != hipSuccess) { (void)hipGetLastError(); return kXSchedErrorInvalidValue; }
    if (device < 0 || device >= kNoAllocMaxDevices) return kXSchedErrorNotSupported;
    // Symbol lookup and launch both act on the current device: it has to be the stream's.
    if (device != current && hipSetDevice(device) != hipSuccess) return kXSchedErrorHardware;

    XResult res = kXSchedSuccess;
    uint32_t *partials = ScratchOnCurrentDevice(device);
    if (partials == nullptr) {
        res = kXSchedErrorHardware;
    } else {
        // As few groups as the limit allows, each with a whole number of load units; every
        // group stores its complete partial (all-zero after an overflow recount), so nothing
        // of an earlier call's contents is read and nothing has to be cleared.
        const uint32_t chunk = hist::ChunkFor(n, hist::kMergeMinChunk);   // grows with n: at most 256 groups up to 2^26 keys
        const uint64_t n_wg = (n + chunk - 1) / chunk;
        XASSERT(n_wg <= kNoAllocMaxGroups && chunk <= hist::kMaxChunk, "group count %llu / chunk %u out of range",
                (unsigned long long)n_wg, chunk);
        const XGuardArgs inert {};
        const dim3 block(hist::kThreads);
        hipLaunchKernelGGL((hist::HistogramKernel<false, true>), dim3((uint32_t)n_wg), block, 0, stream,
                           (const int32_t *)keys, (uint64_t)n, (uint32_t *)bins, n_bins, chunk, partials, inert);
        hipError_t err = hipGetLastError();
        if (err == hipSuccess) {
            hipLaunchKernelGGL(hist::HistogramMergeKernel<false>, dim3(hist::kMergeGroups), dim3(hist::kMergeThreads), 0, stream,
                               (const uint32_t *)partials, (uint32_t)n_wg, (uint32_t *)bins, n_bins, (uint32_t)n_wg, inert);
            err = hipGetLastError();
        }
        if (err != hipSuccess) {
            XWARN("HipHistogramLaunchNoAlloc: launch failed: %d (%s)", (int)err, hipGetErrorString(err));
            res = kXSchedErrorHardware;
        }
    }
    if (device != current) (void)hipSetDevice(current);
    return res;
}

EXPORT_C_FUNC XResult HipHistogramCommandCreate(HwCommandHandle *cmd, const void *keys, size_t n,
                                                void *bins, uint32_t n_bins, int guard)
{
    if (cmd == nullptr || bins == nullptr || (n != 0 && keys == nullptr) || guard < 0 || guard > 3) {
        return kXSchedErrorInvalidValue;
    }
    if (n_bins == 0 || n_bins > 65536) return kXSchedErrorInvalidValue;
    bool merge = n != 0 && n >= hist::MergeMinKeys();
    const char *floor_env = getenv("XSCHED_HIP_HIST_MIN_CHUNK");
    const uint64_t floor = floor_env && *floor_env ? strtoull(floor_env, nullptr, 0)
                                                   : (merge ? hist::kMergeMinChunk : hist::kMinChunk);
    uint32_t chunk = hist::ChunkFor(n, floor);
    uint64_t n_wg = n == 0 ? 1 : (n + chunk - 1) / chunk;
    if (merge && n_wg > hist::kMaxPartials) {
        merge = false;
        chunk = hist::ChunkFor(n);
        n_wg = (n + chunk - 1) / chunk;
    }
    if (n_wg > GuardState::kMaxWorkGroups) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<hist::HipHistogramCommand>(
        keys, n, bins, n_bins, chunk, (uint32_t)n_wg, merge, guard));
    return kXSchedSuccess;
}
