// Guarded streaming AXPY for gfx950: y = fma(alpha, x, y), fp32, in place.
//
// HBM-bound: 12 bytes of traffic per element (read x, read y, write y). The unit of
// work is a chunk of `steps` x 1024 contiguous elements, walked by one wavefront in
// steps of 4 x 128-bit accesses per lane and stream, lane-contiguous so that every
// access of a wave covers 1 KiB. Loads and stores are non-temporal: nothing is reused.
// Because the update is in place, a chunk must be applied exactly once: the wave reads
// the preempt word before it stores anything, and commits the chunk's byte in the
// progress map after its last store.
//
// Two grids:
//   one single-wave work-group per chunk: plain launches of arrays below 2^23 elements.
//       Every chunk is in flight at once, which is what a short array wants; on long
//       arrays these short-lived waves stream at 6.2-6.3 TB/s on MI355X.
//   two long-lived waves per CU, each walking chunks c, c + G, c + 2G, ... with the loads
//       of three steps in flight: guarded launches, and plain launches of long arrays.
//       Same bandwidth (measured: 2 waves per CU 6.2 TB/s, 1 per CU 4.1, 4 or more per CU
//       5.3-5.8 whatever the depth), and nearly all wave slots stay free: a short kernel of
//       another queue that arrives meanwhile finishes ~10 us earlier than beside a grid of
//       262144 work-groups. A guarded launch reads the preempt word in front of every chunk:
//       after a deactivation every wave stops at its next chunk, about a microsecond away,
//       and a launch queued behind has only G work-groups to retire: the device drains in
//       6 us (p50).
//   XSCHED_HIP_AXPY_GRID=chunk keeps the first grid for everything, with the guard at
//       work-group entry: after a deactivation the device then still has to start and retire
//       every remaining work-group, empty, at ~3.3 waves per nanosecond: two launches of
//       262144 work-groups in flight drain in ~180 us.
#include "hip_hal.h"
#include "xsched/hip/hal.h"
#include "xsched/utils/env.h"

using namespace xsched::preempt;

namespace xsched::hip
{

namespace axpy
{

constexpr uint32_t kLanes = 64;
constexpr uint32_t kStepElems = 1024;                      // unit in which chunk sizes are counted

typedef float float4 __attribute__((ext_vector_type(4))); // 128-bit access unit

__device__ __forceinline__ float4 ld_nt(const float4 *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_nt(float4 *p, float4 v) { __builtin_nontemporal_store(v, p); }

__device__ __forceinline__ float4 fma4(float a, float4 x, float4 y)
{
    float4 r;
    r.x = __builtin_fmaf(a, x.x, y.x);
    r.y = __builtin_fmaf(a, x.y, y.y);
    r.z = __builtin_fmaf(a, x.z, y.z);
    r.w = __builtin_fmaf(a, x.w, y.w);
    return r;
}

// n4: number of whole float4 in the arrays; tail: the 0..3 trailing scalars, done by
// the last work-group.
// kVecPerStep float4 per lane and stream are requested before anything is stored:
// 4 -> steps of 1024 elements, 8 -> steps of 2048 elements.
template <bool kGuard, uint32_t kVecPerStep>
__global__ __launch_bounds__(64)
void AxpyVec4Kernel(float alpha, const float4 *x, float4 *y,
                    uint64_t n4, uint32_t tail, uint32_t steps, XGuardArgs g)
{
    constexpr uint32_t kStepVecs = kLanes * kVecPerStep;
    const uint32_t wg = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint64_t wg_base = (uint64_t)wg * steps * kStepVecs;
    XGuardWave guard(g, wg);

    const bool full = wg_base + (uint64_t)steps * kStepVecs <= n4;
    // The guard comes before the loads: a flushed work-group then costs no memory
    // traffic at all, which keeps the drain after a deactivation short; with 8 waves per
    // SIMD the extra round trip does not show in the bandwidth (measured).
    if (kGuard) {
        if (!guard.Enter()) return;
    }
    if (full) {
        for (uint32_t s = 0; s < steps; ++s) {
            const uint64_t base = wg_base + (uint64_t)s * kStepVecs + lane;
            float4 xv[kVecPerStep], yv[kVecPerStep];
#pragma unroll
            for (uint32_t u = 0; u < kVecPerStep; ++u) {
                xv[u] = ld_nt(&x[base + u * kLanes]);
                yv[u] = ld_nt(&y[base + u * kLanes]);
            }
#pragma unroll
            for (uint32_t u = 0; u < kVecPerStep; ++u) {
                st_nt(&y[base + u * kLanes], fma4(alpha, xv[u], yv[u]));
            }
        }
    } else {
        const uint64_t end = wg_base + (uint64_t)steps * kStepVecs;
        for (uint64_t i = wg_base + lane; i < end && i < n4; i += kLanes) {
            st_nt(&y[i], fma4(alpha, ld_nt(&x[i]), ld_nt(&y[i])));
        }
        if (wg == gridDim.x - 1 && lane < tail) {
            const float *xs = (const float *)(x + n4);
            float *ys = (float *)(y + n4);
            ys[lane] = __builtin_fmaf(alpha, xs[lane], ys[lane]);
        }
    }
    if (kGuard) guard.Commit();
}

// Guarded launches: grid-stride over chunks, see the head of this file. `n_chunks`
// chunks of `steps` x 1024 elements; the progress map has one byte per chunk.
// A wave walks its chunks c, c + G, c + 2G, ... step by step and keeps the loads of
// kDepth steps in flight: step j is stored while steps j+1 .. j+kDepth-1 are on their
// way and step j+kDepth is requested right behind the stores. The preempt word is read
// in front of the first store of every chunk; a chunk that has begun is finished and
// committed, so it is applied exactly once.
template <uint32_t kDepth, bool kGuard>
__global__ __launch_bounds__(64)
void AxpyPersistentKernel(float alpha, const float4 *x, float4 *y, uint64_t n4, uint32_t tail,
                          uint32_t steps, uint32_t n_chunks, XGuardArgs g)
{
    constexpr uint32_t kVecPerStep = 4;
    constexpr uint32_t kStepVecs = kLanes * kVecPerStep;
    const uint32_t lane = threadIdx.x;
    const uint32_t stride = gridDim.x;
    const uint32_t *flag = kGuard ? xguard_flag_copy(g, blockIdx.x) : nullptr;
    // an earlier launch of this epoch was flushed: this one must not run ahead of its replay
    if (kGuard && xguard_epoch_flushed(g)) return;

    // Ring slot d holds step ring_s[d] of chunk ring_c[d]; the slots follow each other in
    // the wave's sequence of steps.
    uint32_t ring_c[kDepth], ring_s[kDepth];
    float4 xv[kDepth][kVecPerStep], yv[kDepth][kVecPerStep];
    {
        uint32_t c = blockIdx.x, st = 0;
#pragma unroll
        for (uint32_t d = 0; d < kDepth; ++d) {
            ring_c[d] = c;
            ring_s[d] = st;
            if (++st == steps) { st = 0; c += stride; }
        }
    }
#pragma unroll
    for (uint32_t d = 0; d < kDepth; ++d) {
        const uint32_t c = ring_c[d];
        if (c < n_chunks && ((uint64_t)c + 1) * steps * kStepVecs <= n4) {
            const uint64_t base = ((uint64_t)c * steps + ring_s[d]) * kStepVecs + lane;
#pragma unroll
            for (uint32_t u = 0; u < kVecPerStep; ++u) {
                xv[d][u] = ld_nt(&x[base + u * kLanes]);
                yv[d][u] = ld_nt(&y[base + u * kLanes]);
            }
        }
    }

    bool skip = false;   // the chunk whose steps are passing by was committed before the flush
    while (true) {
        // no unroll pragma here: the constant trip count is unrolled anyway, and with the
        // pragma the compiler warns about a copy of the loop that it drops afterwards
        for (uint32_t d = 0; d < kDepth; ++d) {
            const uint32_t c = ring_c[d];
            const uint32_t st = ring_s[d];
            if (c >= n_chunks) return;   // the sequence only grows: every later step is beyond, too
            const bool full = ((uint64_t)c + 1) * steps * kStepVecs <= n4;
            if (st == 0) {
                // The scalar read of the preempt word waits for itself only: the vector loads
                // stay in flight across it. A flushed wave drops what it has loaded.
                if (kGuard) {
                    const XGuardVerdict v = xguard_recheck_verdict(xguard_read_flag(flag), g.epoch);
                    if (v.note_flush && lane == 0) xguard_note_flush(g);
                    if (!v.run) return;
                    skip = g.resume && g.done && xguard_committed(g, c);
                }
                if (!skip && !full) {
                    // the last chunk of an array that does not fill it, and the 0..3 scalars behind
                    const uint64_t chunk_base = (uint64_t)c * steps * kStepVecs;
                    const uint64_t end = chunk_base + (uint64_t)steps * kStepVecs;
                    for (uint64_t i = chunk_base + lane; i < end && i < n4; i += kLanes) {
                        st_nt(&y[i], fma4(alpha, ld_nt(&x[i]), ld_nt(&y[i])));
                    }
                    if (c == n_chunks - 1 && lane < tail) {
                        const float *xs = (const float *)(x + n4);
                        float *ys = (float *)(y + n4);
                        ys[lane] = __builtin_fmaf(alpha, xs[lane], ys[lane]);
                    }
                    if (kGuard && g.done && lane == 0) xguard_commit(g, c);
                }
            }
            if (full && !skip) {
                const uint64_t base = ((uint64_t)c * steps + st) * kStepVecs + lane;
#pragma unroll
                for (uint32_t u = 0; u < kVecPerStep; ++u) {
                    st_nt(&y[base + u * kLanes], fma4(alpha, xv[d][u], yv[d][u]));
                }
                if (kGuard && st == steps - 1 && g.done && lane == 0) xguard_commit(g, c);
            }
            // this slot's next step: kDepth steps further on in the sequence
            uint32_t nc = c, ns = st + kDepth;
            while (ns >= steps) { ns -= steps; nc += stride; }
            ring_c[d] = nc;
            ring_s[d] = ns;
            if (nc < n_chunks && ((uint64_t)nc + 1) * steps * kStepVecs <= n4) {
                const uint64_t nb = ((uint64_t)nc * steps + ns) * kStepVecs + lane;
#pragma unroll
                for (uint32_t u = 0; u < kVecPerStep; ++u) {
                    xv[d][u] = ld_nt(&x[nb + u * kLanes]);
                    yv[d][u] = ld_nt(&y[nb + u * kLanes]);
                }
            }
        }
    }
}

// Fallback for pointers that are not 16-byte aligned: same chunking, 32-bit accesses.
template <bool kGuard>
__global__ __launch_bounds__(64)
void AxpyScalarKernel(float alpha, const float *__restrict__ x, float *__restrict__ y,
                      uint64_t n, uint32_t steps, XGuardArgs g)
{
    const uint32_t wg = blockIdx.x;
    XGuardWave guard(g, wg);
    if (kGuard) {
        if (!guard.Enter()) return;
    }
    const uint64_t begin = (uint64_t)wg * steps * kStepElems;
    const uint64_t end = begin + (uint64_t)steps * kStepElems;
    for (uint64_t i = begin + threadIdx.x; i < end && i < n; i += kLanes) {
        y[i] = __builtin_fmaf(alpha, x[i], y[i]);
    }
    if (kGuard) guard.Commit();
}

class HipAxpyCommand final : public HipGuardedCommand
{
public:
    /// steps: chunk size per work-group in units of 1024 elements.
    HipAxpyCommand(float alpha, const float *x, float *y, size_t n, uint32_t steps, uint32_t n_wg,
                   int guard_mode, bool chunk_grid)
        : HipGuardedCommand(n_wg, guard_mode), alpha_(alpha), x_(x), y_(y), n_(n), steps_(steps)
        , chunk_grid_(chunk_grid) {}

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        if (n_ == 0) return hipSuccess;
        const hipEvent_t stop = TakeStopEvent();
        const bool aligned = (((uintptr_t)x_ | (uintptr_t)y_) & 15) == 0;
        const dim3 grid(n_wg_), block(kLanes);
        const uint32_t waves = PersistentWaves();
        if (aligned && guarded && !chunk_grid_) {
            const dim3 pgrid(n_wg_ < waves ? n_wg_ : waves);
            LaunchWithStop(stop, (AxpyPersistentKernel<3, true>), pgrid, block, stream, alpha_, (const float4 *)x_,
                               (float4 *)y_, (uint64_t)(n_ / 4), (uint32_t)(n_ % 4), steps_, n_wg_, g);
        } else if (aligned && !guarded && !chunk_grid_ && n_wg_ >= 16 * waves) {
            // A long array: the same few long-lived waves stream it as fast as one wave per
            // chunk does and leave nearly all wave slots to whatever else runs on the device.
            LaunchWithStop(stop, (AxpyPersistentKernel<3, false>), dim3(waves), block, stream, alpha_, (const float4 *)x_,
                               (float4 *)y_, (uint64_t)(n_ / 4), (uint32_t)(n_ % 4), steps_, n_wg_, g);
        } else if (aligned) {
            const uint64_t n4 = n_ / 4;
            const uint32_t tail = (uint32_t)(n_ % 4);
            // An even chunk is walked in steps of 2048 elements (8 accesses in flight
            // per lane and stream), an odd one in steps of 1024.
            const bool wide = (steps_ % 2) == 0;
            const uint32_t steps = wide ? steps_ / 2 : steps_;
            const float4 *xv = (const float4 *)x_;
            float4 *yv = (float4 *)y_;
            if (guarded && wide)       LaunchWithStop(stop, (AxpyVec4Kernel<true, 8>), grid, block, stream, alpha_, xv, yv, n4, tail, steps, g);
            else if (guarded)          LaunchWithStop(stop, (AxpyVec4Kernel<true, 4>), grid, block, stream, alpha_, xv, yv, n4, tail, steps, g);
            else if (wide)             LaunchWithStop(stop, (AxpyVec4Kernel<false, 8>), grid, block, stream, alpha_, xv, yv, n4, tail, steps, g);
            else                       LaunchWithStop(stop, (AxpyVec4Kernel<false, 4>), grid, block, stream, alpha_, xv, yv, n4, tail, steps, g);
        } else {
            if (guarded) {
                LaunchWithStop(stop, AxpyScalarKernel<true>, grid, block, stream, alpha_, x_, y_,
                                   (uint64_t)n_, steps_, g);
            } else {
                LaunchWithStop(stop, AxpyScalarKernel<false>, grid, block, stream, alpha_, x_, y_,
                                   (uint64_t)n_, steps_, g);
            }
        }
        return hipGetLastError();
    }

private:
    /// Work-groups (= waves) of a guarded launch: a fixed number per compute unit.
    static uint32_t PersistentWaves()
    {
        static const uint32_t waves = []() {
            int64_t per_cu = 2;
            GetEnvInt64("XSCHED_HIP_AXPY_WAVES_PER_CU", per_cu);
            if (per_cu < 1) per_cu = 1;
            if (per_cu > 64) per_cu = 64;
            int dev = 0, cus = 256;
            if (hipGetDevice(&dev) == hipSuccess) {
                (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            }
            return (uint32_t)(per_cu * (cus > 0 ? cus : 256));
        }();
        return waves;
    }

    const float alpha_;
    const float *x_;
    float *y_;
    const size_t n_;
    const uint32_t steps_;
    const bool chunk_grid_;   // guarded launches keep the one-wave-per-chunk grid
};

} // namespace axpy

using namespace axpy;

/// Steps (of 1024 elements) per work-group: small enough that the device drains in
/// tens of microseconds after a flush, large enough that the grid fits the progress
/// map.
uint32_t AxpyStepsFor(size_t n)
{
    int64_t dflt = 1;
    GetEnvInt64("XSCHED_HIP_AXPY_STEPS", dflt);
    uint64_t steps = (uint64_t)(dflt < 1 ? 1 : dflt);
    while (((uint64_t)n + steps * kStepElems - 1) / (steps * kStepElems) > GuardState::kMaxWorkGroups) steps *= 2;
    return (uint32_t)steps;
}

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipAxpyCommandCreate(HwCommandHandle *cmd, float alpha, const void *x, void *y,
                                           size_t n, int guard)
{
    if (cmd == nullptr || (n != 0 && (x == nullptr || y == nullptr)) || guard < 0 || guard > 3) {
        return kXSchedErrorInvalidValue;
    }
    const uint32_t steps = AxpyStepsFor(n);
    const uint64_t per_wg = (uint64_t)steps * 1024;
    const uint32_t n_wg = n == 0 ? 1 : (uint32_t)((n + per_wg - 1) / per_wg);
    *cmd = HwCommandManager::Add(std::make_shared<axpy::HipAxpyCommand>(
        alpha, (const float *)x, (float *)y, n, steps, n_wg, guard, GetEnv("XSCHED_HIP_AXPY_GRID") == "chunk"));
    return kXSchedSuccess;
}
