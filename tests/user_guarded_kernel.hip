// A kernel as a user of the library would write it: its own work plus the three guard lines of
// xsched/hip/guard.h, submitted through HipGuardedKernelCommandCreate. Built into
// xsched_amd/lib/libuserguarded.so for tests/test_gpu_preempt.py.
//
// In place and not idempotent (y = 0.5 * y + b): a work-group that ran twice, or not at all,
// shows in the result, so the test pins "exactly once" through flushes and replays.
#include <hip/hip_runtime.h>

#include "xsched/hip/guard.h"

constexpr int kChunk = 4096; // elements per work-group

__global__ __launch_bounds__(256)
void UserAffine(float *y, float b, size_t n, XGuardArgs g)
{
    __shared__ uint32_t guard_word;
    XGuardBlock guard(g, blockIdx.x, &guard_word);
    if (!guard.Enter()) return;

    const size_t base = (size_t)blockIdx.x * kChunk;
    for (int i = threadIdx.x; i < kChunk; i += 256) {
        const size_t j = base + i;
        if (j < n) y[j] = __builtin_fmaf(0.5f, y[j], b);
    }

    guard.Commit();
}

extern "C" const void *UserAffineKernel() { return (const void *)UserAffine; }
extern "C" int UserAffineChunk() { return kChunk; }
