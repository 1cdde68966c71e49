/* Host (CPU) hardware-queue adapter: a hardware queue that is an executor thread
 * of this process. It exists so that the whole XQueue stack - in-flight window,
 * markers, suspend/resume, Level-2 flush and replay - runs without a GPU, and it
 * is the backend of the CPU-only configuration (two XQueues streaming fp32
 * vector additions). XSched itself ships no CPU adapter; this one is written to
 * the pattern of its template adapter (reference platforms/example/hal/src/
 * opencl_queue.cpp:7-52, opencl_command.cpp).
 *
 * A host "kernel" is a function called once per work-group index. At preemption
 * level 2 the executor checks the queue's preempt word before each work-group,
 * skips the rest of a flushed kernel and records finished work-groups in a
 * bitmap; Reactivate() replays only the unfinished ones - the same protocol the
 * HIP adapter runs on the device.
 */
#ifndef XSCHED_HOST_HAL_H_
#define XSCHED_HOST_HAL_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Body of a host kernel: process work-group `wg` of `n_wg`. */
typedef void (*HostKernelFn)(void *arg, uint32_t wg, uint32_t n_wg);

/* Create a host hardware queue (starts its executor thread). The handle is
 * process-unique. Destroy with HwQueueDestroy() after its XQueue is gone. */
XResult HostQueueCreate(HwQueueHandle *hwq);

/* A kernel of `n_wg` work-groups. `guarded` != 0 marks it deactivatable (it may be
 * flushed and replayed at level 2); otherwise it always runs to completion.
 * `arg` must stay valid until the command has completed. */
XResult HostKernelCommandCreate(HwCommandHandle *cmd, HostKernelFn fn, void *arg,
                                uint32_t n_wg, int guarded);

/* c[i] = a[i] + b[i] for i < n, fp32, split into work-groups of 16384 elements. */
XResult HostVecAddCommandCreate(HwCommandHandle *cmd, const float *a, const float *b,
                                float *c, size_t n, int guarded);

/* y[i] = fma(alpha, x[i], y[i]) (one rounding per element), in place, work-groups
 * of 16384 elements. */
XResult HostAxpyCommandCreate(HwCommandHandle *cmd, float alpha, const float *x, float *y,
                              size_t n, int guarded);

/* Counters of a host queue, for tests: work-groups executed, work-groups skipped
 * because their kernel was flushed, kernels replayed by Reactivate(). */
XResult HostQueueGetStats(HwQueueHandle hwq, uint64_t *wg_executed, uint64_t *wg_skipped,
                          uint64_t *replays);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HOST_HAL_H_ */
