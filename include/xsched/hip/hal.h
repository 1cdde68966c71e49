/* MI355X HIP hardware-queue adapter: C entry points.
 *
 * HipQueueCreate() is the adapter constructor XSched applications and the HIP
 * interception shim already call (reference
 * platforms/hip/hal/include/xsched/hip/hal/hal.h:11, implemented there in
 * platforms/hip/hal/src/hip_queue.cpp:56-71). The queue it returns supports
 * preemption levels 1 (block) AND 2 (deactivate / reactivate) and switches
 * between them at run time; the reference adapter is level 1 only
 * (hip_queue.h:25-26).
 *
 * The Hip*CommandCreate() functions build HwCommands for XQueueSubmit(). In
 * XSched the same objects are C++ classes constructed by the shim (reference
 * platforms/hip/hal/include/xsched/hip/hal/hip_command.h:22-254); here they are
 * reachable from C so that any language can submit work without the shim.
 *
 * All pointers are device pointers unless said otherwise. Streams are passed as
 * void* (a hipStream_t). Nothing here takes ownership of user buffers: they must
 * stay valid until the command has completed.
 */
#ifndef XSCHED_HIP_HAL_H_
#define XSCHED_HIP_HAL_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Register `stream` as a hardware queue. The handle equals the stream pointer
 * (reference handle.h:9-12). The default (null) stream is refused with
 * NotSupported, as in the reference (hip_queue.cpp:62-65). */
XResult HipQueueCreate(HwQueueHandle *hwq, void *stream);

/* Counters of one queue, for tests and benches. `out` receives 8 values:
 * [0] launches, [1] replayed launches, [2] deactivations, [3] reactivations,
 * [4] marker waits that returned while polling, [5] marker waits that had to
 * block in the driver, [6] progress-map slots in use, [7] current preempt epoch. */
XResult HipQueueGetStats(HwQueueHandle hwq, uint64_t *out);

/* How the queue's kernel commands carry their completion markers. on != 0 (the default,
 * XSCHED_HIP_MARKER_ON_KERNEL=OFF changes it): as the stop event of the kernel's own launch,
 * which saves the device a packet per marked command (1-3 us) and a waiting caller 2 us.
 * The HIP runtime then learns of the kernel's completion some 20 us after XQueueWait /
 * XQueueWaitAll have returned: hipStreamQuery() on the raw stream says "not ready" and
 * hipStreamSynchronize() blocks for that long. on == 0: every marker is a hipEventRecord()
 * behind its command, and the stream is idle for the runtime as soon as the XQueue is.
 * For programs that wait on the raw stream themselves (the interception shim does this for
 * its queues). Takes effect for commands launched afterwards. No counterpart in the
 * reference, whose HIP adapter records an event behind every marked command
 * (platforms/hip/hal/src/hip_command.cpp:38-44). */
XResult HipQueueSetMarkerOnKernel(HwQueueHandle hwq, int on);

/* Device memory the queue's pools hold for guarded commands, for tests. `out` receives 4
 * values: [0] scratch buffers allocated (the partial histograms of histogram commands),
 * [1] their bytes, [2] progress-map slots allocated, [3] progress-map slots in use. Both
 * pools grow with what is launched and not yet destroyed, not with what waits in the XQueue.
 * No counterpart in the reference (its HIP adapter has no level 2). */
XResult HipQueueGetPoolStats(HwQueueHandle hwq, uint64_t *out);

/* For tests of the guard protocol: stores the queue's current preempt epoch into its
 * "flushed" word, as a work-group does that leaves because a deactivation reached it.
 * Guarded launches of that epoch then do nothing (they wait for a replay, which only a
 * deactivation / reactivation of the queue brings). No counterpart in the reference. */
XResult HipQueueMarkEpochFlushed(HwQueueHandle hwq);

/* ---- guarded victim kernels: flushable at level 2 ---------------------------
 * `guard`: 0 = plain kernel (never flushable, property None),
 *          1 = guarded kernel, property Deactivatable: at level 2 it carries the
 *              work-group entry guard and a progress map; at level 1 the same
 *              command launches the plain variant.
 *          2 = always launch the guarded variant, even at level 1 (for measuring
 *              the cost of the guard).
 *          3 = same as 1 (kept for callers that asked for the AXPY's short-drain grid when
 *              that was not yet its default).
 * A guarded AXPY runs as two long-lived waves per CU that look at the preempt word in front
 * of every chunk: after a deactivation the device drains in microseconds, at the bandwidth
 * of the plain kernel (which uses the same grid from 2^23 elements on). With
 * XSCHED_HIP_AXPY_GRID=chunk every AXPY runs as one short-lived wave per chunk, the guard at
 * its entry: ~180 us of drain. */

/* y[i] = fma(alpha, x[i], y[i]) in place, fp32, i < n. 128-bit loads/stores when
 * x and y are 16-byte aligned. */
XResult HipAxpyCommandCreate(HwCommandHandle *cmd, float alpha, const void *x, void *y,
                             size_t n, int guard);

/* C[M,N] = A[M,K] * B[K,N]; A, B, C row-major bf16, fp32 accumulation in ascending
 * k, round-to-nearest-even on store. Any M, N, K >= 1 (at most 2^18 tiles). The fast MFMA
 * kernel takes M, N in multiples of 128, K in multiples of 64 (K, N <= 2^22) and matrices
 * aligned to 16 bytes: it works on 256x256 tiles of C, or on 128x128 tiles when M or N is no
 * multiple of 256 or the large tiles would cover at most half of the compute units
 * (XSCHED_HIP_GEMM_TILE=128|256 overrides that). Where only M is not as the fast kernel wants
 * it, the fast kernel takes the rows up to the last multiple of 128 and the kernel below the
 * rest, in one command. Every other shape or alignment runs on a
 * bounds-checked kernel with 64x64 tiles (XSCHED_HIP_GEMM_TILE=64 forces it): correct and
 * guarded like the others, 5-20 times slower (180-230 TFLOP/s where rows are 16-byte aligned,
 * 60 where they are not). Every element is summed in the same order
 * in all three. */
XResult HipGemmBf16CommandCreate(HwCommandHandle *cmd, const void *A, const void *B, void *C,
                                 int M, int N, int K, int guard);

/* bins[keys[i]] += 1 for i < n; keys are int32 in [0, n_bins), bins are uint32 and
 * are NOT cleared by the command. n_bins <= 65536. */
XResult HipHistogramCommandCreate(HwCommandHandle *cmd, const void *keys, size_t n, void *bins,
                                  uint32_t n_bins, int guard);

/* The same histogram (bins[keys[i]] += 1, bins not cleared) enqueued on `stream` (a
 * hipStream_t; NULL = the default stream) directly, as two plain kernel launches, by an entry
 * point that allocates nothing: no hipMalloc / hipFree, no pool, no XQueue, no command object.
 * No counterpart in the reference. It is for callers that cannot allocate device memory where
 * they call it: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation. The partial histograms that HipHistogramCommandCreate keeps in a buffer of its
 * queue's pool live in a static device array of 16.25 MiB (256 partials) instead, which every
 * GPU the library has run this call on holds until the process ends. Limits and rules:
 *   - n <= 2^26 keys (InvalidValue and a warning above that); n_bins <= 65536;
 *   - every call on one GPU uses that GPU's one array: calls whose kernels can overlap on a
 *     GPU (different streams, no ordering between them) race; calls on one stream do not;
 *   - nothing of the array has to be zero: each launch overwrites all it reads;
 *   - the launches are not flushable (no guard): level-2 preemption does not apply;
 *   - the address of the array on a GPU is looked up once, when the first hardware queue is
 *     created on that GPU (HipQueueCreate) or else at the first call there: a caller that
 *     captures this call into a graph does one of the two before the capture begins.
 * Returns after enqueueing; the caller synchronises the stream. */
XResult HipHistogramLaunchNoAlloc(void *stream, const void *keys, size_t n, void *bins,
                                  uint32_t n_bins);

/* A kernel of the caller's own that has the guard of xsched/hip/guard.h compiled in (see the
 * head of that file for the three lines). The kernel's LAST parameter must be an XGuardArgs:
 * `args` / `arg_sizes` describe the parameters in front of it (copied at creation), the guard
 * arguments are supplied at every launch. The grid is one-dimensional, `n_workgroups`
 * work-groups (at most 2^18); the kernel identifies its work-group to the guard by
 * blockIdx.x. Property Deactivatable: at level 2 a launch can be flushed and is replayed by
 * the reactivation, every work-group taking effect exactly once; at level 1 the guard lets
 * every work-group through. Takes the place of the instrumentation the reference applies to
 * CUDA kernels (platforms/cuda/hal/src/level2/instrument.cpp:224-231,
 * platforms/cuda/hal/inject/inject.cu:43-83). */
XResult HipGuardedKernelCommandCreate(HwCommandHandle *cmd, const void *host_func,
                                      uint32_t n_workgroups,
                                      uint32_t block_x, uint32_t block_y, uint32_t block_z,
                                      void **args, const size_t *arg_sizes, size_t n_args,
                                      uint32_t shared_mem_bytes);

/* ---- generic commands (level 1 semantics; they are drain points at level 2) -- */

/* hipMemcpyAsync; `kind` is a hipMemcpyKind value. reference hip_command.h:188 */
XResult HipMemcpyCommandCreate(HwCommandHandle *cmd, void *dst, const void *src, size_t bytes,
                               int kind);

/* hipMemsetAsync. reference hip_command.h:189 */
XResult HipMemsetCommandCreate(HwCommandHandle *cmd, void *dst, int value, size_t bytes);

/* hipMemsetD16Async / hipMemsetD32Async: `count` elements of `width_bytes` (2 or 4) bytes,
 * `dst` aligned to the width. reference hip_command.h:190-192 */
XResult HipMemsetWideCommandCreate(HwCommandHandle *cmd, void *dst, uint32_t value, size_t count,
                                   uint32_t width_bytes);

/* hipEventRecord(event) in queue order; property Idempotent, always
 * synchronizable. reference hip_command.h:197-219 */
XResult HipEventRecordCommandCreate(HwCommandHandle *cmd, void *event);

/* hipStreamWaitEvent(event, flags) in queue order. reference hip_command.h:236-254 */
XResult HipEventWaitCommandCreate(HwCommandHandle *cmd, void *event, uint32_t flags);

/* Wait, in queue order, until the event-record command `record_cmd` of ANOTHER XQueue has
 * completed. `record_cmd` must still be owned by the caller (create this command BEFORE
 * submitting the record command; NotFound otherwise) and must come from
 * HipEventRecordCommandCreate (InvalidValue otherwise). The wait happens on the host, on the
 * launch thread of the waiting XQueue, and follows the record command through level-2
 * flushes and replays of its queue. reference hip_command.h:240-241, hip_command.cpp:174-177,
 * shim.cpp:242-244 */
XResult HipRecordedEventWaitCommandCreate(HwCommandHandle *cmd, HwCommandHandle record_cmd);

/* hipLaunchKernel of an arbitrary kernel. `args[i]` points to argument i of
 * `arg_sizes[i]` bytes; the values are copied at creation (the reference gets the
 * sizes from code-object metadata instead: hip_command.cpp:53-73,
 * kernel_param.cpp:256-345). `host_func` is the kernel's host-side symbol. */
XResult HipKernelCommandCreate(HwCommandHandle *cmd, const void *host_func,
                               uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                               uint32_t block_x, uint32_t block_y, uint32_t block_z,
                               void **args, const size_t *arg_sizes, size_t n_args,
                               uint32_t shared_mem_bytes);

/* hipModuleLaunchKernel of `function` (a hipFunction_t). `packed_args` holds every argument
 * at its offset in the kernel argument segment (`bytes` in all) and is copied at creation.
 * reference hip_command.h:124-186 */
XResult HipModuleKernelCommandCreate(HwCommandHandle *cmd, void *function,
                                     uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                                     uint32_t block_x, uint32_t block_y, uint32_t block_z,
                                     uint32_t shared_mem_bytes,
                                     const void *packed_args, size_t bytes);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HIP_HAL_H_ */
