/* The CPU-only configuration as a harness over the host adapter (C entry points in
 * libhalhost.so): two XQueues at level 1 under the local scheduler with the
 * highest-priority-first policy; the low-priority queue streams fp32 vector additions
 * back to back, the high-priority queue submits a short one every period. Everything goes
 * through the public API (HostQueueCreate, XQueueCreate, XQueueSetLaunchConfig,
 * XHintPriority, HostVecAddCommandCreate, XQueueSubmit, XQueueWaitAll), timed the way the
 * reference's preemption micro-benchmark is laid out: a background thread that launches,
 * a main thread that measures (platforms/cuda/test/main/level.cu:37-86, launch
 * configuration 8 / 4 as at :165). No reference counterpart as a library.
 */
#ifndef XSCHED_HOST_BENCH_H_
#define XSCHED_HOST_BENCH_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* dst[i] = element first + i of the seeded uniform[-1, 1) stream (seed, stream):
 * bits = splitmix64(splitmix64(seed ^ stream * 0xD1B54A32D192ED03) + index),
 * value = (bits >> 40) * 2^-23 - 1. */
void HostBenchFillUniform(float *dst, uint64_t first, uint64_t count, uint64_t seed, uint64_t stream);

typedef struct {
    uint64_t bg_n;          /* elements of a background vector addition               */
    uint64_t fg_n;          /* elements of a foreground vector addition               */
    int32_t  bg_burst;      /* background commands per stream (1000 in the named
                               configuration); streams repeat until the foreground has
                               its samples                                            */
    int32_t  threshold;     /* in-flight window of both queues                        */
    int32_t  batch;         /* marker period of both queues                           */
    int32_t  samples;       /* foreground commands per phase                          */
    int64_t  period_us;     /* one foreground command every period                    */
} HostBenchConfig;

typedef struct {
    double   alone_s, contended_s;   /* wall time of the two phases                   */
    uint64_t bg_commands;            /* background commands completed while contended */
    uint64_t fg_commands;            /* foreground commands in all                    */
} HostBenchResult;

/* bg_a, bg_b, bg_c: arrays of bg_n floats (c = a + b is computed over and over);
 * fg_a, fg_b, fg_c likewise with fg_n. alone_us / contended_us receive `samples`
 * latencies each (submit -> XQueueWaitAll return, microseconds, steady clock).
 * Installs the local scheduler with HPF for the run and puts the app-managed one back. */
XResult HostBenchRunVecAdd(const HostBenchConfig *cfg, const float *bg_a, const float *bg_b, float *bg_c,
                           const float *fg_a, const float *fg_b, float *fg_c,
                           double *alone_us, double *contended_us, HostBenchResult *res);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HOST_BENCH_H_ */
