/* Contention benchmark harness for the MI355X HIP adapter (C entry points).
 *
 * It drives the adapter only through the public API (HipQueueCreate, XQueueCreate,
 * XQueueSetLaunchConfig, XHintPriority / XHintLaxity, Hip*CommandCreate,
 * XQueueSubmit, XQueueWaitAll, XQueueSuspend / XQueueResume), the way the
 * reference's demo applications do (reference
 * examples/Linux/3_intra_process_sched/app_concurrent.hip:26-96) and times the way
 * its preemption micro-benchmark does (platforms/cuda/test/main/level.cu:37-86).
 * No reference counterpart as a library; it exists so that a measurement needs no
 * per-call Python overhead on the timed path.
 */
#ifndef XSCHED_HIP_BENCH_H_
#define XSCHED_HIP_BENCH_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { kXBenchAxpy = 0, kXBenchGemm = 1, kXBenchHist = 2 };

typedef struct {
    int32_t  kind;        /* kXBenchAxpy / Gemm / Hist                                  */
    int32_t  guard;       /* guard mode of its commands (see hal.h)                     */
    uint64_t n;           /* axpy: elements, hist: keys, gemm: M = N = K = n            */
    int32_t  level;       /* XPreemptLevel of its XQueue                                */
    int32_t  threshold;   /* in-flight window                                           */
    int32_t  batch;       /* marker period                                              */
    int32_t  priority;    /* XHintPriority (HPF) / critical priority (LAX)              */
    int64_t  laxity_us;   /* >= 0: XHintLaxity(laxity, lax_prio = PRIORITY_MIN, priority) */
    int64_t  period_us;   /* foreground: one command every period; background: ignored  */
} XBenchQueueSpec;

typedef struct {
    int32_t  policy;       /* XPolicyType for the local scheduler; 0 = app-managed       */
    int32_t  n_bg;         /* number of background XQueues (each on its own stream)      */
    XBenchQueueSpec bg;
    XBenchQueueSpec fg;
    int32_t  bg_burst;     /* background commands submitted between two drains           */
    uint64_t seed;
} XBenchConfig;

typedef struct {
    double   elapsed_s;        /* wall time of the phase                                 */
    uint64_t bg_commands;      /* background commands completed in the phase             */
    double   bg_stream_ms;     /* device time on bg stream 0 between first and last
                                  command of the phase, from HIP events on that stream   */
    uint64_t bg_stream_cmds;   /* commands of bg queue 0 inside bg_stream_ms             */
    uint64_t fg_samples;       /* foreground latencies written                           */
    uint64_t fg_deadline_miss; /* foreground commands that completed later than
                                  ready time + fg.laxity_us (0 when no laxity)           */
    uint64_t stats[8];         /* HipQueueGetStats of bg queue 0 at the end              */
} XBenchPhaseResult;

typedef struct XBench XBench;

/* Allocate device buffers, fill them with the seeded synthetic inputs, create the
 * streams / HwQueues / XQueues. Returns NULL on bad arguments. */
XBench *XBenchCreate(const XBenchConfig *cfg);
void XBenchDestroy(XBench *b);

/* Foreground alone: `samples` commands, one per period; latency = submit ->
 * XQueueWaitAll return, microseconds, steady clock. */
XResult XBenchRunForegroundAlone(XBench *b, int samples, double *latency_us, XBenchPhaseResult *res);

/* Background alone for `commands` commands per queue, back to back. */
XResult XBenchRunBackgroundAlone(XBench *b, int commands, XBenchPhaseResult *res);

/* Foreground every period while all background queues stream back to back. */
XResult XBenchRunContended(XBench *b, int samples, double *latency_us, XBenchPhaseResult *res);

/* Level-2 / level-1 preemption latency of background queue 0 while it streams:
 * `samples` rounds of XQueueSuspend(kQueueSuspendFlagSyncHwQueue) and
 * XQueueResume, each timed on the host (microseconds). */
XResult XBenchRunPreempt(XBench *b, int samples, double *suspend_us, double *resume_us,
                         XBenchPhaseResult *res);

/* Copy `count` elements starting at `first` of a result buffer to the host:
 * which = 0: background queue `q` output (axpy y / gemm C / hist bins),
 * which = 1: foreground output. Element size: axpy 4, gemm 2, hist 4 bytes.
 * `applied` receives how many commands have been applied to that buffer so far. */
XResult XBenchReadOutput(XBench *b, int which, int q, uint64_t first, uint64_t count, void *dst,
                         uint64_t *applied);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HIP_BENCH_H_ */
