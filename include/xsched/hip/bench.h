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
    int64_t  laxity_us;   /* >= 0: XHintLaxity(laxity, lax_priority, priority) under the
                             laxity policy: the queue runs at lax_priority until laxity_us
                             after it became ready, then at `priority`                  */
    int64_t  period_us;   /* foreground: one command every period; background: ignored  */
    int32_t  lax_priority;/* see laxity_us                                              */
    int32_t  reserved;
    int64_t  deadline_us; /* > 0: a foreground command that completes later than this
                             after its submission counts as a deadline miss             */
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
                                  submission + fg.deadline_us (0 when no deadline)       */
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

/* Where the latency of one foreground command goes. One command per period, `samples` of
 * them, alone or (contended != 0) beside the background queues; a timing event is recorded
 * in stream order right before and right after the kernel. out holds 4 values per sample,
 * microseconds:
 *   [0] submit   host time until everything is handed over: through an XQueue the three
 *                XQueueSubmit calls (the launch itself runs inside them when the launch
 *                thread sleeps), otherwise the event records and the launch call
 *   [1] device   time between the two events on the device (hipEventElapsedTime): from the
 *                point the stream reaches the command to the kernel's end
 *   [2] wait     from there until the host knows the command is done (XQueueWaitAll returns;
 *                HwQueueSynchronize returns; hipStreamQuery polling succeeds)
 *   [3] total    [0] + [2]
 * mode 0: through the foreground XQueue (same path as XBenchRunForegroundAlone / Contended,
 *         plus the two event-record commands);
 * mode 1: the adapter without the XQueue core: HwQueueLaunch + HwQueueSynchronize on a
 *         stream of its own;
 * mode 2: plain HIP: a stand-in kernel of the same traffic launched with <<<>>> on a stream
 *         of its own and awaited by polling hipStreamQuery (AXPY foreground only): the floor
 *         the device and runtime set, with nothing of this library on the path.
 * The foreground output buffer is updated in every mode (applied counts them all). */
XResult XBenchRunForegroundBreakdown(XBench *b, int samples, int mode, int contended, double *out,
                                     XBenchPhaseResult *res);

/* Level-2 / level-1 preemption latency of background queue 0 while it streams:
 * `samples` rounds of XQueueSuspend(kQueueSuspendFlagSyncHwQueue) and
 * XQueueResume, each timed on the host (microseconds). */
XResult XBenchRunPreempt(XBench *b, int samples, double *suspend_us, double *resume_us,
                         XBenchPhaseResult *res);

/* The same loop timed on the DEVICE: XQueueSuspend without the hardware-queue sync, then
 * two timing events recorded back to back, one on an idle helper stream (it completes at
 * once: the device time at which the deactivation is out) and one on the queue's stream
 * behind everything in flight (it completes when the flushed launches have left the
 * device). drain_us[i] is the time between the two as hipEventElapsedTime reports it:
 * the device-side preemption latency, without any host wake-up in it. */
XResult XBenchRunPreemptDeviceTimed(XBench *b, int samples, double *drain_us, XBenchPhaseResult *res);

/* ---- mixed stress: many XQueues, one priority each, random arrivals ------------- */

typedef struct {
    int32_t  policy;        /* XPolicyType of the local scheduler                        */
    int32_t  n_queues;      /* <= 64; queue i has priority i and runs kernel i % 3:
                               0 AXPY over axpy_n elements, 1 GEMM gemm_n^3, 2 histogram
                               of hist_n keys                                            */
    int32_t  level;         /* XPreemptLevel of every queue                              */
    int32_t  guard;         /* guard mode of every command                               */
    int32_t  threshold;
    int32_t  batch;
    uint64_t axpy_n, gemm_n, hist_n;
    double   mean_interarrival_us; /* per queue, exponential                             */
    uint64_t seed;          /* arrivals: interval k of queue i = -mean * ln(1 - u),
                               u = top 53 bits of synthetic stream (seed, 1000 + i)
                               at index k, as a fraction of 2^53                         */
} XBenchStressConfig;

/* Creates the queues and their seeded inputs; queue i is "background queue i" for
 * XBenchReadOutput. */
XBench *XBenchCreateStress(const XBenchStressConfig *cfg);

/* Runs the arrival processes for `duration_s` seconds of arrivals, one thread per
 * queue: wait for the arrival time, submit one command, wait for it. The latency of a
 * command is completion minus ARRIVAL time (so it includes the time the queue was
 * behind). latency_us holds n_queues rows of `cap` values; counts[i] receives how many
 * were written for queue i (commands beyond `cap` are still executed and counted in
 * `applied`). */
XResult XBenchRunStress(XBench *b, double duration_s, double *latency_us, uint64_t cap,
                        uint64_t *counts, XBenchPhaseResult *res);

/* The same with only the queues whose bit is set in `queue_mask` (bit i = queue i) taking
 * arrivals, each with its own arrival process as above; the others stay idle. One bit set:
 * that queue's latency with the device to itself, the figure its latency in the full run is
 * compared with. */
XResult XBenchRunStressQueues(XBench *b, double duration_s, uint64_t queue_mask, double *latency_us,
                              uint64_t cap, uint64_t *counts, XBenchPhaseResult *res);

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
