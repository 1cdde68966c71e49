/* XQueue C API: preemptible command queues layered over a hardware queue.
 *
 * Signatures and error behaviour match reference include/xsched/xqueue.h:16-112
 * (implemented there in preempt/src/xqueue/xqueue.cpp:255-402 and
 * preempt/src/hal/{hw_queue,hw_command}.cpp). Argument errors come back as
 * XResult codes; internal failures log and terminate the process.
 */
#ifndef XSCHED_XQUEUE_H_
#define XSCHED_XQUEUE_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Attach a new XQueue to hardware queue `hwq` (made by a HAL constructor such as
 * HipQueueCreate). `level` is an XPreemptLevel, `flags` an XQueueCreateFlag mask.
 * A hardware queue carries at most one XQueue; asking again returns the existing
 * handle. kQueueCreateFlagBlockingSubmit is answered with NotSupported.
 * reference xqueue.h:16, xqueue.cpp:12-49 */
XResult XQueueCreate(XQueueHandle *xq, HwQueueHandle hwq, int64_t level, int64_t flags);

/* Detach and destroy: resumes the queue if suspended and waits for every
 * submitted command. reference xqueue.h:21, xqueue.cpp:51-71 */
XResult XQueueDestroy(XQueueHandle xq);

/* Look up the XQueue attached to `hwq`. reference xqueue.h:29 */
XResult XQueueGet(XQueueHandle *xq, HwQueueHandle hwq);

/* Switch preemption level at run time; drains the queue first. Needs a hardware
 * queue that reports dynamic-level support and `level` within its maximum.
 * reference xqueue.h:35, xqueue.cpp:274-290 */
XResult XQueueSetPreemptLevel(XQueueHandle xq, XPreemptLevel level);

/* Set the in-flight window (`threshold`) and the marker period (`batch_size`);
 * a value <= 0 keeps the current one. threshold >= batch_size is required.
 * reference xqueue.h:42, xqueue.cpp:292-312 */
XResult XQueueSetLaunchConfig(XQueueHandle xq, int64_t threshold, int64_t batch_size);

/* Hand a command over to the queue. Ownership moves: the handle is no longer
 * registered afterwards. reference xqueue.h:49, xqueue.cpp:314-330 */
XResult XQueueSubmit(XQueueHandle xq, HwCommandHandle hw_cmd);

/* Wait for one still-registered command. reference xqueue.h:55 */
XResult XQueueWait(XQueueHandle xq, HwCommandHandle hw_cmd);

/* Wait until everything submitted so far has completed. reference xqueue.h:60 */
XResult XQueueWaitAll(XQueueHandle xq);

/* Idle / Ready. reference xqueue.h:66 */
XResult XQueueQuery(XQueueHandle xq, XQueueState *state);

/* Stop / continue execution; both are re-entrant. `flags` are XQueueSuspendFlag /
 * XQueueResumeFlag masks. reference xqueue.h:72,78; async_xqueue.cpp:91-150 */
XResult XQueueSuspend(XQueueHandle xq, int64_t flags);
XResult XQueueResume(XQueueHandle xq, int64_t flags);

/* Number of commands submitted over the queue's lifetime. reference xqueue.h:84 */
XResult XQueueProfileHwCommandCount(XQueueHandle xq, int64_t *count);

/* How many of them were launched on the submitting thread instead of the launch
 * thread (see HwQueueExtension::SupportDirectLaunch). No counterpart in the reference. */
XResult XQueueProfileDirectLaunchCount(XQueueHandle xq, int64_t *count);

/* Unregister a hardware queue; refused (NotAllowed) while an XQueue is attached.
 * reference xqueue.h:90, hw_queue.cpp:30-49 */
XResult HwQueueDestroy(HwQueueHandle hwq);

/* Bypass the XQueue: launch / drain directly on the hardware queue.
 * reference xqueue.h:96,101 */
XResult HwQueueLaunch(HwQueueHandle hwq, HwCommandHandle hw_cmd);
XResult HwQueueSynchronize(HwQueueHandle hwq);

/* A command whose launch body is a user function. `data` stays owned by the
 * caller and must outlive the launch. reference xqueue.h:107 */
XResult HwCommandCreateCallback(HwCommandHandle *hw_cmd, LaunchCallback launch, void *data);

/* Drop a command that was never submitted. reference xqueue.h:112 */
XResult HwCommandDestroy(HwCommandHandle hw_cmd);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_XQUEUE_H_ */
