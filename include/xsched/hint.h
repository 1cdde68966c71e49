/* XHint C API: scheduling hints relayed to the active scheduler / policy.
 * Signatures match reference include/xsched/hint.h:13-56 (implemented there in
 * preempt/src/sched/hint.cpp:12-71).
 */
#ifndef XSCHED_HINT_H_
#define XSCHED_HINT_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Choose the scheduler; `policy` matters for kSchedulerLocal only.
 * reference hint.h:13, agent.cpp:111-140 */
XResult XHintSetScheduler(XSchedulerType scheduler, XPolicyType policy);

/* Larger `prio` wins; clamped by the policy to [PRIORITY_MIN, PRIORITY_MAX].
 * reference hint.h:22 */
XResult XHintPriority(XQueueHandle xq, Priority prio);

/* Share of the device in percent. reference hint.h:29 */
XResult XHintUtilization(XQueueHandle xq, Utilization util);

/* Policy-wide timeslice in microseconds. reference hint.h:34 */
XResult XHintTimeslice(Timeslice ts_us);

/* The queue runs at `lax_prio` until `lax_us` after it became ready and at
 * `crit_prio` from then on. reference hint.h:43 */
XResult XHintLaxity(XQueueHandle xq, Laxity lax_us, Priority lax_prio, Priority crit_prio);

/* Relative deadline: ready time + `ddl_us`. reference hint.h:50 */
XResult XHintDeadline(XQueueHandle xq, Deadline ddl_us);

/* Concurrency of the K-earliest-deadline-first policy. reference hint.h:56 */
XResult XHintKDeadline(size_t k);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HINT_H_ */
