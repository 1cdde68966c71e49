// Configuration surface: defaults and the environment variables that steer the
// queue and the scheduler. Names and defaults equal the reference's
// (protocol/include/xsched/protocol/def.h:3-70) so existing deployments keep
// their settings.
#pragma once

// Launch defaults of a freshly created XQueue (def.h:3-5).
#define XSCHED_DEFAULT_PREEMPT_LEVEL       kPreemptLevelBlock
#define XSCHED_DEFAULT_COMMAND_THRESHOLD   16
#define XSCHED_DEFAULT_COMMAND_BATCH_SIZE  8

// XQueue auto-creation by an interception shim (def.h:7-16).
#define XSCHED_AUTO_XQUEUE_ENV_NAME              "XSCHED_AUTO_XQUEUE"             // ON | OFF
#define XSCHED_AUTO_XQUEUE_LEVEL_ENV_NAME        "XSCHED_AUTO_XQUEUE_LEVEL"       // 1..3
#define XSCHED_AUTO_XQUEUE_THRESHOLD_ENV_NAME    "XSCHED_AUTO_XQUEUE_THRESHOLD"   // >= 1
#define XSCHED_AUTO_XQUEUE_BATCH_SIZE_ENV_NAME   "XSCHED_AUTO_XQUEUE_BATCH_SIZE"  // 1..threshold
#define XSCHED_AUTO_XQUEUE_PRIORITY_ENV_NAME     "XSCHED_AUTO_XQUEUE_PRIORITY"    // -256..255
#define XSCHED_AUTO_XQUEUE_UTILIZATION_ENV_NAME  "XSCHED_AUTO_XQUEUE_UTILIZATION" // 0..100
#define XSCHED_AUTO_XQUEUE_TIMESLICE_ENV_NAME    "XSCHED_AUTO_XQUEUE_TIMESLICE"   // us
#define XSCHED_AUTO_XQUEUE_DEADLINE_ENV_NAME     "XSCHED_AUTO_XQUEUE_DEADLINE"    // us
#define XSCHED_AUTO_XQUEUE_KDEADLINE_ENV_NAME    "XSCHED_AUTO_XQUEUE_KDEADLINE"   // k
#define XSCHED_AUTO_XQUEUE_LAXITY_ENV_NAME       "XSCHED_AUTO_XQUEUE_LAXITY"      // us

// Path of the real HIP runtime for an interception shim (def.h:25).
#define XSCHED_HIP_LIB_ENV_NAME  "XSCHED_HIP_LIB"

// Daemon rendezvous: the server listens on channel key 1, each client on its
// pid (def.h:35-38).
#define XSCHED_SERVER_CHANNEL_KEY   1
#define XSCHED_SERVER_DEFAULT_PORT  50000

#define XSCHED_UNKNOWN_NAME  "Unknown"

// Scheduler selection (def.h:45-49).
#define XSCHED_SCHEDULER_ENV_NAME  "XSCHED_SCHEDULER"
#define XSCHED_SCHEDULER_NAME_APP  "APP"
#define XSCHED_SCHEDULER_NAME_LCL  "LCL"
#define XSCHED_SCHEDULER_NAME_GLB  "GLB"

// What a scheduler-issued suspend additionally waits for (def.h:51-54).
#define XSCHED_SCHEDULER_SUSPEND_SYNC_HWQ_ENV_NAME   "XSCHED_SCHEDULER_SUSPEND_SYNC_HWQ"
#define XSCHED_SCHEDULER_SUSPEND_WAIT_ALL_ENV_NAME   "XSCHED_SCHEDULER_SUSPEND_WAIT_ALL"
#define XSCHED_SCHEDULER_SUSPEND_WAIT_IDLE_ENV_NAME  "XSCHED_SCHEDULER_SUSPEND_WAIT_IDLE"

// Policy selection; setting it implies the local scheduler (def.h:56-70).
#define XSCHED_POLICY_ENV_NAME   "XSCHED_POLICY"
#define XSCHED_POLICY_NAME_HPF   "HPF"
#define XSCHED_POLICY_NAME_HHPF  "HHPF"
#define XSCHED_POLICY_NAME_CHPF  "CHPF"
#define XSCHED_POLICY_NAME_UP    "UP"
#define XSCHED_POLICY_NAME_PUP   "PUP"
#define XSCHED_POLICY_NAME_SPUP  "SPUP"
#define XSCHED_POLICY_NAME_KEDF  "KEDF"
#define XSCHED_POLICY_NAME_LAX   "LAX"
#define XSCHED_POLICY_NAME_AWF   "AWF"
#define XSCHED_POLICY_NAME_CFS   "CFS"
#define XSCHED_POLICY_NAME_MLFQ  "MLFQ"

// ---- settings of the MI355X HIP backend (no reference counterpart) ----------
// Where the Level-2 preempt word lives: "host" (pinned host memory, written by a
// CPU store) or "device" (fine-grained device memory, written through a stream
// memory operation).
#define XSCHED_HIP_FLAG_MEM_ENV_NAME     "XSCHED_HIP_FLAG_MEM"
// Microseconds the launch thread polls a marker before it blocks in the driver.
#define XSCHED_HIP_SYNC_SPIN_US_ENV_NAME "XSCHED_HIP_SYNC_SPIN_US"
// Path of the daemon's Unix-domain socket directory.
#define XSCHED_SOCKET_DIR_ENV_NAME       "XSCHED_SOCKET_DIR"
/* ON (default) | OFF: launch on the submitting thread when the launch thread sleeps
 * (adapters that allow it, see HwQueueExtension::SupportDirectLaunch) */
#define XSCHED_DIRECT_LAUNCH_ENV_NAME    "XSCHED_DIRECT_LAUNCH"
