/* Public C types of the XQueue / XHint API.
 *
 * Every enumerator value and typedef width here is wire-visible (language
 * bindings, scheduler daemon messages) and therefore equals the value used by
 * XSched itself: reference include/xsched/types.h:10-149.
 */
#ifndef XSCHED_TYPES_H_
#define XSCHED_TYPES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- opaque handles (reference types.h:10-14) ---------------------------- */
typedef uint64_t XDevice;          /* (XDeviceType << 32) | XDeviceId            */
typedef uint32_t XDeviceId;        /* packed PCI address of the device           */
typedef uint64_t XQueueHandle;
typedef uint64_t HwQueueHandle;
typedef uint64_t HwCommandHandle;

/* ---- result codes (reference types.h:16-25) ------------------------------ */
typedef enum {
    kXSchedSuccess           = 0,
    kXSchedErrorHardware     = 1,
    kXSchedErrorInvalidValue = 2,
    kXSchedErrorNotFound     = 3,
    kXSchedErrorNotAllowed   = 4,
    kXSchedErrorNotSupported = 5,
    kXSchedErrorBadResponse  = 6,
    kXSchedErrorUnknown      = 999,
} XResult;

/* ---- platforms and device classes (reference types.h:27-46) -------------- */
typedef enum {
    kPlatformUnknown = 0, kPlatformVPI = 1, kPlatformCUDA = 2, kPlatformCUDLA = 3,
    kPlatformHIP = 4, kPlatformAscend = 5, kPlatformOpenCL = 6, kPlatformLevelZero = 7,
} XPlatform;

typedef enum {
    kDeviceTypeUnknown = 0, kDeviceTypeCPU = 1, kDeviceTypeGPU = 2, kDeviceTypeNPU = 3,
    kDeviceTypeFPGA = 4, kDeviceTypeASIC = 5, kDeviceTypeMCA = 6,
} XDeviceType;

/* ---- preemption levels (reference types.h:48-54) -------------------------
 * Block      : stop launching; commands already in flight drain.
 * Deactivate : in-flight commands are additionally flushed from the device and
 *              replayed on resume.
 * Interrupt  : the running command is killed / context-switched.             */
typedef enum {
    kPreemptLevelUnknown    = 0,
    kPreemptLevelBlock      = 1,
    kPreemptLevelDeactivate = 2,
    kPreemptLevelInterrupt  = 3,
    kPreemptLevelMax,
} XPreemptLevel;

/* ---- queue state, features, flags (reference types.h:56-91) -------------- */
typedef enum {
    kQueueStateUnknown = 0,
    kQueueStateIdle    = 1,   /* nothing submitted that has not completed */
    kQueueStateReady   = 2,   /* has pending or in-flight commands        */
} XQueueState;

typedef enum {
    kQueueFeatureNone               = 0x0000,
    kQueueFeatureAsyncSubmit        = 0x0001,
    kQueueFeatureDynamicLevel       = 0x0002,
    kQueueFeatureDynamicThreshold   = 0x0004,
    kQueueFeatureDynamicBatchSize   = 0x0008,
    kQueueFeatureSyncSuspend        = 0x0010,
    kQueueFeatureResumeDropCommands = 0x0020,
    kQueueFeatureMaskAll            = -1,
} XQueueFeature;

typedef enum {
    kQueueCreateFlagNone           = 0x0000,
    kQueueCreateFlagBlockingSubmit = 0x0001,
    kQueueCreateFlagMaskAll        = -1,
} XQueueCreateFlag;

typedef enum {
    kQueueSuspendFlagNone        = 0x0000,
    kQueueSuspendFlagSyncHwQueue = 0x0001,  /* also drain the hardware queue    */
    kQueueSuspendFlagWaitAll     = 0x0002,  /* finish everything submitted first */
    kQueueSuspendFlagWaitIdle    = 0x0004,  /* wait for the next idle transition */
    kQueueSuspendFlagMaskAll     = -1,
} XQueueSuspendFlag;

typedef enum {
    kQueueResumeFlagNone         = 0x0000,
    kQueueResumeFlagDropCommands = 0x0001,  /* discard everything submitted so far */
    kQueueResumeFlagMaskAll      = -1,
} XQueueResumeFlag;

/* ---- schedulers and policies (reference types.h:93-118) ------------------ */
typedef enum {
    kSchedulerUnknown    = 0,
    kSchedulerAppManaged = 1,
    kSchedulerLocal      = 2,
    kSchedulerGlobal     = 3,
    kSchedulerMax,
} XSchedulerType;

typedef enum {
    kPolicyUnknown                           = 0,
    kPolicyHighestPriorityFirst              = 1,
    kPolicyHeterogeneousHighestPriorityFirst = 2,
    kPolicyCPUHighestPriorityFirst           = 3,
    kPolicyUtilizationPartition              = 4,
    kPolicyProcessUtilizationPartition       = 5,
    kPolicyStrictProcessUtilizationPartition = 6,
    kPolicyKEarliestDeadlineFirst            = 7,
    kPolicyLaxity                            = 8,
    kPolicyActiveWindowFirst                 = 9,
    kPolicyCompletelyFairScheduler           = 10,
    kPolicyMultiLevelFeedbackQueue           = 11,
    kPolicyMax,
} XPolicyType;

/* Launch body of a callback command. It runs on the XQueue's launch thread with
 * the launch lock held, so it must only enqueue work (reference types.h:120). */
typedef XResult (*LaunchCallback)(HwQueueHandle, void *);

/* ---- hint value domains (reference types.h:122-145) ---------------------- */
typedef int32_t Priority;              /* larger runs first */
#define PRIORITY_NO_EXECUTE -256
#define PRIORITY_MIN        -255
#define PRIORITY_DEFAULT     000
#define PRIORITY_MAX         255

typedef int32_t Utilization;           /* percent */
#define UTILIZATION_MIN      0
#define UTILIZATION_DEFAULT  100
#define UTILIZATION_MAX      100

typedef int64_t Timeslice;             /* microseconds */
#define TIMESLICE_MIN        100
#define TIMESLICE_DEFAULT    5000
#define TIMESLICE_MAX        10000000
#define TIMESLICE_UNLIMITED  UINT64_MAX

typedef int64_t Laxity;                /* microseconds */
#define NO_LAXITY           -1

typedef int64_t Deadline;              /* microseconds */
#define NO_DEADLINE         -1

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_TYPES_H_ */
