/* Transparent HIP interception for MI355X: libshimhip.so.
 *
 * The library defines the HIP runtime entry points listed below under their own names.
 * Put in front of libamdhip64.so (LD_PRELOAD, or ahead of it on the link line), it turns
 * the stream work of an unmodified HIP program into XQueue commands: every stream the
 * program creates gets an XQueue configured from the XSCHED_AUTO_XQUEUE* variables
 * (nothing happens without XSCHED_AUTO_XQUEUE=ON), kernel launches, copies, fills and
 * event operations on such a stream are submitted to it, and the synchronising calls
 * wait on the XQueue. It takes the place of the reference's shim
 * (platforms/hip/shim/src/shim.cpp:21-322, entry points generated into
 * platforms/hip/shim/src/intercept.cpp), which replaces libamdhip64.so as a whole.
 *
 * Kernels that have the guard of xsched/hip/guard.h compiled in (last parameter an
 * XGuardArgs, one-dimensional grid) are submitted as guarded commands and can be flushed and
 * replayed at level 2; all other kernels are drain points there, as in the reference.
 *
 * Intercepted:
 *   kernels   hipLaunchKernel, hipModuleLaunchKernel, hipExtModuleLaunchKernel,
 *             hipLaunchCooperativeKernel, hipExtLaunchKernel              (shim.cpp:34-98)
 *   code      __hipRegisterFatBinary, __hipRegisterFunction, __hipUnregisterFatBinary,
 *             hipModuleLoad, hipModuleLoadData, hipModuleLoadDataEx,
 *             hipModuleGetFunction, hipModuleUnload                       (shim.cpp:100-111)
 *   memory    hipMemcpyAsync, hipMemcpyWithStream, hipMemcpyHtoDAsync, hipMemcpyDtoHAsync,
 *             hipMemcpyDtoDAsync, hipMemcpy2DAsync, hipMemcpyPeerAsync, hipMemsetAsync,
 *             hipMemsetD8Async, hipMemsetD16Async, hipMemsetD32Async, hipMemcpy, hipMemcpyHtoD,
 *             hipMemcpyDtoH, hipMemcpyDtoD, hipMemset, hipFree, hipFreeAsync,
 *             hipMallocAsync                                              (shim.cpp:113-150, shim.h:37-50)
 *   events    hipEventRecord, hipEventRecordWithFlags, hipEventQuery, hipEventSynchronize,
 *             hipEventElapsedTime, hipEventDestroy, hipStreamWaitEvent    (shim.cpp:152-257)
 *   streams   hipStreamCreate, hipStreamCreateWithFlags, hipStreamCreateWithPriority,
 *             hipStreamDestroy, hipStreamSynchronize, hipStreamQuery, hipStreamAddCallback,
 *             hipLaunchHostFunc, hipDeviceSynchronize, hipCtxSynchronize  (shim.cpp:259-320)
 *   graphs    hipStreamBeginCapture, hipStreamEndCapture (a capturing stream is left to the
 *             runtime), hipGraphLaunch (ordered behind the stream's XQueue)
 *
 * The two functions below are for tests and tools; a program under the shim needs neither.
 */
#ifndef XSCHED_HIP_SHIM_H_
#define XSCHED_HIP_SHIM_H_

#include "xsched/types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The explicit arguments of `kernel` (its mangled name) as the code object `image` of
 * `bytes` bytes records them: a clang offload bundle as hipcc embeds it (plain, or
 * compressed with zstd or zlib), or a bare AMDGPU ELF file. Writes up to `cap`
 * (offset, size) pairs and the argument count to `n_args`. NotFound: no such kernel;
 * NotSupported: a compressed bundle that cannot be unpacked on this machine (no libzstd /
 * libz); InvalidValue: not a code object, or malformed. Takes the place of the comgr walk
 * in reference platforms/hip/hal/src/kernel_param.cpp:256-345. */
XResult HipShimKernelArgLayout(const void *image, size_t bytes, const char *kernel,
                               uint32_t *offsets, uint32_t *sizes, size_t cap, size_t *n_args);

/* Counters of this process, `out` receives 8 values:
 * [0] kernel launches submitted as XQueue commands,
 * [1] kernel launches handed to the runtime after draining the XQueue (argument layout
 *     unknown, cooperative / ext launches),
 * [2] kernel launches passed straight through (no XQueue on the stream, null stream),
 * [3] copies and fills submitted as commands, [4] copies done after draining the XQueue,
 * [5] event records submitted as commands, [6] cross-queue event waits,
 * [7] kernels whose argument layout is known. (Guarded launches are among [0]; the line that
 * XSCHED_SHIM_STATS=1 prints at exit also has them, and the queues' own counters.) */
XResult HipShimGetStats(uint64_t *out);

#ifdef __cplusplus
}
#endif

#endif /* XSCHED_HIP_SHIM_H_ */
