// MI355X HIP hardware-queue adapter (internal declarations).
//
// HipQueue  - HwQueue over one hipStream_t: Level-1 launch and marker sync,
//             Level-2 deactivate / reactivate through the device-side guard.
// HipCommand - HwCommand with an optional completion marker (hipEvent).
// Replaces reference platforms/hip/hal/src/{hip_queue,hip_command}.cpp, which are
// Level-1 only. Calls the HIP runtime directly (no dlopen'd driver table).
#pragma once

#include <atomic>
#include <memory>
#include <mutex>
#include <vector>

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "shim_hooks.h"
#include "xsched/hip/guard.h"
#include "xsched/types.h"
#include "xsched/utils/xassert.h"
#include "xsched/preempt/hal/extensions.h"
#include "xsched/preempt/hal/hw_command.h"
#include "xsched/preempt/hal/hw_queue.h"

#define HIP_ASSERT(expr) \
    do { hipError_t e_ = (expr); \
         XASSERT(e_ == hipSuccess, "HIP error %d (%s) at %s", (int)e_, hipGetErrorString(e_), #expr); \
    } while (0)

namespace xsched::hip
{

/// Process-wide pool of timing-less events used as completion markers. Grows by
/// small chunks on demand (the reference creates 513 at the first use:
/// event_pool.h:26-32, utils/pool.h:15-24).
/// Events for markers, in two lists. An event that has gone through hipEventRecord() keeps
/// the stream of that record with the runtime: asking it while THAT stream captures a graph
/// fails (hipErrorCapturedEvent), whatever the event has been used for since. Handing an
/// event to a kernel launch as its stop event leaves no such trace and clears none, so the
/// markers that ride on kernels are events that were never recorded, and stay apart.
class EventPool
{
public:
    static EventPool &Instance();
    /// never_recorded: an event that no hipEventRecord() has seen (for a stop event).
    hipEvent_t Pop(bool never_recorded = false);
    void Push(hipEvent_t ev, bool recorded = true);
private:
    std::mutex mtx_;
    std::vector<hipEvent_t> fresh_;     // never recorded
    std::vector<hipEvent_t> recorded_;
};

/// Level-2 state of one queue: the preempt word and the progress-map slots.
class GuardState
{
public:
    static constexpr uint32_t kMaxWorkGroups = 1u << 18;   // per guarded command
    static constexpr uint32_t kSlotBytes = kMaxWorkGroups; // one byte per work-group
    static constexpr uint32_t kSlotsPerArena = 16;         // 4 MiB per arena

    /// A progress map and the generation tag its current owner writes into it.
    struct Slot { uint8_t *done = nullptr; uint32_t gen = 0; uint32_t index = 0; bool needs_clear = false; };

    explicit GuardState(int device);
    ~GuardState();

    /// Device-visible address of copy 0 of the preempt word, and copies - 1.
    const uint32_t *FlagDevPtr() const { return flag_dev_; }
    uint32_t FlagMask() const { return copies_ - 1; }
    /// The word in which flushed work-groups leave the epoch of their launch (cached device memory).
    uint32_t *FlushedDevPtr() const { return flushed_dev_; }
    uint32_t Epoch() const { return epoch_.load(std::memory_order_acquire); }

    /// Bump the preempt word; visible to running kernels within a memory round trip.
    void Deactivate(hipStream_t op_stream);
    /// Returns once the latest Deactivate() is visible to the device.
    void WaitFlagWritten(hipStream_t op_stream);

    /// A progress map with a fresh generation tag. The map is normally not cleared: bytes of
    /// earlier owners carry other tags. The caller has to clear it, in the order of its own
    /// stream, for the slot's first owner (fresh memory) and whenever the 8-bit tag wraps
    /// (needs_clear). Blocks on the device only when a new arena has to be allocated.
    Slot AcquireSlot();
    void ReleaseSlot(const Slot &slot);
    uint64_t SlotsInUse();
    uint64_t SlotsAllocated();
    /// Makes sure that a slot is free, allocating an arena if none is (the queue's device
    /// must be current). Called where waiting for an allocation harms nobody: when the queue
    /// goes to level 2 and at every submission of a guarded command, so that AcquireSlot(),
    /// which runs at launch time with the XQueue's locks held, finds one.
    void ReserveSlots();

private:
    uint8_t *AllocateArena();
    void AddArenaLocked(uint8_t *arena);
    const int device_;
    bool flag_on_host_ = false;
    uint32_t copies_ = 1;            // power of two
    uint32_t *flag_host_ = nullptr;  // pinned image of all copies (the word itself when on host)
    uint32_t *flag_dev_ = nullptr;   // GPU address of copy 0
    uint32_t *flushed_dev_ = nullptr; // written by flushed work-groups, read by later launches
    std::atomic<uint32_t> epoch_ { 0 };

    bool write_through_bar_ = false; // CPU stores straight into device memory
    std::mutex mtx_;                    // the preempt word (Deactivate)
    std::mutex slots_mtx_;              // everything below; never held across an allocation
    std::vector<uint8_t *> arenas_;
    std::vector<uint8_t *> slot_ptr_;   // by slot index
    std::vector<uint32_t> slot_gen_;    // last generation handed out, by slot index
    std::vector<uint32_t> free_slots_;  // slot indices
    uint64_t in_use_ = 0;
};

/// Device buffers that commands of one queue borrow for data they pass from one of their
/// kernels to the next (or from a flushed launch to its replay). A command takes a buffer
/// at its first launch and gives it back when it is destroyed, i.e. after its last launch
/// has left the device; buffers are recycled, never freed before the pool is. Commands in
/// flight at the same time must not share one: the copies of the preempt word are written
/// one after the other, so a work-group of a later command can still pass its entry
/// check while an earlier command has already been flushed and needs its data for the replay.
class ScratchPool
{
public:
    explicit ScratchPool(int device): device_(device) {}
    ~ScratchPool();
    /// A buffer of at least `bytes`, or nullptr when the device has no memory for one.
    /// Allocates only when none is free.
    void *Acquire(size_t bytes);
    void Release(void *ptr);
    size_t Buffers();
    size_t Bytes();
    /// Makes sure that a buffer of `bytes` is free (the first time: one for each command that
    /// will be in flight), so that the next Acquire(), at launch time, allocates nothing. The
    /// pool grows to what the queue holds at once plus one, however many commands wait in
    /// the XQueue.
    void Reserve(size_t bytes);

private:
    struct Buffer { void *ptr; size_t bytes; bool busy; };
    static constexpr int kInitialBuffers = 3;
    bool HasFreeLocked(size_t bytes) const;
    void *Allocate(size_t bytes);
    const int device_;
    std::mutex mtx_;                 // never held across an allocation
    std::vector<Buffer> buffers_;
};

class HipQueue;

class HipCommand : public preempt::HwCommand, public preempt::HwCommandExtension
{
public:
    explicit HipCommand(preempt::XCommandProperties props = preempt::kCommandPropertyNone)
        : HwCommand(props) {}
    virtual ~HipCommand();

    virtual void Synchronize() override;
    virtual bool Synchronizable() override { return wants_marker_; }
    /// The event itself is taken at launch, when the queue (and with it the kind of marker)
    /// is known.
    virtual bool EnableSynchronization() override { wants_marker_ = true; return true; }

    /// Enqueue on the queue's stream and (re-)record the marker behind it.
    /// `replay` is true when called from Reactivate().
    hipError_t LaunchWrapper(HipQueue &q, bool replay);

    /// Whether Reactivate() must enqueue this command again.
    virtual bool ReplayOnReactivate() const { return false; }


    /// Whether Enqueue() ends with a kernel launch that takes the marker (TakeStopEvent());
    /// decides which kind of event the command gets as its marker.
    virtual bool MarkerGoesWithKernel() const { return false; }

    /// Every command of this adapter except the host-side event wait only enqueues on
    /// the stream, so it may be launched on the submitting thread.
    virtual bool DirectLaunchable() override { return true; }
    virtual bool CompletedWithoutWaiting() override;

protected:
    virtual hipError_t Enqueue(HipQueue &q, bool replay) = 0;
    /// For an Enqueue() that ends with a kernel launch: the marker, to be handed to that LAST
    /// launch as its stop event (hipExtLaunchKernel and its relatives). The runtime then puts
    /// the event's completion signal on the kernel's own dispatch packet, and LaunchWrapper()
    /// records no marker behind the command. A recorded marker is a packet of its own that
    /// the next dispatch has to wait for: 1-3 us of device time per marked command, 2 us of a
    /// waiting caller's latency. nullptr when the command carries no marker or its queue
    /// records markers (HipQueue::MarkerOnKernel()): then launch the ordinary way. Whoever
    /// receives an event here must launch with it.
    hipEvent_t TakeStopEvent();
    /// Polls the event for the marker polling budget (no system call), then blocks in the driver.
    void WaitForEvent(hipEvent_t event);
    hipEvent_t marker_ = nullptr;

private:
    HipQueue *queue_ = nullptr; // for wait statistics; set at launch
    bool wants_marker_ = false;     // EnableSynchronization() was called
    bool marker_on_kernel_ = false; // this launch: the marker went out with a kernel
    bool marker_recorded_ = false;  // the marker has been through hipEventRecord()
};

/// hipLaunchKernelGGL, with `stop` (may be null) bound to the dispatch as its stop event.
template <typename... Args, typename F = void (*)(Args...)>
inline void LaunchWithStop(hipEvent_t stop, F kernel, const dim3 &grid, const dim3 &block, hipStream_t stream, Args... args)
{
    if (stop != nullptr) hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, nullptr, stop, 0, args...);
    else hipLaunchKernelGGL(kernel, grid, block, 0, stream, args...);
}

/// Base of the guarded victim kernels.
class HipGuardedCommand : public HipCommand
{
public:
    /// guard_mode: 0 plain, 1 guarded at level >= 2, 2 guarded always, 3 same as 1.
    HipGuardedCommand(uint32_t n_wg, int guard_mode)
        : HipCommand(guard_mode ? preempt::kCommandPropertyDeactivatable : preempt::kCommandPropertyNone)
        , n_wg_(n_wg), guard_mode_(guard_mode) {}
    virtual ~HipGuardedCommand();

    virtual bool ReplayOnReactivate() const override { return guard_mode_ != 0; }
    virtual bool MarkerGoesWithKernel() const override { return true; }
    uint32_t WorkGroups() const { return n_wg_; }

    /// The first launch takes a progress map (level 2) and whatever PrepareLaunch() borrows
    /// from the queue, with the XQueue's locks held. Either can mean a hipMalloc, which
    /// synchronises the device, when the queue's pools have nothing free: this call, from
    /// HipQueue::OnHwCommandSubmit() on the submitting thread and before any lock of the
    /// XQueue is taken, makes sure they have. It takes nothing itself: a command that waits
    /// in the XQueue holds no device memory.
    void PrepareOnSubmit(HipQueue &q);

protected:
    virtual hipError_t Enqueue(HipQueue &q, bool replay) override final;
    /// Called before every LaunchKernel() with the queue the command is launched on, for
    /// commands that need something of the queue (its scratch buffer).
    virtual hipError_t PrepareLaunch(HipQueue &) { return hipSuccess; }
    /// Called at submission: reserve in the queue's pools what PrepareLaunch() will take.
    virtual void ReserveOnSubmit(HipQueue &) {}
    /// Launch the kernel. `guarded` selects the variant with the guard compiled in.
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) = 0;

    const uint32_t n_wg_;
    const int guard_mode_;

private:
    void TakeSlot(HipQueue &q);
    std::shared_ptr<GuardState> guard_state_; // keeps the slot's arena alive
    GuardState::Slot slot_;
};

class HipQueue : public preempt::HwQueue, public preempt::HwQueueExtension
{
public:
    explicit HipQueue(hipStream_t stream);
    virtual ~HipQueue();

    virtual void Launch(std::shared_ptr<preempt::HwCommand> hw_cmd) override;
    virtual void Synchronize() override;
    virtual void Deactivate() override;
    virtual void Reactivate(const preempt::CommandLog &log) override;

    virtual XDevice       GetDevice()            override { return xdevice_; }
    virtual HwQueueHandle GetHandle()            override { return (HwQueueHandle)stream_; }
    virtual bool          SupportDynamicLevel()  override { return true; }
    virtual XPreemptLevel GetMaxSupportedLevel() override { return kPreemptLevelDeactivate; }
    virtual void OnPreemptLevelChange(XPreemptLevel level) override;
    virtual void OnXQueueCreate() override;
    virtual void OnHwCommandSubmit(std::shared_ptr<preempt::HwCommand> hw_cmd) override;
    /// Launch() and Synchronize() only issue stream calls under the caller's lock; the
    /// calling thread's current device is switched for the call and put back.
    virtual bool SupportDirectLaunch() override { return true; }
    virtual bool DeactivationConcernsInFlightWorkOnly() override { return true; }

    hipStream_t Stream() const { return stream_; }
    XPreemptLevel Level() const { return level_.load(std::memory_order_acquire); }
    /// Whether the markers of kernel commands go out as the stop event of the kernel itself
    /// (see HipCommand::TakeStopEvent()) instead of being recorded behind it. The price: the
    /// runtime learns of such a kernel's completion from its own handler thread, some 20 us
    /// after the event shows it, and until then hipStreamQuery() on the stream says "not
    /// ready" and hipStreamSynchronize() blocks. Queues whose users wait through the XQueue
    /// want it on (the default, XSCHED_HIP_MARKER_ON_KERNEL); the interception shim, whose
    /// applications ask the stream, turns it off for its queues.
    bool MarkerOnKernel() const { return marker_on_kernel_.load(std::memory_order_relaxed); }
    void SetMarkerOnKernel(bool on) { marker_on_kernel_.store(on, std::memory_order_relaxed); }
    const std::shared_ptr<GuardState> &Guard() const { return guard_; }
    const std::shared_ptr<ScratchPool> &Scratch() const { return scratch_; }

    // statistics (see HipQueueGetStats)
    std::atomic<uint64_t> n_launch { 0 }, n_replay { 0 }, n_deactivate { 0 }, n_reactivate { 0 };
    std::atomic<uint64_t> n_wait_polled { 0 }, n_wait_blocked { 0 };

private:
    const hipStream_t stream_;
    int device_ = 0;
    XDevice xdevice_ = 0;
    std::atomic<XPreemptLevel> level_ { kPreemptLevelUnknown };
    std::atomic<bool> marker_on_kernel_ { true };
    std::shared_ptr<GuardState> guard_;
    hipStream_t op_stream_ = nullptr; // flag writes when the word lives in device memory
    std::shared_ptr<ScratchPool> scratch_;

    // The newest command handed to the stream, while it carries a marker that was recorded
    // right behind it: Synchronize() then waits for that marker instead of putting another
    // one on the stream.
    std::mutex tail_mtx_;
    std::shared_ptr<preempt::HwCommand> tail_marked_;
};

/// Microseconds a marker wait polls before it blocks in the driver.
int64_t SyncSpinMicros();

/// While a stream of the process captures a graph in the default (global) mode, the runtime
/// refuses waits, queries and allocations from every thread that has not declared itself
/// relaxed, and invalidates the capture on top. The adapter's own waits and allocations
/// concern its own streams and markers, never a capturing one (the shim leaves a capturing
/// stream to the runtime), so they run relaxed; the thread's mode is put back afterwards
/// because the thread may be the application's.
class RelaxedCaptureScope
{
public:
    RelaxedCaptureScope() { (void)hipThreadExchangeStreamCaptureMode(&mode_); }
    ~RelaxedCaptureScope() { (void)hipThreadExchangeStreamCaptureMode(&mode_); }
private:
    hipStreamCaptureMode mode_ = hipStreamCaptureModeRelaxed;
};

/// Looks up, once per device, where HipHistogramLaunchNoAlloc's static scratch array lives on
/// `device` (which must be the calling thread's current device). False if the runtime refuses.
bool ResolveNoAllocScratch(int device);

} // namespace xsched::hip
