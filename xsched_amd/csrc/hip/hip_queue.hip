// HipQueue, its Level-2 guard state, the marker pool and the command base classes.
#include <chrono>
#include <fcntl.h>
#include <unistd.h>
#include <cstring>
#include <string>
#include <thread>

#include "hip_hal.h"
#include "xsched/hip/hal.h"
#include "xsched/utils/env.h"
#include "xsched/protocol/def.h"
#include "xsched/protocol/device.h"

using namespace xsched::preempt;
using namespace xsched::protocol;

namespace xsched::hip
{

namespace
{

/// Makes `device` current for the calling thread and restores what was current before.
/// The launch thread always has it current (OnXQueueCreate); an application thread that
/// launches directly may not.
class DeviceScope
{
public:
    explicit DeviceScope(int device)
    {
        int cur = device;
        if (hipGetDevice(&cur) == hipSuccess && cur != device) {
            previous_ = cur;
            HIP_ASSERT(hipSetDevice(device));
        }
    }
    ~DeviceScope() { if (previous_ >= 0) (void)hipSetDevice(previous_); }

private:
    int previous_ = -1;
};

} // namespace

namespace
{

/// The runtime takes the completion signals of a device queue's packets from a pool (64 to
/// begin with), and every 256 packets of a queue (a kernel launch is one packet, an event
/// record two) one call into it takes 30-45 us longer than the others. For a queue that gets a
/// command every few milliseconds and waits for it, that is every 60th to 85th command, more
/// than 1 % of them: it was the p99 of such a queue on an idle device (70-80 us at a median
/// of 30). With a pool of 512 the long calls did not show in 800 commands (p99 43 us). The
/// pool's size is read from the environment when the runtime starts, so it is asked for when
/// this library is loaded; a value the user has set stays, and XSCHED_HIP_SIGNAL_POOL=0 keeps
/// this library from touching the variable (any other number is the size asked for).
bool g_signal_pool_asked_for = false;   // this library set the variable (it was not set before)

__attribute__((constructor)) void AskForLargerSignalPool()
{
    int64_t size = 512;
    GetEnvInt64("XSCHED_HIP_SIGNAL_POOL", size);
    if (size <= 0) return;
    g_signal_pool_asked_for = getenv("ROC_SIGNAL_POOL_SIZE") == nullptr;
    (void)setenv("ROC_SIGNAL_POOL_SIZE", std::to_string(size).c_str(), 0 /* keep what is set */);
}

/// Said once, when the first queue is created: what the variable holds and who set it. The
/// runtime reads it at its first call in the process, so a value set by this library only
/// counts if the library was loaded before that (a program that used the GPU first, then
/// loaded the adapter, has the runtime's own pool of 64 whatever the variable says now).
void ReportSignalPool()
{
    static std::once_flag once;
    std::call_once(once, []() {
        const char *v = getenv("ROC_SIGNAL_POOL_SIZE");
        XINFO("ROC_SIGNAL_POOL_SIZE=%s (%s); the HIP runtime reads it at its first call in the process", v ? v : "(unset)",
              g_signal_pool_asked_for ? "set by this library when it was loaded" : "as found in the environment");
    });
}

} // namespace


int64_t SyncSpinMicros()
{
    static const int64_t us = []() {
        int64_t v = 200;
        GetEnvInt64(XSCHED_HIP_SYNC_SPIN_US_ENV_NAME, v);
        return v < 0 ? (int64_t)0 : v;
    }();
    return us;
}

namespace
{
/// Polls the event for up to `spin_us` (no system call, no sleep / wake latency); true once
/// it has completed, false when the time is up (the caller then blocks in the driver, so a
/// long wait does not burn a core).
bool PollEvent(hipEvent_t ev, int64_t spin_us)
{
    if (spin_us <= 0) return false;
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::microseconds(spin_us);
    for (int probes = 1;; ++probes) {
        const hipError_t err = hipEventQuery(ev);
        if (err == hipSuccess) return true;
        XASSERT(err == hipErrorNotReady, "hipEventQuery failed: %d (%s)", (int)err, hipGetErrorString(err));
        if ((probes & 7) == 0 && std::chrono::steady_clock::now() >= deadline) return false;
        __builtin_ia32_pause();
    }
}
} // namespace

// ---- EventPool ---------------------------------------------------------------

EventPool &EventPool::Instance()
{
    static EventPool *pool = new EventPool(); // never destroyed: commands may outlive main()
    return *pool;
}

hipEvent_t EventPool::Pop(bool never_recorded)
{
    std::lock_guard<std::mutex> lock(mtx_);
    std::vector<hipEvent_t> &from = (never_recorded || recorded_.empty()) ? fresh_ : recorded_;
    if (from.empty()) {
        for (int i = 0; i < 16; ++i) {
            hipEvent_t ev = nullptr;
            HIP_ASSERT(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
            fresh_.push_back(ev);
        }
    }
    hipEvent_t ev = from.back();
    from.pop_back();
    return ev;
}

void EventPool::Push(hipEvent_t ev, bool recorded)
{
    std::lock_guard<std::mutex> lock(mtx_);
    (recorded ? recorded_ : fresh_).push_back(ev);
}

// ---- GuardState --------------------------------------------------------------
// Placement of the preempt word (XSCHED_HIP_FLAG_MEM):
//   device (default) fine-grained device memory, read by kernels from local memory.
//          How the CPU rewrites the copies (XSCHED_HIP_FLAG_WRITE):
//            bar   (default when the device exposes all of its memory to the CPU)
//                  plain CPU stores through the PCIe aperture: posted writes, no
//                  runtime call, visible to the device about a microsecond later
//            copy  one small host-to-device copy on a side stream
//   host   pinned, coherent host memory mapped into the device. The CPU flips the
//          copies with plain stores; kernels read them across the host link,
//          which limits them to a few tens of millions of work-groups per second.
// XSCHED_HIP_FLAG_COPIES: number of copies (power of two, default 64).

namespace
{
// Whether the CPU can load and store the word at `p`, asked of the kernel instead of found
// out by faulting: writing to a pipe makes the kernel read the user's bytes and reading from
// it makes the kernel store them, and for an address the process cannot access both return
// EFAULT. No signal is raised and no process-wide handler is touched, so other threads may
// do what they like meanwhile.
bool CpuCanAccess(uint32_t *p)
{
    int fds[2];
    if (pipe2(fds, O_CLOEXEC | O_NONBLOCK) != 0) return false;
    bool ok = write(fds[1], p, sizeof(uint32_t)) == (ssize_t)sizeof(uint32_t);   // loads *p
    ok = ok && read(fds[0], p, sizeof(uint32_t)) == (ssize_t)sizeof(uint32_t);   // stores it back
    close(fds[0]);
    close(fds[1]);
    return ok;
}

// CPU stores through the PCIe aperture are only of use if the device sees them: store a
// pattern with the CPU, read the word back with a device copy, put the zero back.
bool CpuStoresReachDevice(uint32_t *dev_word)
{
    const uint32_t pattern = 0x5CA1AB1Eu;
    __atomic_store_n(dev_word, pattern, __ATOMIC_RELEASE);
    __builtin_ia32_sfence();
    uint32_t seen = 0;
    bool ok = hipMemcpy(&seen, dev_word, sizeof seen, hipMemcpyDeviceToHost) == hipSuccess && seen == pattern;
    __atomic_store_n(dev_word, 0u, __ATOMIC_RELEASE);
    __builtin_ia32_sfence();
    ok = ok && hipMemcpy(&seen, dev_word, sizeof seen, hipMemcpyDeviceToHost) == hipSuccess && seen == 0u;
    return ok;
}

// The answer is a property of the device (and of this kind of allocation): found once per
// device, under a lock, with the first preempt word allocated there.
bool BarWritesWork(int device, uint32_t *dev_word)
{
    static std::mutex mtx;
    static int known[64] = {}; // 0 unknown, 1 yes, 2 no
    std::lock_guard<std::mutex> lock(mtx);
    const int slot = device >= 0 && device < 64 ? device : 63;
    if (known[slot] == 0) {
        int large_bar = 0;
        (void)hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, device);
        const bool ok = large_bar != 0 && CpuCanAccess(dev_word) && CpuStoresReachDevice(dev_word);
        known[slot] = ok ? 1 : 2;
    }
    return known[slot] == 1;
}
} // namespace

GuardState::GuardState(int device): device_(device)
{
    flag_on_host_ = GetEnv(XSCHED_HIP_FLAG_MEM_ENV_NAME) == "host";
    int64_t copies = 64;
    GetEnvInt64("XSCHED_HIP_FLAG_COPIES", copies);
    copies_ = 1;
    while ((int64_t)copies_ * 2 <= copies && copies_ < 4096) copies_ *= 2;

    // no launch ever carries epoch 0xFFFFFFFF
    HIP_ASSERT(hipMalloc((void **)&flushed_dev_, 256));
    HIP_ASSERT(hipMemset(flushed_dev_, 0xFF, 256));

    const size_t bytes = (size_t)copies_ * kXGuardFlagStrideWords * sizeof(uint32_t);
    HIP_ASSERT(hipHostMalloc((void **)&flag_host_, bytes, hipHostMallocMapped | hipHostMallocCoherent));
    memset(flag_host_, 0, bytes);
    if (flag_on_host_) {
        HIP_ASSERT(hipHostGetDevicePointer((void **)&flag_dev_, flag_host_, 0));
        HIP_ASSERT(hipDeviceSynchronize());
        return;
    }
    HIP_ASSERT(hipExtMallocWithFlags((void **)&flag_dev_, bytes, hipDeviceMallocFinegrained));
    HIP_ASSERT(hipMemset(flag_dev_, 0, bytes));
    // hipMemset returns before its fills have run: nothing may be launched against the words before this
    HIP_ASSERT(hipDeviceSynchronize());

    const std::string how = GetEnv("XSCHED_HIP_FLAG_WRITE");
    if (how != "copy") write_through_bar_ = BarWritesWork(device_, flag_dev_);
    if (how == "bar" && !write_through_bar_) {
        XWARN("XSCHED_HIP_FLAG_WRITE=bar, but device memory is not CPU-accessible; using copies");
    }
}

GuardState::~GuardState()
{
    // Arenas and the word are only released here, when no command holds the state
    // any more (each guarded command keeps a reference while it owns a slot).
    for (uint8_t *a : arenas_) (void)hipFree(a);
    if (!flag_on_host_ && flag_dev_) (void)hipFree(flag_dev_);
    if (flushed_dev_) (void)hipFree(flushed_dev_);
    if (flag_host_) (void)hipHostFree(flag_host_);
}

void GuardState::Deactivate(hipStream_t op_stream)
{
    std::lock_guard<std::mutex> lock(mtx_);
    const uint32_t e = epoch_.fetch_add(1, std::memory_order_acq_rel) + 1;
    uint32_t *target = (flag_on_host_ || !write_through_bar_) ? flag_host_ : flag_dev_;
    for (uint32_t c = 0; c < copies_; ++c) {
        __atomic_store_n(&target[(size_t)c * kXGuardFlagStrideWords], e, __ATOMIC_RELEASE);
    }
    if (!flag_on_host_ && write_through_bar_) {
        __builtin_ia32_sfence(); // push the write-combined stores out now
    } else if (!flag_on_host_) {
        const size_t bytes = (size_t)copies_ * kXGuardFlagStrideWords * sizeof(uint32_t);
        HIP_ASSERT(hipMemcpyAsync(flag_dev_, flag_host_, bytes, hipMemcpyHostToDevice, op_stream));
    }
}

void GuardState::WaitFlagWritten(hipStream_t op_stream)
{
    RelaxedCaptureScope relaxed;
    if (!flag_on_host_ && !write_through_bar_) HIP_ASSERT(hipStreamSynchronize(op_stream));
}

uint8_t *GuardState::AllocateArena()
{
    DeviceScope scope(device_);
    RelaxedCaptureScope relaxed;
    uint8_t *arena = nullptr;
    const size_t bytes = (size_t)kSlotsPerArena * kSlotBytes;
    // Not cleared here: hipMemset() on device memory returns before the fill has run,
    // and a kernel launched afterwards on a non-blocking stream overtakes it (its first
    // progress bytes were then wiped, and a replay applied those work-groups again).
    // Every slot is cleared in the order of its owner's stream instead, see Enqueue().
    HIP_ASSERT(hipMalloc((void **)&arena, bytes));
    return arena;
}

void GuardState::AddArenaLocked(uint8_t *arena)
{
    arenas_.push_back(arena);
    for (uint32_t i = 0; i < kSlotsPerArena; ++i) {
        free_slots_.push_back((uint32_t)slot_ptr_.size());
        slot_ptr_.push_back(arena + (size_t)i * kSlotBytes);
        slot_gen_.push_back(0);
    }
}

void GuardState::ReserveSlots()
{
    {
        std::lock_guard<std::mutex> lock(slots_mtx_);
        if (!free_slots_.empty()) return;
    }
    // Outside the lock: a launch that finds a slot free does not wait for this allocation.
    // Two threads that both find nothing free add an arena each, which is harmless.
    uint8_t *arena = AllocateArena();
    std::lock_guard<std::mutex> lock(slots_mtx_);
    AddArenaLocked(arena);
}

GuardState::Slot GuardState::AcquireSlot()
{
    std::unique_lock<std::mutex> lock(slots_mtx_);
    while (free_slots_.empty()) {
        lock.unlock();
        uint8_t *arena = AllocateArena();
        lock.lock();
        AddArenaLocked(arena);
    }
    Slot slot;
    slot.index = free_slots_.back();
    free_slots_.pop_back();
    slot.done = slot_ptr_[slot.index];
    uint32_t gen = slot_gen_[slot.index] + 1;
    if (gen > 255) gen = 1;
    // first owner: the memory is as hipMalloc left it; later: tags of 255 owners ago could collide
    slot.needs_clear = gen == 1;
    slot_gen_[slot.index] = gen;
    slot.gen = gen;
    in_use_++;
    return slot;
}

void GuardState::ReleaseSlot(const Slot &slot)
{
    std::lock_guard<std::mutex> lock(slots_mtx_);
    free_slots_.push_back(slot.index);
    in_use_--;
}

uint64_t GuardState::SlotsAllocated()
{
    std::lock_guard<std::mutex> lock(slots_mtx_);
    return slot_ptr_.size();
}

uint64_t GuardState::SlotsInUse()
{
    std::lock_guard<std::mutex> lock(slots_mtx_);
    return in_use_;
}

// ---- HipCommand --------------------------------------------------------------

HipCommand::~HipCommand()
{
    if (marker_ != nullptr) EventPool::Instance().Push(marker_, marker_recorded_);
}

hipError_t HipCommand::LaunchWrapper(HipQueue &q, bool replay)
{
    queue_ = &q;
    if (wants_marker_ && marker_ == nullptr) {
        const bool for_a_kernel = MarkerGoesWithKernel() && q.MarkerOnKernel();
        marker_ = EventPool::Instance().Pop(for_a_kernel);
        marker_recorded_ = !for_a_kernel;
    }
    marker_on_kernel_ = false;
    hipError_t err;
    if (marker_ != nullptr && !marker_recorded_) {
        // A launch that takes an event is one of the calls that the runtime refuses, and
        // answers by invalidating the capture, while ANOTHER stream of the process captures a
        // graph in the default (global) mode; like the adapter's waits it concerns this
        // queue's stream only.
        RelaxedCaptureScope relaxed;
        err = Enqueue(q, replay);
    } else {
        err = Enqueue(q, replay);
    }
    if (UNLIKELY(err != hipSuccess)) return err;
    // Recording again after a replay moves the marker behind the replayed work,
    // which is what a later Synchronize() has to wait for (a replayed kernel that carries
    // the marker itself does the same).
    if (marker_ != nullptr && !marker_on_kernel_) {
        marker_recorded_ = true;
        err = hipEventRecord(marker_, q.Stream());
    }
    return err;
}

hipEvent_t HipCommand::TakeStopEvent()
{
    if (marker_ == nullptr || marker_recorded_) return nullptr;
    marker_on_kernel_ = true;
    return marker_;
}

bool HipCommand::CompletedWithoutWaiting()
{
    if (marker_ == nullptr) return false;
    RelaxedCaptureScope relaxed;
    const hipError_t err = hipEventQuery(marker_);
    if (err != hipSuccess) (void)hipGetLastError();
    return err == hipSuccess;
}

// Marker wait, sized for device work in the 10 us .. 1 ms range: poll the event
// for a bounded time (no system call, no sleep/wake latency), then fall back to
// the driver's blocking wait so that a long wait does not burn a core.
void HipCommand::Synchronize()
{
    XASSERT(marker_ != nullptr, "Synchronize() needs EnableSynchronization() before launch");
    WaitForEvent(marker_);
}

void HipCommand::WaitForEvent(hipEvent_t event)
{
    RelaxedCaptureScope relaxed;
    if (PollEvent(event, SyncSpinMicros())) {
        if (queue_) queue_->n_wait_polled.fetch_add(1, std::memory_order_relaxed);
        return;
    }
    if (queue_) queue_->n_wait_blocked.fetch_add(1, std::memory_order_relaxed);
    HIP_ASSERT(hipEventSynchronize(event));
}

// ---- HipGuardedCommand -------------------------------------------------------

HipGuardedCommand::~HipGuardedCommand()
{
    if (slot_.done != nullptr) guard_state_->ReleaseSlot(slot_);
}

// Zeroes one progress-map slot, in stream order in front of its owner's first launch.
__global__ __launch_bounds__(256) void ClearSlotKernel(uint4 *slot)
{
    slot[blockIdx.x * 256 + threadIdx.x] = uint4 { 0, 0, 0, 0 };
}

// Level 1 (or guard_mode 0): the plain kernel, nothing else on the stream.
// Level 2: the first launch takes a progress map (cleared only for the slot's first owner
// and every 255th after it: otherwise the generation tag is new); every launch (first or
// replay) carries the epoch current at enqueue time.
hipError_t HipGuardedCommand::Enqueue(HipQueue &q, bool replay)
{
    const bool level2 = q.Level() >= kPreemptLevelDeactivate;
    const bool guarded = guard_mode_ == 2 || (guard_mode_ != 0 && level2);

    XGuardArgs g;
    g.flag = q.Guard()->FlagDevPtr();
    g.done = nullptr;
    g.gen = 0;
    g.epoch = q.Guard()->Epoch();
    g.resume = replay ? 1u : 0u;
    g.flag_mask = q.Guard()->FlagMask();
    g.flushed = q.Guard()->FlushedDevPtr();

    if (guarded && level2) {
        if (slot_.done == nullptr) TakeSlot(q);   // a free one was seen to at submission
        if (slot_.needs_clear) {
            slot_.needs_clear = false;
            // a kernel, not hipMemsetAsync: a stream under capture records no memset node
            static_assert(GuardState::kSlotBytes % (16 * 256) == 0, "one 16-byte store per thread");
            ClearSlotKernel<<<dim3((unsigned)(GuardState::kSlotBytes / 16 / 256)), dim3(256), 0, q.Stream()>>>((uint4 *)slot_.done);
            hipError_t err = hipGetLastError();
            if (err != hipSuccess) return err;
        }
        g.done = slot_.done;
        g.gen = slot_.gen;
    }
    hipError_t err = PrepareLaunch(q);
    if (err != hipSuccess) return err;
    return LaunchKernel(q.Stream(), guarded, g);
}

void HipGuardedCommand::TakeSlot(HipQueue &q)
{
    XASSERT(n_wg_ <= GuardState::kMaxWorkGroups, "too many work-groups for a guarded command");
    guard_state_ = q.Guard();
    slot_ = guard_state_->AcquireSlot();
}

void HipGuardedCommand::PrepareOnSubmit(HipQueue &q)
{
    if (guard_mode_ != 0 && q.Level() >= kPreemptLevelDeactivate && slot_.done == nullptr) q.Guard()->ReserveSlots();
    ReserveOnSubmit(q);
}

// ---- HipQueue ----------------------------------------------------------------

HipQueue::HipQueue(hipStream_t stream): stream_(stream)
{
    HIP_ASSERT(hipGetDevice(&device_));
    hipDeviceProp_t prop;
    HIP_ASSERT(hipGetDeviceProperties(&prop, device_));
    xdevice_ = MakeDevice(kDeviceTypeGPU, MakePciId(prop.pciDomainID, prop.pciBusID, prop.pciDeviceID, 0));
    guard_ = std::make_shared<GuardState>(device_);
    scratch_ = std::make_shared<ScratchPool>(device_);
    marker_on_kernel_.store(GetEnvOption("XSCHED_HIP_MARKER_ON_KERNEL", true));
    HIP_ASSERT(hipStreamCreateWithFlags(&op_stream_, hipStreamNonBlocking)); // default priority
    // The entry point that allocates nothing needs the address of its static array on this
    // device; looked up here, at set-up, it never has to be looked up under a graph capture.
    ResolveNoAllocScratch(device_);
    ReportSignalPool();
    // Nothing of the application may still be running on the stream (hip_queue.cpp:35-36).
    HIP_ASSERT(hipStreamSynchronize(stream_));
}

HipQueue::~HipQueue()
{
    if (op_stream_) (void)hipStreamDestroy(op_stream_);
}

void HipQueue::OnXQueueCreate() { HIP_ASSERT(hipSetDevice(device_)); }

void HipQueue::OnPreemptLevelChange(XPreemptLevel level)
{
    XASSERT(level <= kPreemptLevelDeactivate, "unsupported level: %d", level);
    if (level >= kPreemptLevelDeactivate) {
        // the progress maps of the first guarded commands: allocated here, on the thread
        // that configures the queue, and not in front of the first launch
        DeviceScope scope(device_);
        guard_->ReserveSlots();
    }
    level_.store(level, std::memory_order_release);
}


ScratchPool::~ScratchPool()
{
    for (auto &buf : buffers_) (void)hipFree(buf.ptr);
}

void *ScratchPool::Allocate(size_t bytes)
{
    DeviceScope scope(device_);
    RelaxedCaptureScope relaxed;
    void *ptr = nullptr;
    if (hipMalloc(&ptr, bytes) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return ptr;
}

bool ScratchPool::HasFreeLocked(size_t bytes) const
{
    for (auto &buf : buffers_) {
        if (!buf.busy && buf.bytes >= bytes) return true;
    }
    return false;
}

void *ScratchPool::Acquire(size_t bytes)
{
    {
        std::lock_guard<std::mutex> lock(mtx_);
        Buffer *best = nullptr;
        for (auto &buf : buffers_) {
            if (!buf.busy && buf.bytes >= bytes && (best == nullptr || buf.bytes < best->bytes)) best = &buf;
        }
        if (best != nullptr) { best->busy = true; return best->ptr; }
    }
    // Nothing free (more commands in flight than Reserve() has seen submissions ahead of
    // them, or no Reserve() at all): allocate for this command.
    void *ptr = Allocate(bytes);
    if (ptr == nullptr) return nullptr;
    std::lock_guard<std::mutex> lock(mtx_);
    buffers_.push_back(Buffer { ptr, bytes, true });
    return ptr;
}

void ScratchPool::Reserve(size_t bytes)
{
    int count = 0;
    {
        std::lock_guard<std::mutex> lock(mtx_);
        if (HasFreeLocked(bytes)) return;
        // the first time: for this command and the ones that will be in flight with it
        count = buffers_.empty() ? kInitialBuffers : 1;
    }
    for (int i = 0; i < count; ++i) {
        void *ptr = Allocate(bytes);
        if (ptr == nullptr) return;
        std::lock_guard<std::mutex> lock(mtx_);
        buffers_.push_back(Buffer { ptr, bytes, false });
    }
}

void ScratchPool::Release(void *ptr)
{
    std::lock_guard<std::mutex> lock(mtx_);
    for (auto &buf : buffers_) {
        if (buf.ptr == ptr) { buf.busy = false; return; }
    }
}

size_t ScratchPool::Buffers()
{
    std::lock_guard<std::mutex> lock(mtx_);
    return buffers_.size();
}

size_t ScratchPool::Bytes()
{
    std::lock_guard<std::mutex> lock(mtx_);
    size_t bytes = 0;
    for (auto &buf : buffers_) bytes += buf.bytes;
    return bytes;
}

// On the submitting thread, before the XQueue takes any of its locks: a guarded command takes
// its progress map and scratch buffer here, so that a launch under those locks (the launch
// thread's, or the submitter's own direct launch) never waits for an allocation, and a
// scheduler's Suspend() never waits for such a launch.
void HipQueue::OnHwCommandSubmit(std::shared_ptr<HwCommand> hw_cmd)
{
    auto *guarded = dynamic_cast<HipGuardedCommand *>(hw_cmd.get());
    if (guarded == nullptr) return;
    DeviceScope scope(device_);
    guarded->PrepareOnSubmit(*this);
}

void HipQueue::Launch(std::shared_ptr<HwCommand> hw_cmd)
{
    auto *cmd = dynamic_cast<HipCommand *>(hw_cmd.get());
    XASSERT(cmd != nullptr, "hw_cmd is not a HipCommand");
    DeviceScope scope(device_);
    hipError_t err = cmd->LaunchWrapper(*this, false);
    XASSERT(err == hipSuccess, "failed to enqueue command: %d (%s)", (int)err, hipGetErrorString(err));
    n_launch.fetch_add(1, std::memory_order_relaxed);
    {
        std::lock_guard<std::mutex> lock(tail_mtx_);
        if (cmd->Synchronizable()) tail_marked_ = std::move(hw_cmd);
        else tail_marked_ = nullptr;
    }
}

// Waits for the marker of the newest command when that command carries one (recorded at
// launch, so it is on its way through the device's queue together with the command: a wait
// that begins later finds it done or nearly so). Otherwise a marker is recorded now, behind
// whatever the stream holds, and polled like any marker: every marker is one more packet
// the device's command processor works through in order, a few microseconds each, which a
// command that a submitter waits for at once should not pay twice. Asking the runtime about
// the stream itself (hipStreamQuery / hipStreamSynchronize) is several times slower when the
// newest operation on it is a kernel: the runtime then has to put a marker of its own behind
// the kernel first and hears of its completion through its signal thread.
void HipQueue::Synchronize()
{
    DeviceScope scope(device_);
    std::shared_ptr<HwCommand> tail;
    {
        std::lock_guard<std::mutex> lock(tail_mtx_);
        tail = tail_marked_;
    }
    if (tail != nullptr) {
        // (a replay re-records this marker behind the replayed work: still the stream's end;
        // an event-record command is waited for through the application's event, as its
        // XQueue waits for it as a batch marker: hip_command.h:197-219. Once its XQueue has
        // seen the command complete, the application is free to destroy that event, so a
        // completed command is not asked again: nothing newer is on the stream, or it would
        // be the tail.)
        if (tail->GetState() < kCommandStateCompleted) tail->Synchronize();
        std::lock_guard<std::mutex> lock(tail_mtx_);
        if (tail_marked_ == tail) tail_marked_ = nullptr;   // done: nothing of the stream is left to wait for, and the command is let go
        return;
    }
    RelaxedCaptureScope relaxed;
    hipEvent_t marker = EventPool::Instance().Pop(false);
    hipError_t err = hipEventRecord(marker, stream_);
    XASSERT(err == hipSuccess, "hipEventRecord failed: %d (%s)", (int)err, hipGetErrorString(err));
    if (!PollEvent(marker, SyncSpinMicros())) HIP_ASSERT(hipEventSynchronize(marker));
    EventPool::Instance().Push(marker);
}

void HipQueue::Deactivate()
{
    XASSERT(Level() >= kPreemptLevelDeactivate, "Deactivate() not supported on level-%d", Level());
    DeviceScope scope(device_);   // the copy variant of the flag write enqueues on this device's side stream
    guard_->Deactivate(op_stream_);
    n_deactivate.fetch_add(1, std::memory_order_relaxed);
}

// No device synchronisation and no read-back: flushed launches are still draining
// on the stream; the replays are queued behind them with the new epoch and sort
// out, work-group by work-group, what is left to do. Commands that cannot be
// flushed (plain kernels, copies) are never behind an in-flight flushable command,
// so they have run to completion and are skipped; marker-only commands (event
// records) that follow a replayed kernel are recorded again to keep their place.
void HipQueue::Reactivate(const CommandLog &log)
{
    XASSERT(Level() >= kPreemptLevelDeactivate, "Reactivate() not supported on level-%d", Level());
    // Whoever executes the scheduling operation calls this, possibly an application thread
    // in the middle of its own submission: its current device is put back afterwards.
    DeviceScope scope(device_);
    n_reactivate.fetch_add(1, std::memory_order_relaxed);
    // A replay carries the new epoch; the word must already show it, or the replay
    // would flush itself.
    guard_->WaitFlagWritten(op_stream_);

    bool replaying = false;
    for (auto &hw_cmd : log) {
        auto *cmd = dynamic_cast<HipCommand *>(hw_cmd.get());
        if (cmd == nullptr) continue;
        const bool flushable = cmd->ReplayOnReactivate();
        const bool idempotent = cmd->GetProps(kCommandPropertyIdempotent) != 0;
        if (!flushable && !(replaying && idempotent)) continue;
        replaying = true;
        hipError_t err = cmd->LaunchWrapper(*this, true);
        XASSERT(err == hipSuccess, "failed to replay command: %d (%s)", (int)err, hipGetErrorString(err));
        n_replay.fetch_add(1, std::memory_order_relaxed);
    }
}

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipQueueCreate(HwQueueHandle *hwq, void *stream)
{
    if (hwq == nullptr) {
        XWARN("HipQueueCreate failed: hwq is nullptr");
        return kXSchedErrorInvalidValue;
    }
    if (stream == nullptr) {
        XWARN("HipQueueCreate failed: the default stream is not supported");
        return kXSchedErrorNotSupported;
    }
    const HwQueueHandle h = (HwQueueHandle)stream;
    XResult res = HwQueueManager::Add(h, [&]() { return std::make_shared<HipQueue>((hipStream_t)stream); });
    if (res == kXSchedSuccess) *hwq = h;
    return res;
}

EXPORT_C_FUNC XResult HipQueueMarkEpochFlushed(HwQueueHandle hwq)
{
    auto q = std::dynamic_pointer_cast<HipQueue>(HwQueueManager::Get(hwq));
    if (q == nullptr) return kXSchedErrorNotFound;
    const uint32_t epoch = q->Guard()->Epoch();
    // behind whatever the stream still holds, as a flushed work-group's store would be
    hipError_t err = hipMemcpyAsync(q->Guard()->FlushedDevPtr(), &epoch, sizeof(epoch), hipMemcpyHostToDevice, q->Stream());
    if (err == hipSuccess) err = hipStreamSynchronize(q->Stream());
    return err == hipSuccess ? kXSchedSuccess : kXSchedErrorUnknown;
}

EXPORT_C_FUNC XResult HipQueueGetStats(HwQueueHandle hwq, uint64_t *out)
{
    if (out == nullptr) return kXSchedErrorInvalidValue;
    auto q = std::dynamic_pointer_cast<HipQueue>(HwQueueManager::Get(hwq));
    if (q == nullptr) return kXSchedErrorNotFound;
    out[0] = q->n_launch.load();
    out[1] = q->n_replay.load();
    out[2] = q->n_deactivate.load();
    out[3] = q->n_reactivate.load();
    out[4] = q->n_wait_polled.load();
    out[5] = q->n_wait_blocked.load();
    out[6] = q->Guard()->SlotsInUse();
    out[7] = q->Guard()->Epoch();
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipQueueSetMarkerOnKernel(HwQueueHandle hwq, int on)
{
    auto q = std::dynamic_pointer_cast<HipQueue>(HwQueueManager::Get(hwq));
    if (q == nullptr) return kXSchedErrorNotFound;
    q->SetMarkerOnKernel(on != 0);
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipQueueGetPoolStats(HwQueueHandle hwq, uint64_t *out)
{
    if (out == nullptr) return kXSchedErrorInvalidValue;
    auto q = std::dynamic_pointer_cast<HipQueue>(HwQueueManager::Get(hwq));
    if (q == nullptr) return kXSchedErrorNotFound;
    out[0] = q->Scratch()->Buffers();
    out[1] = q->Scratch()->Bytes();
    out[2] = q->Guard()->SlotsAllocated();
    out[3] = q->Guard()->SlotsInUse();
    return kXSchedSuccess;
}
