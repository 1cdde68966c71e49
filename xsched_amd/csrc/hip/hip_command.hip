// Generic HIP commands: copies, fills, events, arbitrary kernels. None of them can
// be flushed; at level 2 the launch thread lets earlier flushable commands finish
// before it launches one of these (except the event commands, which write no
// memory and are tagged idempotent, as the reference's CUDA adapter does:
// platforms/cuda/hal/src/common/cuda_command.cpp:160-161).
#include <cstring>

#include "hip_hal.h"
#include "xsched/hip/hal.h"

using namespace xsched::preempt;

namespace xsched::hip
{

namespace
{

class HipMemcpyCommand final : public HipCommand
{
public:
    HipMemcpyCommand(void *dst, const void *src, size_t bytes, hipMemcpyKind kind)
        : dst_(dst), src_(src), bytes_(bytes), kind_(kind) {}
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    { return hipMemcpyAsync(dst_, src_, bytes_, kind_, q.Stream()); }
private:
    void *dst_; const void *src_; size_t bytes_; hipMemcpyKind kind_;
};

class HipMemsetCommand final : public HipCommand
{
public:
    HipMemsetCommand(void *dst, int value, size_t bytes): dst_(dst), value_(value), bytes_(bytes) {}
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    { return hipMemsetAsync(dst_, value_, bytes_, q.Stream()); }
private:
    void *dst_; int value_; size_t bytes_;
};

// Fills of 16- and 32-bit elements (reference hip_command.h:190-192).
class HipMemsetWideCommand final : public HipCommand
{
public:
    HipMemsetWideCommand(void *dst, uint32_t value, size_t count, uint32_t width)
        : dst_(dst), value_(value), count_(count), width_(width) {}
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    {
        if (width_ == 2) return hipMemsetD16Async((hipDeviceptr_t)dst_, (unsigned short)value_, count_, q.Stream());
        return hipMemsetD32Async((hipDeviceptr_t)dst_, (int)value_, count_, q.Stream());
    }
private:
    void *dst_; uint32_t value_; size_t count_; uint32_t width_;
};

// The user's event is the marker: always synchronizable (hip_command.h:197-219).
class HipEventRecordCommand final : public HipCommand
{
public:
    explicit HipEventRecordCommand(hipEvent_t event): HipCommand(kCommandPropertyIdempotent), event_(event) {}
    virtual void Synchronize() override { WaitForEvent(event_); }
    virtual bool Synchronizable() override { return true; }
    virtual bool EnableSynchronization() override { return true; }
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override { return hipEventRecord(event_, q.Stream()); }
private:
    hipEvent_t event_;
};

class HipEventWaitCommand final : public HipCommand
{
public:
    HipEventWaitCommand(hipEvent_t event, unsigned flags)
        : HipCommand(kCommandPropertyIdempotent), event_(event), flags_(flags) {}
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    { return hipStreamWaitEvent(q.Stream(), event_, flags_); }
private:
    hipEvent_t event_; unsigned flags_;
};

// Cross-queue ordering against an event-record COMMAND of another XQueue (what the
// interception shim builds for hipStreamWaitEvent on an event it has seen recorded:
// reference hip_command.h:236-254, hip_command.cpp:174-184, shim.cpp:216-246). The wait is
// on the host, in BeforeLaunch(), and on the record command's COMPLETION as the XQueue that
// owns it reports it, not on the raw event: after a level-2 flush the raw event signals
// although the work in front of it was only flushed, while the owning XQueue repeats that
// wait after the replay. Until the record command has been submitted there is nothing to
// wait on, so that comes first. Nothing is enqueued on the stream.
class HipRecordedEventWaitCommand final : public HipCommand
{
public:
    explicit HipRecordedEventWaitCommand(std::shared_ptr<HwCommand> record)
        : HipCommand(kCommandPropertyIdempotent), record_(std::move(record)) {}
    virtual void BeforeLaunch() override
    {
        record_->WaitUntil(kCommandStatePending);
        record_->Wait();
    }
    virtual bool DirectLaunchable() override { return false; } // BeforeLaunch() blocks
protected:
    virtual hipError_t Enqueue(HipQueue &, bool) override { return hipSuccess; }
private:
    const std::shared_ptr<HwCommand> record_;
};

// Arguments are copied at creation, so the caller's storage may go away before the
// launch thread gets to the command.
class HipKernelCommand final : public HipCommand
{
public:
    HipKernelCommand(const void *func, dim3 grid, dim3 block, void **args, const size_t *sizes,
                     size_t n_args, uint32_t shmem)
        : func_(func), grid_(grid), block_(block), shmem_(shmem)
    {
        size_t total = 0;
        for (size_t i = 0; i < n_args; ++i) total += ROUND_UP(sizes[i], 16);
        storage_.resize(total);
        arg_ptrs_.resize(n_args);
        size_t off = 0;
        for (size_t i = 0; i < n_args; ++i) {
            memcpy(storage_.data() + off, args[i], sizes[i]);
            arg_ptrs_[i] = storage_.data() + off;
            off += ROUND_UP(sizes[i], 16);
        }
    }
    virtual bool MarkerGoesWithKernel() const override { return true; }
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    {
        if (const hipEvent_t stop = TakeStopEvent()) {
            return hipExtLaunchKernel(func_, grid_, block_, arg_ptrs_.data(), shmem_, q.Stream(), nullptr, stop, 0);
        }
        return hipLaunchKernel(func_, grid_, block_, arg_ptrs_.data(), shmem_, q.Stream());
    }
private:
    const void *func_; dim3 grid_, block_; uint32_t shmem_;
    std::vector<char> storage_;
    std::vector<void *> arg_ptrs_;
};

// A kernel of a loaded module (hipFunction_t). The arguments arrive as ONE buffer in which
// every argument already sits at its offset of the kernel argument segment, the form
// hipModuleLaunchKernel takes through its `extra` list (reference hip_command.h:124-186 keeps
// the caller's parameter arrays instead and has to know HIP's internal structures for that:
// kernel_param.cpp:347-390).
class HipModuleKernelCommand final : public HipCommand
{
public:
    HipModuleKernelCommand(hipFunction_t func, dim3 grid, dim3 block, uint32_t shmem,
                           const void *packed, size_t bytes)
        : func_(func), grid_(grid), block_(block), shmem_(shmem)
        , storage_((const char *)packed, (const char *)packed + bytes) {}
    virtual bool MarkerGoesWithKernel() const override { return true; }
protected:
    virtual hipError_t Enqueue(HipQueue &q, bool) override
    {
        size_t bytes = storage_.size();
        void *extra[] = { HIP_LAUNCH_PARAM_BUFFER_POINTER, storage_.data(),
                          HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END };
        // The launch that takes a stop event counts work-items, in 32 bits per dimension.
        const uint64_t items[3] = { (uint64_t)grid_.x * block_.x, (uint64_t)grid_.y * block_.y, (uint64_t)grid_.z * block_.z };
        const bool fits = items[0] <= UINT32_MAX && items[1] <= UINT32_MAX && items[2] <= UINT32_MAX;
        if (const hipEvent_t stop = fits ? TakeStopEvent() : nullptr) {
            return hipExtModuleLaunchKernel(func_, (uint32_t)items[0], (uint32_t)items[1], (uint32_t)items[2],
                                            block_.x, block_.y, block_.z, shmem_, q.Stream(), nullptr, extra,
                                            nullptr, stop, 0);
        }
        return hipModuleLaunchKernel(func_, grid_.x, grid_.y, grid_.z, block_.x, block_.y, block_.z,
                                     shmem_, q.Stream(), nullptr, extra);
    }
private:
    hipFunction_t func_; dim3 grid_, block_; uint32_t shmem_;
    std::vector<char> storage_;
};

// A kernel of the caller's own with the guard of xsched/hip/guard.h compiled in. Its last
// parameter is an XGuardArgs; the caller's arguments in front of it are copied at creation,
// the guard arguments are appended at every launch (first or replay) as the queue then has
// them. This is what binary instrumentation gives every CUDA kernel in the reference
// (platforms/cuda/hal/src/level2/instrument.cpp:224-231, inject.cu:43-83); here the kernel's
// author writes the three guard lines and any kernel becomes flushable at level 2.
class HipUserGuardedCommand final : public HipGuardedCommand
{
public:
    HipUserGuardedCommand(const void *func, uint32_t n_wg, dim3 block, void **args, const size_t *sizes,
                          size_t n_args, uint32_t shmem)
        : HipGuardedCommand(n_wg, 1), func_(func), block_(block), shmem_(shmem)
    {
        size_t total = 0;
        for (size_t i = 0; i < n_args; ++i) total += ROUND_UP(sizes[i], 16);
        storage_.resize(total);
        arg_ptrs_.resize(n_args + 1);
        size_t off = 0;
        for (size_t i = 0; i < n_args; ++i) {
            memcpy(storage_.data() + off, args[i], sizes[i]);
            arg_ptrs_[i] = storage_.data() + off;
            off += ROUND_UP(sizes[i], 16);
        }
    }
protected:
    // The kernel has one variant: below level 2 the guard finds the preempt word equal to the
    // launch's epoch (nothing deactivates a level-1 queue) and no progress map.
    virtual hipError_t LaunchKernel(hipStream_t stream, bool, const XGuardArgs &g) override
    {
        guard_args_ = g;
        arg_ptrs_.back() = &guard_args_;
        if (const hipEvent_t stop = TakeStopEvent()) {
            return hipExtLaunchKernel(func_, dim3(n_wg_), block_, arg_ptrs_.data(), shmem_, stream, nullptr, stop, 0);
        }
        return hipLaunchKernel(func_, dim3(n_wg_), block_, arg_ptrs_.data(), shmem_, stream);
    }
private:
    const void *func_; dim3 block_; uint32_t shmem_;
    std::vector<char> storage_;
    std::vector<void *> arg_ptrs_;
    XGuardArgs guard_args_;
};

} // namespace

std::shared_ptr<HwCommand> MakeRecordedEventWait(std::shared_ptr<HwCommand> record)
{
    if (record == nullptr || dynamic_cast<HipEventRecordCommand *>(record.get()) == nullptr) return nullptr;
    return std::make_shared<HipRecordedEventWaitCommand>(std::move(record));
}

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipMemcpyCommandCreate(HwCommandHandle *cmd, void *dst, const void *src,
                                             size_t bytes, int kind)
{
    if (cmd == nullptr || kind < 0 || kind > (int)hipMemcpyDefault) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipMemcpyCommand>(dst, src, bytes, (hipMemcpyKind)kind));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipMemsetCommandCreate(HwCommandHandle *cmd, void *dst, int value, size_t bytes)
{
    if (cmd == nullptr) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipMemsetCommand>(dst, value, bytes));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipMemsetWideCommandCreate(HwCommandHandle *cmd, void *dst, uint32_t value,
                                                 size_t count, uint32_t width_bytes)
{
    if (cmd == nullptr || (width_bytes != 2 && width_bytes != 4)) return kXSchedErrorInvalidValue;
    if (((uintptr_t)dst & (width_bytes - 1)) != 0) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipMemsetWideCommand>(dst, value, count, width_bytes));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipGuardedKernelCommandCreate(HwCommandHandle *cmd, const void *host_func,
                                                    uint32_t n_workgroups,
                                                    uint32_t bx, uint32_t by, uint32_t bz,
                                                    void **args, const size_t *arg_sizes, size_t n_args,
                                                    uint32_t shared_mem_bytes)
{
    if (cmd == nullptr || host_func == nullptr || (n_args != 0 && (args == nullptr || arg_sizes == nullptr))) {
        return kXSchedErrorInvalidValue;
    }
    if (n_workgroups == 0 || n_workgroups > GuardState::kMaxWorkGroups) return kXSchedErrorInvalidValue;
    if (bx == 0 || by == 0 || bz == 0 || (uint64_t)bx * by * bz > 1024) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipUserGuardedCommand>(
        host_func, n_workgroups, dim3(bx, by, bz), args, arg_sizes, n_args, shared_mem_bytes));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipModuleKernelCommandCreate(HwCommandHandle *cmd, void *function,
                                                   uint32_t gx, uint32_t gy, uint32_t gz,
                                                   uint32_t bx, uint32_t by, uint32_t bz,
                                                   uint32_t shared_mem_bytes,
                                                   const void *packed_args, size_t bytes)
{
    if (cmd == nullptr || function == nullptr || (bytes != 0 && packed_args == nullptr)) return kXSchedErrorInvalidValue;
    if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0 ||
        (uint64_t)bx * by * bz > 1024) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipModuleKernelCommand>(
        (hipFunction_t)function, dim3(gx, gy, gz), dim3(bx, by, bz), shared_mem_bytes, packed_args, bytes));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipEventRecordCommandCreate(HwCommandHandle *cmd, void *event)
{
    if (cmd == nullptr || event == nullptr) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipEventRecordCommand>((hipEvent_t)event));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipEventWaitCommandCreate(HwCommandHandle *cmd, void *event, uint32_t flags)
{
    if (cmd == nullptr || event == nullptr) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipEventWaitCommand>((hipEvent_t)event, flags));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipRecordedEventWaitCommandCreate(HwCommandHandle *cmd, HwCommandHandle record_cmd)
{
    if (cmd == nullptr) return kXSchedErrorInvalidValue;
    auto record = HwCommandManager::Get(record_cmd);
    if (record == nullptr) return kXSchedErrorNotFound;
    if (dynamic_cast<HipEventRecordCommand *>(record.get()) == nullptr) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipRecordedEventWaitCommand>(std::move(record)));
    return kXSchedSuccess;
}

EXPORT_C_FUNC XResult HipKernelCommandCreate(HwCommandHandle *cmd, const void *host_func,
                                             uint32_t gx, uint32_t gy, uint32_t gz,
                                             uint32_t bx, uint32_t by, uint32_t bz,
                                             void **args, const size_t *arg_sizes, size_t n_args,
                                             uint32_t shared_mem_bytes)
{
    if (cmd == nullptr || host_func == nullptr || (n_args != 0 && (args == nullptr || arg_sizes == nullptr))) {
        return kXSchedErrorInvalidValue;
    }
    if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0 ||
        (uint64_t)bx * by * bz > 1024) return kXSchedErrorInvalidValue;
    *cmd = HwCommandManager::Add(std::make_shared<HipKernelCommand>(
        host_func, dim3(gx, gy, gz), dim3(bx, by, bz), args, arg_sizes, n_args, shared_mem_bytes));
    return kXSchedSuccess;
}
