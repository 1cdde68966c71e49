#include <algorithm>
#include <utility>
#include <vector>

#include "xsched/protocol/names.h"

// Display names per enumerator. The strings are the ones XSched prints and
// parses (reference protocol/src/names.cpp:11-82); lookups by name ignore case.
namespace xsched::protocol
{

namespace
{

template <typename E>
using Table = std::vector<std::pair<E, std::string>>;

const std::string kUnknown = XSCHED_UNKNOWN_NAME;

std::string Lower(std::string s)
{
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return (char)tolower(c); });
    return s;
}

template <typename E>
const std::string &NameOf(const Table<E> &table, E key)
{
    for (auto &row : table) if (row.first == key) return row.second;
    return kUnknown;
}

template <typename E>
E KeyOf(const Table<E> &table, const std::string &name, E unknown)
{
    const std::string want = Lower(name);
    for (auto &row : table) if (Lower(row.second) == want) return row.first;
    return unknown;
}

const Table<XPlatform> &Platforms()
{
    static const Table<XPlatform> t {
        { kPlatformUnknown, kUnknown }, { kPlatformVPI, "VPI" }, { kPlatformCUDA, "CUDA" },
        { kPlatformCUDLA, "cuDLA" }, { kPlatformHIP, "HIP" }, { kPlatformAscend, "Ascend" },
        { kPlatformOpenCL, "OpenCL" }, { kPlatformLevelZero, "LevelZero" },
    };
    return t;
}

const Table<XDeviceType> &DeviceTypes()
{
    static const Table<XDeviceType> t {
        { kDeviceTypeUnknown, kUnknown }, { kDeviceTypeCPU, "CPU" }, { kDeviceTypeGPU, "GPU" },
        { kDeviceTypeNPU, "NPU" }, { kDeviceTypeFPGA, "FPGA" }, { kDeviceTypeASIC, "ASIC" },
    };
    return t;
}

const Table<XPreemptLevel> &Levels()
{
    static const Table<XPreemptLevel> t {
        { kPreemptLevelUnknown, kUnknown }, { kPreemptLevelBlock, "Block" },
        { kPreemptLevelDeactivate, "Deactivate" }, { kPreemptLevelInterrupt, "Interrupt" },
    };
    return t;
}

const Table<XSchedulerType> &Schedulers()
{
    static const Table<XSchedulerType> t {
        { kSchedulerUnknown, kUnknown },
        { kSchedulerAppManaged, XSCHED_SCHEDULER_NAME_APP },
        { kSchedulerLocal, XSCHED_SCHEDULER_NAME_LCL },
        { kSchedulerGlobal, XSCHED_SCHEDULER_NAME_GLB },
    };
    return t;
}

const Table<XPolicyType> &Policies()
{
    static const Table<XPolicyType> t {
        { kPolicyUnknown, kUnknown },
        { kPolicyHighestPriorityFirst, XSCHED_POLICY_NAME_HPF },
        { kPolicyHeterogeneousHighestPriorityFirst, XSCHED_POLICY_NAME_HHPF },
        { kPolicyCPUHighestPriorityFirst, XSCHED_POLICY_NAME_CHPF },
        { kPolicyUtilizationPartition, XSCHED_POLICY_NAME_UP },
        { kPolicyProcessUtilizationPartition, XSCHED_POLICY_NAME_PUP },
        { kPolicyStrictProcessUtilizationPartition, XSCHED_POLICY_NAME_SPUP },
        { kPolicyKEarliestDeadlineFirst, XSCHED_POLICY_NAME_KEDF },
        { kPolicyLaxity, XSCHED_POLICY_NAME_LAX },
        { kPolicyActiveWindowFirst, XSCHED_POLICY_NAME_AWF },
        { kPolicyCompletelyFairScheduler, XSCHED_POLICY_NAME_CFS },
        { kPolicyMultiLevelFeedbackQueue, XSCHED_POLICY_NAME_MLFQ },
    };
    return t;
}

} // namespace

XPlatform GetPlatform(const std::string &n) { return KeyOf(Platforms(), n, kPlatformUnknown); }
const std::string &GetPlatformName(XPlatform p) { return NameOf(Platforms(), p); }

XDeviceType GetDeviceType(const std::string &n) { return KeyOf(DeviceTypes(), n, kDeviceTypeUnknown); }
const std::string &GetDeviceTypeName(XDeviceType t) { return NameOf(DeviceTypes(), t); }

XPreemptLevel GetPreemptLevel(const std::string &n) { return KeyOf(Levels(), n, kPreemptLevelUnknown); }
const std::string &GetPreemptLevelName(XPreemptLevel l) { return NameOf(Levels(), l); }

XSchedulerType GetSchedulerType(const std::string &n) { return KeyOf(Schedulers(), n, kSchedulerUnknown); }
const std::string &GetSchedulerTypeName(XSchedulerType t) { return NameOf(Schedulers(), t); }

XPolicyType GetPolicyType(const std::string &n) { return KeyOf(Policies(), n, kPolicyUnknown); }
const std::string &GetPolicyTypeName(XPolicyType t) { return NameOf(Policies(), t); }

} // namespace xsched::protocol
