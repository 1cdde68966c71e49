// What the adapter offers to the interception shim beyond its C entry points.
#pragma once

#include <memory>

#include "xsched/preempt/hal/hw_command.h"

namespace xsched::hip
{

/// A command that waits, in the order of the queue it is submitted to, for `record` (an
/// event-record command, possibly submitted long ago, of any XQueue) to complete. Nothing
/// is enqueued on the stream. nullptr if `record` is not an event-record command.
/// (reference hip_command.h:236-254, shim.cpp:242-244)
std::shared_ptr<preempt::HwCommand> MakeRecordedEventWait(std::shared_ptr<preempt::HwCommand> record);

} // namespace xsched::hip
