// Optional side interfaces of the plugin boundary. No counterpart in the reference.
//
// HwQueue and HwCommand keep exactly the virtual functions, in the order, of reference
// preempt/include/xsched/preempt/hal/{hw_queue,hw_command}.h, so an adapter built against
// those headers is never called past the end of its vtable. What this implementation asks
// of an adapter beyond that contract lives in the two classes below. An adapter that wants
// the behaviour inherits them NEXT TO HwQueue / HwCommand; the XQueue finds them with
// dynamic_cast and treats an object without them as the reference would.
#pragma once

namespace xsched::preempt
{

class HwQueueExtension
{
public:
    virtual ~HwQueueExtension() = default;

    /// True: Launch() and Synchronize() may be called from ANY thread that holds the
    /// XQueue's launch lock, not only from the launch thread. The XQueue then launches a
    /// command on the submitting thread when the launch thread is asleep and nothing is
    /// queued ahead of it, which takes the wake-up of that thread (tens of microseconds on
    /// an idle core) out of the submit-to-device path.
    virtual bool SupportDirectLaunch() { return false; }

    /// True when Deactivate() / Reactivate() concern nothing but launches that are in
    /// flight (a deactivation changes a word that only running kernels read). The XQueue
    /// then skips both for a queue that is suspended while it has nothing in flight: a
    /// scheduler that suspends every queue below the one that just became ready, busy or
    /// not, otherwise pays a device write per idle queue on every command, and a round of
    /// replays of nothing on every resume.
    virtual bool DeactivationConcernsInFlightWorkOnly() { return false; }
};

class HwCommandExtension
{
public:
    virtual ~HwCommandExtension() = default;

    /// See HwQueueExtension::SupportDirectLaunch(): true when this command may be launched
    /// on the submitting thread, i.e. its BeforeLaunch() never blocks.
    virtual bool DirectLaunchable() { return false; }

    /// True when the device is known to have completed this (synchronizable, launched)
    /// command; never blocks. A submitter that finds the window full asks the oldest marker
    /// this way before it gives the launch to the launch thread.
    virtual bool CompletedWithoutWaiting() { return false; }
};

} // namespace xsched::preempt
