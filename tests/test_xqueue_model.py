"""Pins the launch-loop model (oracle/xqueue_model.py) on facts read off the reference's
code, so that a slip in the restatement (off-by-one in the marker rule, syncing the
newest instead of the oldest marker, retiring too much) fails here."""
from oracle.xqueue_model import DEACTIVATABLE, IDEMPOTENT, NONE, XQueueModel


def launches(m):
    return [t for t in m.trace if t.startswith('L')]


def test_marker_positions_closed_form():
    # idx - last >= batch with last = -1 initially: markers fall on batch-1, 2*batch-1, ...
    # (launch_worker.cpp:242-245, launch_worker.h:74). batch 4 -> 3,7,11; batch 8 -> 7,15.
    for thr, batch in [(8, 4), (16, 8), (4, 2), (1, 1), (6, 3)]:
        m = XQueueModel(thr, batch)
        for i in range(1, 40):
            m.submit()
            m.complete(i)          # the device keeps up: the window never fills
        marked = [int(t[1:-1]) for t in launches(m) if t.endswith('*')]
        assert marked == [i for i in range(1, 40) if (i + 1) % batch == 0]


def test_window_8_4_waits_for_oldest_marker():
    # threshold 8, batch 4, device stalled: 8 launches, then the launch thread waits on the
    # OLDEST marker at or after the log's front - idx 3 - (launch_worker.cpp:200-216).
    m = XQueueModel(8, 4)
    m.burst(20)
    assert m.trace == ['L1', 'L2', 'L3*', 'L4', 'L5', 'L6', 'L7*', 'L8', 'CS3']
    # marker 3 done: 1..3 retire, in flight 5, launches continue until 8 are in flight again
    m.complete(3)
    assert m.in_flight() == [4, 5, 6, 7, 8, 9, 10, 11]
    assert m.trace[9:] == ['L9', 'L10', 'L11*', 'CS7']
    m.complete(7)
    assert m.in_flight() == list(range(8, 16))     # oscillates between 4..5 and 8 in flight
    assert m.trace[-1] == 'CS11'


def test_drain_sequence_batch_sync_then_full_sync_then_idle():
    # empty buffer after a hardware command: one batch synchronisation on the oldest marker,
    # then a full queue synchronisation, then Idle (command_buffer.cpp:53-93).
    m = XQueueModel(8, 4)
    m.burst(5)
    assert m.trace == ['L1', 'L2', 'L3*', 'L4', 'L5', 'CS3']
    assert m.events == ['ready']
    m.complete(3)
    assert m.trace[-1] == 'QS' and m.in_flight() == [4, 5]
    m.complete(5)
    assert m.events == ['ready', 'idle'] and m.in_flight() == []
    # no marker in flight: the batch synchronisation is skipped (launch_worker.cpp:127-139)
    m2 = XQueueModel(8, 4)
    m2.burst(2)
    assert m2.trace == ['L1', 'L2', 'QS']


def test_threshold_1_batch_1_is_lock_step():
    # idx1: 1-(-1)=2 >= 1 -> marked; window full -> wait on it before launching 2
    m = XQueueModel(1, 1)
    m.burst(2)
    assert m.trace == ['L1*', 'CS1']
    m.complete(1)
    assert m.trace == ['L1*', 'CS1', 'L2*', 'CS2']


def test_level1_suspend_blocks_launches_and_keeps_log():
    m = XQueueModel(8, 4, level=1)
    m.burst(2)                                          # L1 L2, then the drain waits on the queue
    m.suspend()
    m.burst(3)
    assert launches(m) == ['L1', 'L2']                  # nothing launched while paused
    assert 'D' not in m.trace and 'R' not in ''.join(m.trace)
    m.resume()
    # Level 1 keeps the log across suspend/resume (async_xqueue.cpp:121-126): the drain is
    # still waiting for 1..2, the new commands stay pending behind it.
    assert launches(m) == ['L1', 'L2'] and m.in_flight() == [1, 2]
    m.complete(2)
    assert launches(m) == ['L1', 'L2', 'L3*', 'L4', 'L5']


def test_suspend_during_sync_is_retried_after_resume():
    # A pause while the launch thread sits in a driver wait: the wait's result is discarded
    # and repeated after the resume (launch_worker.cpp:284-291, 342-349).
    m = XQueueModel(4, 2, level=2)
    m.burst(6, DEACTIVATABLE)
    assert m.trace == ['L1*', 'L2', 'L3*', 'L4', 'CS1']
    m.suspend()                                         # flush: CS1 returns early
    assert m.trace[-1] == 'D' and m.in_flight() == [1, 2, 3, 4]
    m.resume()
    assert m.trace[-2:] == ['R[1,2,3,4]', 'CS1']        # same command, waited again
    m.complete(1)
    assert m.in_flight()[0] == 2


def test_level2_plain_command_drains_deactivatable_ones_first():
    # A command that is neither deactivatable nor idempotent waits for the in-flight
    # deactivatable commands (launch_worker.cpp:171-198): it syncs the earliest marker that
    # lies behind the newest deactivatable command, or the whole queue if there is none.
    m = XQueueModel(8, 4, level=2)
    m.submit(DEACTIVATABLE, run=False); m.submit(DEACTIVATABLE, run=False)
    m.submit(NONE)
    assert m.trace == ['L1', 'L2', 'QS']
    m.complete(2)
    assert m.trace == ['L1', 'L2', 'QS', 'L3*', 'CS3']
    # idempotent commands do not wait
    m = XQueueModel(8, 4, level=2)
    m.submit(DEACTIVATABLE, run=False); m.submit(IDEMPOTENT)
    assert m.trace[:2] == ['L1', 'L2']
    # with a marker behind the newest deactivatable command that marker is enough
    m = XQueueModel(8, 2, level=2)
    for _ in range(3):
        m.submit(DEACTIVATABLE, run=False)
    m.submit(NONE)
    assert m.trace == ['L1*', 'L2', 'L3*', 'CS3']
    # at level 1 nothing waits
    m = XQueueModel(8, 4, level=1)
    m.submit(DEACTIVATABLE, run=False); m.submit(NONE)
    assert launches(m) == ['L1', 'L2']


def test_resume_with_drop():
    m = XQueueModel(2, 1, level=2)
    m.burst(5, DEACTIVATABLE)
    m.suspend()
    m.resume(drop=True)
    assert m.trace[-1] == 'R[]' or m.trace[-2] == 'R[]'
    assert m.completed == {1, 2, 3, 4, 5} and m.in_flight() == []
    assert m.state == 'idle'


def test_pause_does_not_interrupt_a_driver_wait():
    # Level 1: the launch thread sits inside HwCommand::Synchronize() with its lock released.
    # A suspend + resume in the meantime changes nothing until the wait returns; then the
    # changed pause count makes it wait once more on the same command
    # (launch_worker.cpp:342-349) - visible to the adapter as a second Synchronize().
    m = XQueueModel(2, 1, level=1)
    m.burst(3)
    assert m.trace == ['L1*', 'L2*', 'CS1']
    m.suspend(); m.resume()
    assert m.trace == ['L1*', 'L2*', 'CS1']
    m.complete(1)
    assert m.trace == ['L1*', 'L2*', 'CS1', 'CS1', 'L3*', 'CS2']
