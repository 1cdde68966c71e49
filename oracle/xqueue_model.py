"""ORACLE - test infrastructure only. Deterministic, single-threaded model of XSched's
progressive-launching loop: what the launch thread of one XQueue asks of its hardware
queue (launches, marker placement, command / queue synchronisations, deactivate and
reactivate calls) for a scripted sequence of submissions, device completions, suspends
and resumes. It restates, step for step,
    preempt/src/xqueue/launch_worker.cpp   (LaunchHwCommand :164-263, SyncAllWithLock
                                            :265-301, SyncCmdWithLock :303-368, WorkerLoop
                                            :86-162, Pause/Resume/ResumeAndDrop :33-64)
    preempt/src/xqueue/command_buffer.cpp  (Dequeue :39-97: the synthetic batch-sync then
                                            drain marker when the buffer runs empty)
    preempt/src/xqueue/async_xqueue.cpp    (Suspend :91-113, Resume :115-150)
of the reference. Pinned two ways: by the traces the reference's own build of these files
produces for fixed and seeded random scripts (tests/golden/xqueue_traces.json, written by
tests/golden/make_xqueue_traces.py from oracle/_ref/libxqueue_ref.so; compared call for
call in tests/test_xqueue_trace.py), and by facts read off the code
(tests/test_xqueue_model.py). Not pinned: which thread wins a race inside the reference's
launch thread when the scripts do not serialise it; the scripts here always do.

Trace tokens (what a hardware adapter observes):
    L<idx>     HwQueue::Launch of command idx      L<idx>*  ... with a completion marker
    CS<idx>    HwCommand::Synchronize on idx       QS       HwQueue::Synchronize
    D          HwQueue::Deactivate                 R[i,j,..] HwQueue::Reactivate(log)
The device is modelled by a watermark: complete(i) means every launch up to i has
finished; a deactivation makes every blocked synchronisation return early.
"""
from collections import deque

NONE, DEACTIVATABLE, IDEMPOTENT = 0, 1, 2


class XQueueModel:
    def __init__(self, threshold=16, batch=8, level=1):
        assert threshold >= batch
        self.threshold, self.batch, self.level = threshold, batch, level
        self.next_idx = 1
        self.pending = deque()          # ('hw', idx, props) | ('waitall',)
        self.tail = 'waitall'           # kind of the last enqueued command
        self.state = 'idle'             # XQueue state: idle / ready
        self.log = []                   # in flight: [idx, marker, props]
        self.last_marker = -1
        self.done = 0                   # device watermark
        self.paused = False
        self.pause_count = 0
        self.drop_idx = -1
        self.suspended = False
        self.completed = set()          # command indices in state Completed
        self.trace = []
        self.events = []                # 'ready' / 'idle' transitions
        self._cur = None                # command being processed by the worker
        self._wait = None               # ('cmd', idx, pause_cnt) | ('queue', upto, pause_cnt) | 'paused'
        self._phase = None
        self._flushed = False           # a deactivation happened since the wait began

    # ---- application side --------------------------------------------------------
    def submit(self, props=NONE, run=True):
        """run=False: only enqueue (the launch thread has not looked yet); call run() or a
        later action to let it proceed. Tests use this for a burst that is complete before
        the launch thread wakes up."""
        idx = self.next_idx
        self.next_idx += 1
        if self.state == 'idle':
            self.state = 'ready'
            self.events.append('ready')
        self.pending.append(('hw', idx, props))
        self.tail = 'hw'
        if run:
            self.run()
        return idx

    def burst(self, n, props=NONE):
        for _ in range(n):
            self.submit(props, run=False)
        self.run()

    def wait_all_marker(self):
        """XQueueWaitAll's enqueue step (command_buffer.cpp:127-155)."""
        if self.state == 'idle' or self.tail == 'waitall':
            return
        self.pending.append(('waitall',))
        self.tail = 'waitall'
        self.run()

    def complete(self, upto):
        self.done = max(self.done, upto)
        self.run()

    def suspend(self):
        if self.suspended:
            return
        self.suspended = True
        self.paused = True
        self.pause_count += 1
        if self.level >= 2:
            self.trace.append('D')
            self._flushed = True
        self.run()

    def resume(self, drop=False):
        if not self.suspended:
            return
        self.suspended = False
        if self.level == 1:
            self.paused = False
        elif not drop:
            self.trace.append('R[' + ','.join(str(e[0]) for e in self.log) + ']')
            self.paused = False
        else:
            self.trace.append('R[]')
            for item in self.pending:
                if item[0] == 'hw':
                    self.completed.add(item[1])
            self.pending.clear()
            self._retire_all()
            self.drop_idx = self.next_idx - 1
            self.paused = False
        self.run()

    # ---- launch thread -------------------------------------------------------------
    def in_flight(self):
        return [e[0] for e in self.log]

    def _retire_all(self):
        for e in self.log:
            self.completed.add(e[0])
        self.log = []

    def _retire_upto(self, idx):
        for e in self.log:
            if e[0] <= idx:
                self.completed.add(e[0])
        self.log = [e for e in self.log if e[0] > idx]

    def _markers(self):
        return [e[0] for e in self.log if e[1]]

    def _sync_cmd(self, idx):
        """SyncCmdWithLock: returns True when finished, False when blocked."""
        while True:
            w = self._wait
            inside = isinstance(w, tuple) and w[0] == 'cmd' and w[1] == idx
            if not inside:
                # Top of the loop (lock held): completed? paused? else enter the driver wait.
                if idx in self.completed:
                    return True
                if self.paused:
                    self._wait = 'paused'
                    return False
                self.trace.append(f'CS{idx}')
                self._wait = ('cmd', idx, self.pause_count)
                self._flushed = False
            # Inside HwCommand::Synchronize() (lock released): a pause does not interrupt
            # it; it is noticed only once the wait has returned.
            returned = self.done >= idx or self._flushed
            if not returned:
                return False
            cnt = self._wait[2]
            self._wait = None
            if cnt == self.pause_count:
                break
        self._retire_upto(idx)
        return True

    def _sync_all(self):
        while True:
            w = self._wait
            inside = isinstance(w, tuple) and w[0] == 'queue'
            if not inside:
                if self.paused:
                    self._wait = 'paused'
                    return False
                if not self.log:
                    return True
                self.trace.append('QS')
                self._wait = ('queue', self.log[-1][0], self.pause_count)
                self._flushed = False
            returned = self.done >= self._wait[1] or self._flushed
            if not returned:
                return False
            cnt = self._wait[2]
            self._wait = None
            if cnt == self.pause_count:
                break
        self._retire_all()
        return True

    def _sync(self, target):
        return self._sync_all() if target is None else self._sync_cmd(target)

    def _launch_steps(self, idx, props):
        """LaunchHwCommand as a resumable sequence of phases."""
        if self._phase is None:
            self._phase = 'deact'
            self._target = 'unset'
        if self._phase == 'deact':
            if self._target == 'unset':
                self._target = 'skip'
                if self.level >= 2 and props & (DEACTIVATABLE | IDEMPOTENT) == 0:
                    marker, has = None, False
                    for e in reversed(self.log):
                        if e[1]:
                            marker = e[0]
                        if e[2] & DEACTIVATABLE:
                            has = True
                            break
                    if has:
                        self._target = marker  # None -> whole queue
            if self._target != 'skip':
                if not self._sync(self._target):
                    return False
            self._phase, self._target = 'window', 'unset'
        if self._phase == 'window':
            if self._target == 'unset':
                if len(self.log) >= self.threshold:
                    front = self.log[0][0]
                    ms = [m for m in self._markers() if m >= front]
                    self._target = ms[0] if ms else None
                else:
                    self._target = 'pause-gate'
            if self._target == 'pause-gate':
                if self.paused:
                    self._wait = 'paused'
                    return False
                self._wait = None
            elif not self._sync(self._target):
                return False
            self._phase = 'launch'
        if idx <= self.drop_idx:
            self.completed.add(idx)
        else:
            marker = idx - self.last_marker >= self.batch
            self.trace.append(f'L{idx}*' if marker else f'L{idx}')
            self.log.append([idx, marker, props])
            if marker:
                self.last_marker = idx
        self._phase = None
        return True

    def run(self):
        """Advance the launch thread until it blocks or goes idle."""
        while True:
            if self._cur is None:
                if self.pending:
                    self._cur = self.pending.popleft()
                elif self.tail == 'waitall':
                    if self.state == 'ready':
                        self.state = 'idle'
                        self.events.append('idle')
                    return
                elif self.tail == 'batchsync':
                    self._cur, self.tail = ('waitall',), 'waitall'
                else:
                    self._cur, self.tail = ('batchsync',), 'batchsync'
            kind = self._cur[0]
            if kind == 'hw':
                if not self._launch_steps(self._cur[1], self._cur[2]):
                    return
            elif kind == 'waitall':
                if not self._sync_all():
                    return
            elif kind == 'batchsync':
                ms = self._markers()
                if self._phase is None:
                    self._phase = ('bs', ms[0] if ms else None)
                if self._phase[1] is not None and not self._sync_cmd(self._phase[1]):
                    return
                self._phase = None
            self._cur = None
