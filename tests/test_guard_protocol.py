"""The level-2 guard protocol under adversarial timing, on the CPU.

The device-side guard (include/xsched/hip/guard.h) takes its decisions in two plain functions
of include/xsched/hip/guard_args.h, xguard_entry_verdict and xguard_recheck_verdict. This test
compiles those two functions with gcc and drives them from a simulation of one queue's stream
in which everything the real system leaves to timing is decided by a seeded random scheduler:

  * the preempt word has several copies and the host rewrites them ONE AT A TIME, with device
    steps in between, so work-groups that read different copies disagree for a while;
  * work-groups of a launch run in any order, one step at a time (enter / look again / take
    effect / commit); a launch starts only when the one before it has left (stream order);
  * the host suspends (deactivation), resumes (replay of everything in its in-flight window
    with the new epoch, after all copies are written) and retires its window (when the stream
    has drained and no deactivation fell into the wait) at random moments.

Kernels as the library has them: one that updates in place at work-group granularity (the
guard's entry check, the short-array AXPY and user kernels), one whose long-lived waves walk
chunks (the AXPY's default grid: `flushed` looked at once per wave, the preempt word before
every chunk), one whose work-groups keep everything on chip until a final write and give up
in between (the GEMM), and one of two launches where the second needs every work-group of the
first (the histogram's counting and merge kernels).

Invariants: every work-group of every command takes effect exactly once; on each cell the
commands take effect in submission order (the kernels are in-place, so a later command that
ran ahead of the replay of an earlier one would read what has not been written); a merge
launch never runs with a partial missing; what the host retires has really been executed.
With the `flushed` word switched off in the simulation the same seeds DO break the order,
which is what that word is for."""
import ctypes
import os
import random
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Verdict(ctypes.Structure):
    _fields_ = [("run", ctypes.c_uint32), ("note_flush", ctypes.c_uint32)]


@pytest.fixture(scope="module")
def guard(tmp_path_factory):
    d = tmp_path_factory.mktemp("guard")
    src = d / "verdict.c"
    src.write_text('#include "xsched/hip/guard_args.h"\n'
                   'struct XGuardVerdict entry(uint32_t c, uint32_t f, uint32_t e, uint32_t r, uint32_t m, uint32_t t, uint32_t g)\n'
                   '{ return xguard_entry_verdict(c, f, e, r, m, t, g); }\n'
                   'struct XGuardVerdict recheck(uint32_t c, uint32_t e) { return xguard_recheck_verdict(c, e); }\n')
    so = d / "verdict.so"
    subprocess.run(["gcc", "-O1", "-shared", "-fPIC", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(so)], check=True)
    lib = ctypes.CDLL(str(so))
    lib.entry.restype = Verdict
    lib.entry.argtypes = [ctypes.c_uint32] * 7
    lib.recheck.restype = Verdict
    lib.recheck.argtypes = [ctypes.c_uint32] * 2
    return lib


NO_EPOCH = 0xFFFFFFFF


class Violation(Exception):
    pass


class Sim:
    """One queue: host state, the stream, the device memory the guard uses."""

    def __init__(self, lib, rnd, kinds, n_wg, n_copies, threshold, use_flushed_word=True):
        self.lib, self.rnd = lib, rnd
        self.kinds, self.n_wg, self.n_copies, self.threshold = kinds, n_wg, n_copies, threshold
        self.use_flushed_word = use_flushed_word
        # device memory
        self.copies = [0] * n_copies
        self.flushed = NO_EPOCH
        self.tags = {}            # (command, phase) -> [tag per work-group]
        self.partials = {}        # command -> set of counting work-groups whose partial is stored
        self.history = [[] for _ in range(n_wg)]   # per cell: commands that took effect, in order
        # host
        self.epoch = 0
        self.pending_copy_writes = []
        self.paused = False
        self.window = []          # commands launched and not retired
        self.next_cmd = 0
        self.stream = []          # launches: dict(cmd, phase, epoch, resume, state...)
        self.deactivated_since_drain_began = False

    # ---- host ------------------------------------------------------------------------
    def launch(self, cmd, resume):
        phases = ("count", "merge") if self.kinds[cmd] == "two_launches" else ("only",)
        for phase in phases:
            self.tags.setdefault((cmd, phase), [0] * self.n_wg)
            self.stream.append({"cmd": cmd, "phase": phase, "epoch": self.epoch, "resume": resume,
                                "wg": None})

    def host_actions(self):
        acts = []
        if not self.paused and self.next_cmd < len(self.kinds) and len(self.window) < self.threshold:
            acts.append("submit")
        if not self.paused and not self.pending_copy_writes:
            acts.append("suspend")
        if self.pending_copy_writes:
            acts.append("write_copy")
        if self.paused and not self.pending_copy_writes:
            acts.append("resume")
        if not self.paused and not self.stream and self.window:
            acts.append("retire")
        return acts

    def do_host(self, act):
        if act == "submit":
            self.window.append(self.next_cmd)
            self.launch(self.next_cmd, 0)
            self.next_cmd += 1
        elif act == "suspend":
            self.paused = True
            self.epoch += 1
            self.pending_copy_writes = list(range(self.n_copies))
        elif act == "write_copy":
            self.copies[self.pending_copy_writes.pop(0)] = self.epoch
        elif act == "resume":
            for cmd in self.window:           # the replay of the whole in-flight window
                self.launch(cmd, 1)
            self.paused = False
        elif act == "retire":
            # the stream has drained and the queue is running: what is retired must be done
            for cmd in self.window:
                for w in range(self.n_wg):
                    if self.history[w].count(cmd) != 1:
                        raise Violation(f"command {cmd} retired, cell {w} history {self.history[w]}")
            self.window = []

    # ---- device ------------------------------------------------------------------------
    def effect(self, cmd, w):
        h = self.history[w]
        if cmd in h:
            raise Violation(f"command {cmd} took effect twice on cell {w}")
        if h != list(range(cmd)):
            raise Violation(f"command {cmd} ran on cell {w} after {h}: an earlier command has not been applied yet")
        h.append(cmd)

    def read_flushed(self):
        return self.flushed if self.use_flushed_word else NO_EPOCH

    def entry(self, L, w):
        tag = self.tags[(L["cmd"], L["phase"])][w]
        v = self.lib.entry(self.copies[w % self.n_copies], self.read_flushed(), L["epoch"], L["resume"], 1, tag, L["cmd"] + 1)
        if v.note_flush:
            self.flushed = L["epoch"]
        return bool(v.run)

    def recheck(self, L, w):
        v = self.lib.recheck(self.copies[w % self.n_copies], L["epoch"])
        if v.note_flush:
            self.flushed = L["epoch"]
        return bool(v.run)

    def start_launch(self, L):
        kind = self.kinds[L["cmd"]]
        if kind == "waves" and L["phase"] == "only":
            # long-lived waves: wave v walks chunks v, v + W, ...; `flushed` is looked at once
            n_waves = max(1, self.n_wg // 3)
            L["wg"] = {v: {"pc": "wave_entry", "chunk": v} for v in range(n_waves)}
            L["n_waves"] = n_waves
        else:
            L["wg"] = {w: {"pc": "entry"} for w in range(self.n_wg)}

    def device_step(self):
        L = self.stream[0]
        if L["wg"] is None:
            self.start_launch(L)
        live = [w for w, st in L["wg"].items() if st["pc"] != "gone"]
        if not live:
            self.stream.pop(0)
            return
        w = self.rnd.choice(live)
        st = L["wg"][w]
        cmd, kind, phase = L["cmd"], self.kinds[L["cmd"]], L["phase"]
        tags = self.tags[(cmd, phase)]
        gen = cmd + 1

        if kind == "waves":
            if st["pc"] == "wave_entry":
                st["pc"] = "gone" if self.read_flushed() == L["epoch"] else "chunk"
            elif st["pc"] == "chunk":
                c = st["chunk"]
                if c >= self.n_wg:
                    st["pc"] = "gone"
                elif not self.recheck(L, w):           # the wave's own copy, before every chunk
                    st["pc"] = "gone"
                else:
                    if not (L["resume"] and tags[c] == gen):
                        self.effect(cmd, c)
                        tags[c] = gen                  # a chunk that has begun is finished and committed
                    st["chunk"] = c + L["n_waves"]
            return

        if st["pc"] == "entry":
            if phase == "merge":
                # needs every partial: not flushed in this epoch, every counting tag there, not done itself
                go = (self.read_flushed() != L["epoch"] and all(t == gen for t in self.tags[(cmd, "count")])
                      and not (L["resume"] and tags[w] == gen))
                st["pc"] = "effect" if go else "gone"
            else:
                st["pc"] = ("mid1" if kind in ("abandoning", "two_launches") else "effect") if self.entry(L, w) else "gone"
        elif st["pc"] in ("mid1", "mid2"):
            if not self.recheck(L, w):
                st["pc"] = "gone"                      # nothing written: abandons itself
            else:
                st["pc"] = "mid2" if st["pc"] == "mid1" else "effect"
        elif st["pc"] == "effect":
            if phase == "count":
                self.partials.setdefault(cmd, set()).add(w)
            elif phase == "merge":
                if self.partials.get(cmd, set()) != set(range(self.n_wg)):
                    raise Violation(f"merge of command {cmd} ran with partials {sorted(self.partials.get(cmd, []))}")
                self.effect(cmd, w)
            else:
                self.effect(cmd, w)
            st["pc"] = "commit"
        elif st["pc"] == "commit":
            tags[w] = gen
            st["pc"] = "gone"

    def run(self, max_steps=200000):
        for _ in range(max_steps):
            if (self.next_cmd == len(self.kinds) and not self.window and not self.stream and not self.paused
                    and not self.pending_copy_writes):
                break
            acts = self.host_actions()
            if self.stream:
                acts += ["device"] * 6          # the device makes progress most of the time
            if not acts:
                break
            act = self.rnd.choice(acts)
            # keep the host from suspending for ever: a suspend is a rare event
            if act == "suspend" and self.rnd.random() > 0.08:
                continue
            if act == "device":
                self.device_step()
            else:
                self.do_host(act)
        else:
            raise Violation("the simulation did not finish")
        for w in range(self.n_wg):
            if self.history[w] != list(range(len(self.kinds))):
                raise Violation(f"cell {w} ended with history {self.history[w]}")


def scenario(lib, seed, use_flushed_word=True, n_copies=None, threshold=None):
    rnd = random.Random(seed)
    kinds = [rnd.choice(["entry_only", "waves", "abandoning", "two_launches"]) for _ in range(rnd.randint(4, 10))]
    sim = Sim(lib, rnd, kinds, n_wg=rnd.randint(3, 9), n_copies=n_copies or rnd.choice([1, 2, 4]),
              threshold=threshold or rnd.choice([1, 2, 4]), use_flushed_word=use_flushed_word)
    sim.run()
    return sim


def test_verdicts_in_words(guard):
    e = lambda *a: (lambda v: (v.run, v.note_flush))(guard.entry(*a))
    # copy, flushed, epoch, resume, has_map, my_tag, gen
    assert e(5, NO_EPOCH, 5, 0, 1, 0, 3) == (1, 0)      # current, nothing flushed: run
    assert e(6, NO_EPOCH, 5, 0, 1, 0, 3) == (0, 1)      # the copy has moved on: leave and say so
    assert e(5, 5, 5, 0, 1, 0, 3) == (0, 0)             # an earlier launch of the epoch was flushed
    assert e(5, 4, 5, 0, 1, 0, 3) == (1, 0)             # a flush of an older epoch does not concern it
    assert e(5, NO_EPOCH, 5, 1, 1, 3, 3) == (0, 0)      # replay of a work-group that had committed
    assert e(5, NO_EPOCH, 5, 1, 1, 2, 3) == (1, 0)      # the tag is another command's
    assert e(5, NO_EPOCH, 5, 0, 1, 3, 3) == (1, 0)      # first launches do not look at tags
    assert e(5, NO_EPOCH, 5, 1, 0, 3, 3) == (1, 0)      # no progress map: nothing to skip by
    r = lambda *a: (lambda v: (v.run, v.note_flush))(guard.recheck(*a))
    assert r(7, 7) == (1, 0) and r(8, 7) == (0, 1)


@pytest.mark.parametrize("seed", range(300))
def test_protocol_holds_under_random_timing(guard, seed):
    sim = scenario(guard, seed)
    assert sim.next_cmd == len(sim.kinds) and not sim.window and not sim.stream


def test_without_the_flushed_word_the_same_timings_break_the_order(guard):
    """The control: the simulation does tell a protocol with the window open from one with it
    closed."""
    broken = 0
    for seed in range(300):
        # several copies and several launches in flight: what the word is there for
        scenario(guard, seed, n_copies=4, threshold=4)
        try:
            scenario(guard, seed, use_flushed_word=False, n_copies=4, threshold=4)
        except Violation:
            broken += 1
    assert broken >= 10, f"only {broken} of 300 seeds noticed the missing word"
