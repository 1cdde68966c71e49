"""Launch-loop parity. The reference's own XQueue core, compiled in this container and
driven over a recording hardware queue, wrote tests/golden/xqueue_traces.json: for fixed and
seeded random scripts of bursts, device progress, suspends and resumes at both preemption
levels, the calls it makes on its adapter (launches, marker placement, synchronisation
targets, deactivate / reactivate with the replayed log) and the queue state after every
action. The shipped core (libpreempt.so), driven the same way, must reproduce those traces
call for call, and so must the launch-loop model in oracle/xqueue_model.py."""
import json
import os

import pytest

import xqueue_trace_driver as drv
from oracle import xqueue_model
from oracle.xqueue_model import XQueueModel

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "xqueue_traces.json")) as f:
    GOLDEN = json.load(f)


@pytest.fixture(scope="module")
def product(xs):
    if not os.path.exists(drv.PROBE_LIB):
        pytest.fail("oracle/libxqueue_probe.so missing: run __graft_entry__.build()")
    return drv.Core.product()


def test_property_constants_agree(xs):
    assert (drv.NONE, drv.DEACTIVATABLE, drv.IDEMPOTENT) == \
        (xqueue_model.NONE, xqueue_model.DEACTIVATABLE, xqueue_model.IDEMPOTENT) == (0, 1, 2)


def test_fixture_scripts_are_the_scripts_in_the_tree():
    """The fixture's inputs are regenerated from the seeds, so a change of the script
    generator cannot silently detach the tests from the fixture."""
    for name, (thr, batch, level, actions) in drv.fixed_scripts().items():
        rec = GOLDEN[name]
        assert (rec["threshold"], rec["batch"], rec["level"]) == (thr, batch, level)
        assert [s["action"] for s in rec["steps"]] == actions
    for name in GOLDEN:
        if name.startswith("random_"):
            thr, batch, level, actions = drv.random_script(int(name.split("_")[1]), XQueueModel)
            rec = GOLDEN[name]
            assert (rec["threshold"], rec["batch"], rec["level"]) == (thr, batch, level)
            assert [s["action"] for s in rec["steps"]] == actions


@pytest.mark.parametrize("name", sorted(GOLDEN))
def test_model_matches_reference_traces(name):
    rec = GOLDEN[name]
    model = XQueueModel(rec["threshold"], rec["batch"], rec["level"])
    for i, step in enumerate(rec["steps"]):
        drv.apply_model(model, step["action"])
        want = rec["trace"][:step["trace_len"]]
        assert model.trace == want, f"{name} step {i} {step['action']}\n model {model.trace}\n ref   {want}"
        assert model.state == step["state"], f"{name} step {i}: state"


@pytest.mark.parametrize("name", sorted(GOLDEN))
def test_shipped_core_matches_reference_traces(product, name):
    rec = GOLDEN[name]
    s = drv.Session(product, rec["threshold"], rec["batch"], rec["level"])
    try:
        for i, step in enumerate(rec["steps"]):
            s.apply(step["action"])
            want = rec["trace"][:step["trace_len"]]
            got = s.settle(want)
            assert got == want, f"{name} step {i} {step['action']}\n got {got}\n ref {want}"
            assert s.state() == step["state"], f"{name} step {i}: state"
    finally:
        s.close(drv.last_index([st["action"] for st in rec["steps"]]))


@pytest.mark.skipif(not os.path.exists(drv.REF_LIB), reason="reference build not present")
@pytest.mark.parametrize("seed", range(100, 106))
def test_live_reference_matches_model_and_shipped_core(product, seed):
    """Where the reference build is present: fresh seeds, three-way."""
    ref = drv.Core.reference()
    thr, batch, level, actions = drv.random_script(seed, XQueueModel)
    model = XQueueModel(thr, batch, level)
    a, b = drv.Session(ref, thr, batch, level), drv.Session(product, thr, batch, level)
    try:
        for i, act in enumerate(actions):
            a.apply(act); b.apply(act); drv.apply_model(model, act)
            want = a.settle()
            assert model.trace == want, f"seed {seed} step {i} {act}: model vs reference"
            assert b.settle(want) == want, f"seed {seed} step {i} {act}: shipped vs reference"
            assert a.state() == b.state() == model.state
    finally:
        a.close(drv.last_index(actions)); b.close(drv.last_index(actions))
