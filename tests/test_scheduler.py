"""The level policy (nestquant_amd/scheduler.py) makes the decisions of the reference's streaming/scheduler.py with its
'ema' rule: tests/golden/sched_trace.json holds, per step, the ups / downs / forced downgrades, the number of level-4
experts and the byte budget that the reference's class produced on seeded counts with executor feedback (landed,
released, refused, read errors); the counts and the feedback loop are regenerated here from the same recipe."""
import importlib.util
import json
import os

import numpy as np
import pytest

from nestquant_amd.scheduler import Scheduler

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_sched_fixture", os.path.join(HERE, "golden", "make_sched_fixture.py"))
FX = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(FX)          # its helpers only; the reference is imported inside its main(), which is not called

with open(os.path.join(HERE, "golden", "sched_trace.json")) as f:
    GOLD = json.load(f)


def build(case):
    Ls = case["layers"]
    return Scheduler(Ls, {L: case["fixed"] for L in Ls}, {L: case["default"] for L in Ls}, 9592832, NE=case["NE"], n_float=case["n_float"],
                     predictor="ema", **case["kw"])


@pytest.mark.parametrize("k", range(len(GOLD)))
def test_same_decisions_as_the_reference(k):
    case, want = GOLD[k]["case"], GOLD[k]["trace"]
    assert case == json.loads(json.dumps(FX.CASES[k])), "the recipe changed after the fixture was written"
    S = build(case)
    got = FX.drive(S, FX.counts_stream(case["seed"], len(case["layers"]), case["NE"], case["steps"]), case["fail_every"])
    for t, (g, w) in enumerate(zip(got, want)):
        assert g == w, f"step {t}"
    assert len(got) == len(want)
    assert {k_: int(v) for k_, v in S.stats.items()} == GOLD[k]["stats"]


def test_policy_properties():
    S = Scheduler([0], {0: [0, 1]}, {0: [1, 2, 3, 4]}, 1000, NE=16, n_float=3, half_life=8, refresh=4, cap_GBps=1e-6, tok_per_s=1.0,
                  burst_tokens=4, slots=2)
    assert S.want[0].nonzero()[0].tolist() == [2, 3, 4]                 # fixed experts are never floating; n_float caps the default
    assert (S.level()[0, :2] == 4).all() and (S.level()[0, 2:] == 2).all()
    c = np.zeros((1, 16)); c[0, [5, 6, 7]] = [3, 2, 1]
    ups, downs = S.step(c)                                               # budget: 1000 B per token = one record
    assert ups == [(0, 2)] and not downs
    ups2, _ = S.step(c)
    assert ups2 == [(0, 3)]
    assert S.step(c)[0] == []                                            # both slots taken
    S.landed(0, 2); S.failed(0, 3, read_error=True)
    assert S.level()[0, 2] == 4 and S.state[0, 3] == 0 and S.hold[0, 3] == S.tok + 4
    ups, downs = S.step(c)                                               # 4th token: refresh -> target {5, 6, 7}; 2 leaves
    assert downs == [(0, 2)] and ups == [(0, 5)]
    S.released(0, 2)
    assert S.state[0, 2] == 0 and S.level()[0, 2] == 2
    big = np.ones((1, 16))
    assert S.step(big)[0] == [] and S.stats["big_steps"] == 1            # a step touching more than half the experts upgrades nothing
    with pytest.raises(ValueError, match="ema"):
        Scheduler([0], {0: []}, {0: []}, 1000, predictor="gbdt")
