"""Writes tests/golden/sched_trace.json by running the REFERENCE's level scheduler once, in the build container.

Run only where /root/reference exists:   python tests/golden/make_sched_fixture.py
It imports streaming/scheduler.py (numpy only; predictor='ema', so none of its optional predictor modules is loaded) and
drives it with seeded routing counts and the executor feedback a serving loop would give (upgrades land two steps after
they were issued, downgrades release one step later, some reads fail), storing the inputs' recipe and every step's
decisions. Nothing here is read at test time except the .json file it wrote.
"""
import json
import os
import sys

import numpy as np

REF = "/root/reference/streaming"
OUT = os.path.dirname(os.path.abspath(__file__))


def counts_stream(seed, nl, ne, steps):
    """per step: (counts [nl, ne], ntok). Popularity drifts, so the floating set has to move; a few steps are prefill-sized"""
    rng = np.random.default_rng(seed)
    pop = rng.permutation(ne).astype(np.float64)
    out = []
    for t in range(steps):
        if t % 40 == 39:
            pop = np.roll(pop, 17)
        ntok = 1 if t % 29 else 24
        p = 1.0 / (1.0 + pop) ** 1.1
        c = np.zeros((nl, ne))
        for i in range(nl):
            picks = rng.choice(ne, size=(ntok, 8), p=p / p.sum())
            np.add.at(c[i], picks.reshape(-1), 1)
        out.append((c, ntok))
    return out


def drive(S, stream, fail_every):
    """the feedback loop: ops issued at step t are answered at t + 2 (upgrades) / t + 1 (downgrades)"""
    trace, due, k = [], {}, 0
    for t, (c, ntok) in enumerate(stream):
        for kind, L, e in due.pop(t, []):
            if kind == "landed":
                S.landed(L, e)
            elif kind == "released":
                S.released(L, e)
            else:
                S.failed(L, e, read_error=(kind == "read_error"))
        ups, downs = S.step(c, ntok)
        extra = S.kv_pressure(3) if t == 150 else []
        for L, e in ups:
            k += 1
            kind = "landed" if k % fail_every else ("read_error" if k % (2 * fail_every) else "refused")
            due.setdefault(t + 2, []).append((kind, L, e))
        for L, e in downs + extra:
            due.setdefault(t + 1, []).append(("released", L, e))
        trace.append(dict(ups=[list(x) for x in ups], downs=[list(x) for x in downs], pressure=[list(x) for x in extra],
                          level4=int((S.level() == 4).sum()), budget=float(S.budget)))
    return trace


CASES = [dict(seed=1, layers=[3, 4, 9], NE=64, n_float=9, steps=260, fail_every=7, fixed=[0, 5, 6], default=[1, 2, 3, 4, 5, 7, 8, 9, 10, 11, 12],
              kw=dict(half_life=64, refresh=16, cap_GBps=0.5, tok_per_s=100.0, burst_tokens=8, slots=20, retry_tokens=24, big_frac=0.5)),
         dict(seed=2, layers=[5], NE=256, n_float=51, steps=200, fail_every=11, fixed=list(range(26)), default=list(range(20, 90)),
              kw=dict(slots=None))]


def main():
    sys.path.insert(0, REF)
    import scheduler as R
    out = []
    for case in CASES:
        Ls = case["layers"]
        S = R.Scheduler(Ls, {L: case["fixed"] for L in Ls}, {L: case["default"] for L in Ls}, 9592832, NE=case["NE"], n_float=case["n_float"],
                        predictor="ema", hostloop="py", **case["kw"])
        trace = drive(S, counts_stream(case["seed"], len(Ls), case["NE"], case["steps"]), case["fail_every"])
        out.append(dict(case=case, trace=trace, stats={k: int(v) for k, v in S.stats.items()}))
    with open(os.path.join(OUT, "sched_trace.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
