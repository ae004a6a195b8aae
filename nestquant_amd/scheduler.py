"""Level policy: which experts are served at level 4. Fixed experts always are; a floating set follows decayed routing counts.

Takes the place of the reference's streaming/scheduler.py with its 'ema' rule (:62-118,160-189): the same constructor
arguments, `step(counts, ntok) -> (ups, downs)`, the executor's callbacks `landed / released / failed / cancelled`,
`kv_pressure(n)` and `level()`, the arrays its callers read (`want`, `state`, `score`, `hold`, `fixed`, `pin`, `budget`,
`tok`, `stats`, `li`), and the same decisions on the same counts: tests/golden/sched_trace.json holds every step's ops, the
number of level-4 experts and the byte budget that the reference's class produced on seeded counts with executor feedback.
Pure policy on the CPU: it sees the per-step routing counts (the kernels' `hits` export) and returns level ops for
executor.RankExecutor.apply. The learned predictors of the reference (its default, gbdt_predictor*.py over LightGBM models)
and its C++ host loop are not part of this build: any predictor other than 'ema' is refused.

The rule, and the piece of this module that holds each part of it:
  DecayedCounts   score = routing counts decayed with a half-life of `half_life` tokens;
  FloatingSet     every `refresh` tokens the floating target of a layer that has seen counts becomes its `n_float` best
                  non-fixed experts (a layer without counts keeps `floating_default`);
  ByteBudget      upgrades cost one record each out of a budget that fills with cap_GBps at tok_per_s, holding at most
                  burst_tokens of credit;
  Scheduler.step  level-4 experts outside the target are downgraded at once; wanted level-2 experts are upgraded best score
                  first while the budget and the slot pool allow, the rest wait; a step that routes to more than big_frac of
                  a layer's experts starts no upgrade; a failed read is not retried before retry_tokens.
"""
import numpy as np

IDLE, RISING, UP, FALLING = 0, 1, 2, 3        # floating expert: level 2 / upgrade in flight / level 4 / downgrade in flight
# what an executor callback does to an expert's state: callback -> (state it applies to, state it leaves)
ON_FEEDBACK = {"landed": (RISING, UP), "released": (FALLING, IDLE), "failed": (RISING, IDLE)}


class ByteBudget:
    """bytes of upgrades that may start: fills per token, is capped at a burst, is spent per record"""

    def __init__(s, per_token, burst_tokens):
        s.per_token, s.cap, s.level = per_token, per_token * burst_tokens, 0.0

    def refill(s, ntok):
        s.level = min(s.cap, s.level + s.per_token * ntok)

    def records(s, rec_bytes):
        return int(s.level // rec_bytes)

    def spend(s, nbytes):
        s.level -= nbytes


class DecayedCounts:
    """exponentially decayed routing counts, one per (layer, expert)"""

    def __init__(s, shape, half_life):
        s.keep = 0.5 ** (1 / half_life)
        s.value = np.zeros(shape)

    def add(s, counts, ntok):
        s.value = s.value * s.keep ** ntok + counts


class FloatingSet:
    """the floating experts a layer wants at level 4: the default until the layer has counts, then its best n by score"""

    def __init__(s, fixed, default_of, n):
        s.n = n
        s.mask = np.zeros_like(fixed)
        for i, default in enumerate(default_of):
            s.mask[i, [e for e in default if not fixed[i, e]][:n]] = True

    def refresh(s, score, fixed):
        ranked = np.where(fixed, -np.inf, score)
        # position of every expert in its layer's order by falling score, equal scores by rising index
        place = np.argsort(np.argsort(-ranked, 1, kind="stable"), 1, kind="stable")
        seen = score.sum(1) > 0
        s.mask[seen] = (place < s.n)[seen]


class Scheduler:
    def __init__(s, layers, fixed, floating_default, rec_bytes, NE=256, n_float=51, half_life=512, refresh=64, cap_GBps=6.0,
                 tok_per_s=111.0, big_frac=0.5, burst_tokens=64, slots=None, retry_tokens=None, predictor="ema"):
        if predictor not in (None, "ema"):
            raise ValueError(f"predictor {predictor!r}: only the 'ema' rule is built")
        s.layers = list(layers)
        s.li = dict(zip(s.layers, range(len(s.layers))))          # layer id -> row of the arrays below
        shape = (len(s.layers), NE)
        s.NE, s.rec_bytes, s.big_frac, s.slots, s.refresh_every = NE, rec_bytes, big_frac, slots, refresh
        s.fixed = np.zeros(shape, bool)
        for row, L in enumerate(s.layers):
            s.fixed[row, sorted(fixed[L])] = True
        s.counts = DecayedCounts(shape, half_life)
        s.floating = FloatingSet(s.fixed, [floating_default[L] for L in s.layers], n_float)
        s.bytes = ByteBudget(cap_GBps * 1e9 / tok_per_s, burst_tokens)
        s.state = np.zeros(shape, np.int8)
        s.hold = np.zeros(shape)                        # token count before which a failed read is not retried
        s.retry = refresh if retry_tokens is None else retry_tokens
        s.tok, s.next_refresh = 0, refresh
        s.pin = None                                    # optional bool [layers, NE]: floating experts kept wanted while set
        s.predictor_name = "ema"
        s.stats = dict(ups=0, downs=0, deferred_steps=0, big_steps=0, bytes=0)

    # arrays and figures callers read under the reference's names
    want = property(lambda s: s.floating.mask, lambda s, v: setattr(s.floating, "mask", v))
    score = property(lambda s: s.counts.value, lambda s, v: setattr(s.counts, "value", v))
    budget = property(lambda s: s.bytes.level, lambda s, v: setattr(s.bytes, "level", v))

    def _keys(s, flat):
        """flat indices into [layers, NE] -> [(L, E)]"""
        li, e = np.unravel_index(flat, s.state.shape)
        return [(s.layers[i], int(x)) for i, x in zip(li, e)]

    def _to_falling(s, flat):
        s.state.flat[flat] = FALLING
        s.stats["downs"] += len(flat)
        return s._keys(flat)

    def _start_upgrades(s, hits):
        """wanted level-2 experts, best score first, as far as budget and slots reach"""
        ready = np.flatnonzero((s.state == IDLE) & s.floating.mask & (s.hold <= s.tok))
        if ((hits > 0).sum(1) > s.big_frac * s.NE).any():
            s.stats["big_steps"] += 1                   # a step that touches most of a layer (a prefill) says nothing about locality
            return []
        if not len(ready):
            return []
        room = s.bytes.records(s.rec_bytes)
        if s.slots is not None:                         # slots are held by experts in flight, landed and draining
            in_use = int(np.count_nonzero(s.state != IDLE))
            room = min(room, max(s.slots - in_use, 0))
        if len(ready) > room:
            s.stats["deferred_steps"] += 1
        go = ready[np.argsort(-s.counts.value.flat[ready], kind="stable")[:room]]
        s.state.flat[go] = RISING
        s.bytes.spend(len(go) * s.rec_bytes)
        s.stats["bytes"] += len(go) * s.rec_bytes
        s.stats["ups"] += len(go)
        return s._keys(go)

    def step(s, counts, ntok=1, token_ids=None, new_request=False, sal=None):
        """counts [len(layers), NE]: routing hits of this model step (ntok tokens) -> (ups, downs) as lists of (L, E).
        token_ids, new_request and sal are accepted for the reference's call sites; the 'ema' rule does not use them."""
        hits = np.asarray(counts, np.float64)
        s.counts.add(hits, ntok)
        s.tok += ntok
        s.bytes.refill(ntok)
        if s.tok >= s.next_refresh:
            s.next_refresh += s.refresh_every
            s.floating.refresh(s.counts.value, s.fixed)
        if s.pin is not None:
            s.floating.mask |= s.pin & ~s.fixed
        downs = s._to_falling(np.flatnonzero((s.state == UP) & ~s.floating.mask))
        return s._start_upgrades(hits), downs

    # executor feedback
    def _feedback(s, what, L, e):
        i = s.li[L]
        before, after = ON_FEEDBACK[what]
        if s.state[i, e] != before:
            return False
        s.state[i, e] = after
        return True

    def landed(s, L, e):
        s._feedback("landed", L, e)

    def released(s, L, e):
        s._feedback("released", L, e)

    def failed(s, L, e, read_error=False):
        if s._feedback("failed", L, e) and read_error:
            s.hold[s.li[L], e] = s.tok + s.retry
            s.stats["read_errors"] = s.stats.get("read_errors", 0) + 1

    cancelled = failed

    def kv_pressure(s, n):
        """downgrade the n lowest-score level-4 floating experts now; they stay unwanted until a refresh selects them again"""
        up = np.flatnonzero(s.state == UP)
        low = up[np.argsort(s.counts.value.flat[up], kind="stable")[:n]]
        s.floating.mask.flat[low] = False
        return s._to_falling(low)

    def level(s):
        """[len(layers), NE]: the level each expert is served at, as far as the scheduler knows"""
        return np.where(s.fixed | (s.state == UP), 4, 2)

    def close(s):
        pass
