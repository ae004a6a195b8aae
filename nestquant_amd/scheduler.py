"""Level policy: which experts are served at level 4. Fixed experts always are; a floating set follows decayed routing counts.

Host-side mirror of the reference's streaming/scheduler.py with its 'ema' rule (:62-118,160-189): the same constructor
arguments, `step(counts, ntok) -> (ups, downs)`, the executor's callbacks `landed / released / failed`, `kv_pressure(n)`
and `level()`, and the same decisions on the same counts (pinned by a trace of the reference's class,
tests/golden/sched_trace.json). Pure policy on the CPU: it sees the per-step routing counts (the kernels' `hits` export)
and returns level ops for executor.RankExecutor.apply. The learned predictors of the reference (its default,
gbdt_predictor*.py over LightGBM models) and its C++ host loop are not part of this build: any predictor other than
'ema' is refused.

Rule: score = counts decayed with a half-life of `half_life` tokens; every `refresh` tokens the floating target of a layer
that has seen counts becomes its `n_float` best non-fixed experts (a layer without counts keeps `floating_default`);
level-4 experts outside the target are downgraded at once; wanted level-2 experts are upgraded best score first while the
byte budget (cap_GBps at tok_per_s, at most burst_tokens of credit) and the slot pool allow, the rest wait; a step that
routes to more than big_frac of a layer's experts starts no upgrade; a failed read is not retried before retry_tokens.
"""
import numpy as np

IDLE, RISING, UP, FALLING = 0, 1, 2, 3        # floating expert: level 2 / upgrade in flight / level 4 / downgrade in flight


class Scheduler:
    def __init__(s, layers, fixed, floating_default, rec_bytes, NE=256, n_float=51, half_life=512, refresh=64, cap_GBps=6.0,
                 tok_per_s=111.0, big_frac=0.5, burst_tokens=64, slots=None, retry_tokens=None, predictor="ema"):
        if predictor not in (None, "ema"):
            raise ValueError(f"predictor {predictor!r}: only the 'ema' rule is built")
        s.layers = list(layers)
        s.li = {L: i for i, L in enumerate(s.layers)}
        nl = len(s.layers)
        s.NE, s.nf, s.R, s.rb, s.big, s.slots = NE, n_float, refresh, rec_bytes, big_frac, slots
        s.a = 0.5 ** (1 / half_life)
        s.fixed = np.zeros((nl, NE), bool)
        s.want = np.zeros((nl, NE), bool)
        for L in s.layers:
            i = s.li[L]
            s.fixed[i, list(fixed[L])] = True
            s.want[i, [e for e in floating_default[L] if not s.fixed[i, e]][:n_float]] = True
        s.score = np.zeros((nl, NE))
        s.state = np.zeros((nl, NE), np.int8)
        s.hold = np.zeros((nl, NE))                     # token count before which a failed read is not retried
        s.per_tok = cap_GBps * 1e9 / tok_per_s
        s.cap = s.per_tok * burst_tokens
        s.budget = 0.0
        s.retry = refresh if retry_tokens is None else retry_tokens
        s.tok, s.next_refresh = 0, refresh
        s.pin = None                                    # optional bool [layers, NE]: floating experts kept wanted while set
        s.predictor_name = "ema"
        s.stats = dict(ups=0, downs=0, deferred_steps=0, big_steps=0, bytes=0)

    def _refresh(s):
        seen = s.score.sum(1) > 0
        ranked = np.argsort(-np.where(s.fixed, -np.inf, s.score), 1, kind="stable")[:, :s.nf]
        target = np.zeros_like(s.want)
        np.put_along_axis(target, ranked, True, 1)
        s.want[seen] = target[seen]

    def step(s, counts, ntok=1, token_ids=None, new_request=False, sal=None):
        """counts [len(layers), NE]: routing hits of this model step (ntok tokens) -> (ups, downs) as lists of (L, E).
        token_ids, new_request and sal are accepted for the reference's call sites; the 'ema' rule does not use them."""
        c = np.asarray(counts, np.float64)
        s.score = s.score * s.a ** ntok + c
        s.tok += ntok
        s.budget = min(s.cap, s.budget + s.per_tok * ntok)
        if s.tok >= s.next_refresh:
            s.next_refresh += s.R
            s._refresh()
        if s.pin is not None:
            s.want |= s.pin & ~s.fixed
        downs = [(s.layers[i], int(e)) for i, e in zip(*np.nonzero((s.state == UP) & ~s.want))]
        for L, e in downs:
            s.state[s.li[L], e] = FALLING
        ups = []
        ready = (s.state == IDLE) & s.want & (s.hold <= s.tok)
        if ((c > 0).sum(1) > s.big * s.NE).any():
            s.stats["big_steps"] += 1
        elif ready.any():
            i, e = np.nonzero(ready)
            order = np.argsort(-s.score[i, e], kind="stable")
            n = int(s.budget // s.rb)
            if s.slots is not None:                     # slots are held by experts in flight, landed and draining
                n = max(0, min(n, s.slots - int((s.state > IDLE).sum())))
            if len(order) > n:
                s.stats["deferred_steps"] += 1
            for k in order[:n]:
                ups.append((s.layers[i[k]], int(e[k])))
                s.state[i[k], e[k]] = RISING
            s.budget -= len(ups) * s.rb
            s.stats["bytes"] += len(ups) * s.rb
        s.stats["ups"] += len(ups)
        s.stats["downs"] += len(downs)
        return ups, downs

    # executor feedback
    def landed(s, L, e):
        if s.state[s.li[L], e] == RISING:
            s.state[s.li[L], e] = UP

    def released(s, L, e):
        if s.state[s.li[L], e] == FALLING:
            s.state[s.li[L], e] = IDLE

    def failed(s, L, e, read_error=False):
        i = s.li[L]
        if s.state[i, e] == RISING:
            s.state[i, e] = IDLE
            if read_error:
                s.hold[i, e] = s.tok + s.retry
                s.stats["read_errors"] = s.stats.get("read_errors", 0) + 1

    cancelled = failed

    def kv_pressure(s, n):
        """downgrade the n lowest-score level-4 floating experts now; they stay unwanted until a refresh selects them again"""
        i, e = np.nonzero(s.state == UP)
        if not len(i):
            return []
        low = np.argsort(s.score[i, e], kind="stable")[:n]
        downs = [(s.layers[i[k]], int(e[k])) for k in low]
        for L, x in downs:
            s.state[s.li[L], x] = FALLING
            s.want[s.li[L], x] = False
        s.stats["downs"] += len(downs)
        return downs

    def level(s):
        """[len(layers), NE]: the level each expert is served at, as far as the scheduler knows"""
        return np.where(s.fixed | (s.state == UP), 4, 2)

    def close(s):
        pass
