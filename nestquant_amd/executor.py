"""Per-rank executor: carries out level ops (upgrades to level 4, downgrades to level 2) on one rank's layers.

Takes the place of the reference's streaming/executor.py (`RankExecutor`, :38-165) behind the same public surface -- the
constructor arguments, `apply`, `poll`, `cancel_up`, `io_stats`, `busy`, and the counters and maps its callers and tests read
(`free`, `slot_of`, `pend`, `ops`, `wait_apply`, `n_landed`, ...): one pool of device slots (one refinement record each) for
all layers of the rank, one upgrade engine (stream_engine.Engine, native) on the rank's record file, one Mailbox per layer.

    ex = RankExecutor(rankfile, layers={L: (MoELayer, Mailbox, experts{E: resident expert})}, nslot, n_host, qd)
    ex.apply(ups, downs, sched)   issue ops without waiting; an upgrade with no free slot waits (first in, first out) for
                                  the next slot a downgrade frees; with wait_for_slot=False it is refused (sched.failed)
    ex.poll(sched)                after a layer call: ops the mailbox applied -> sched.landed / sched.released and slot
                                  release (issue=False: do not start waiting upgrades, e.g. during graph capture)
    ex.cancel_up(L, E)            best-effort skip of a stale upgrade (reference :120-135)
    ex.io_stats()                 I/O figures since the caller's previous call (reference :136-160)
    shadow=True                   every read, copy and mailbox op happens but the posted row stays the level-2 row

How it is built: every op is an `Op` object that moves through explicit states -- QUEUED (an upgrade waiting for a slot),
ISSUED (handed to the engine), WRITTEN (the engine reports the device writes done; the layer's mailbox has not applied the
row yet) -- and leaves the books when the mailbox's host counter shows its sequence number. Slots live in a `SlotPool`, the
addresses a layer's mailbox is written through in a `Port`, the rows of every expert in a `Rows` cache; the maps the
reference keeps side by side (its `ops`, `up_tag`, `wait_apply`, `pend`) are views derived from the op objects.

Invariants, as the reference's (:13-15): one outstanding op per expert; a slot is reused only after the level-2 row that
replaced it was applied; a failed read never posts its row, so its expert stays at level 2. A downgrade whose row copy the
engine reports as failed keeps its slot (the level-4 row is still live and points into it) and is posted again.

Left out (the reference's prefill-borrow and slot-lending extensions, :166-271, belong to its serving integration).
"""
import collections
import enum
from dataclasses import dataclass

import numpy as np
import torch

from . import p4rec
from .moe import entry, validate_row

CANCELLED_BELOW = -1e8            # an engine report with t_read at or below this: the op was dropped before it started
REPOST_LIMIT = 3                  # times a downgrade whose row copy failed is posted again before the failure is raised


class State(enum.Enum):
    QUEUED = 0        # upgrade waiting for a free slot (not yet known to the engine)
    ISSUED = 1        # in the engine: reading, copying, or queued there
    WRITTEN = 2       # device writes done, row staged and seq bumped; waiting for the layer's mailbox to apply it


@dataclass
class Op:
    key: tuple        # (layer, expert)
    level: int        # 4: upgrade, 2: downgrade
    state: State
    tag: int = 0      # engine tag (0 while QUEUED)
    seq: int = 0      # mailbox sequence number the op's row carries
    reposts: int = 0


class SlotPool:
    """fixed pool of device slots of `rb` bytes: a free stack and the owner of every taken slot"""

    def __init__(s, nslot, rb, device):
        s.mem = torch.empty(nslot, rb, dtype=torch.uint8, device=device)
        s.base, s.rb, s.n = s.mem.data_ptr(), rb, nslot
        s.free = list(range(nslot))[::-1]
        s.owner = {}                                              # key -> slot

    def take(s, key):
        slot = s.free.pop()
        s.owner[key] = slot
        return slot

    def give_back(s, key):
        s.free.append(s.owner.pop(key))

    def addr(s, slot):
        return s.base + slot * s.rb


class Port:
    """where one layer's mailbox is written: device addresses of its stage rows and sequence numbers, the host mirror of the
    applied counters, and the host's own sequence numbers"""

    def __init__(s, mailbox):
        s.mb = mailbox
        s.stage0, s.stride, s.seq0 = mailbox.stage.data_ptr(), mailbox.stage.stride(0) * 8, mailbox.seq.data_ptr()
        s.applied = mailbox.applied_host.numpy()

    def stage(s, E):
        return s.stage0 + s.stride * E

    def seq(s, E):
        return s.seq0 + 4 * E

    def next_seq(s, E):
        return s.mb.hseq[E] + 1


class Rows:
    """table rows of every expert, precomputed as numpy so that the serving thread spends no time building them: the
    level-2 row, and the level-4 row as (row with the record at address 0, per-word factor of the record's address)"""

    def __init__(s, layers, lay, probe_addr):
        s.lay, s.at = lay, {}
        for L, (layer, _, experts) in layers.items():
            for E, ex in experts.items():
                s.at[L, E] = s._build(layer, ex, probe_addr)

    def _build(s, layer, ex, probe_addr):
        keep = ex.signs
        if hasattr(ex, "sc"):
            ex.signs = ex.sc[2]                                   # the level-2 row carries the level-2 scale vector
        try:
            low = entry(ex, 2)
        finally:
            ex.signs = keep
        at0, at1 = p4rec.row(ex, s.lay, 0, entry), p4rec.row(ex, s.lay, 1, entry)
        validate_row(low, layer.H, layer.I)
        validate_row(at0 + (at1 - at0) * probe_addr, layer.H, layer.I)
        layer.rare_rows |= bool(low[4] or low[8] or low[19])
        return low.numpy().copy(), at0.numpy().copy(), (at1 - at0).numpy().copy()

    def low(s, key):
        return s.at[key][0]

    def high(s, key, addr):
        _, at0, factor = s.at[key]
        return at0 + factor * addr


class RankExecutor:
    def __init__(s, rf, layers, nslot, n_host=64, qd=8, device=None, wait_for_slot=True, shadow=False, alt_path=None, qd_alt=0, tier=None,
                 engine=None):
        """engine: an object with the Engine interface to use instead of `rf.engine(...)` (tests of the bookkeeping pass a
        host-only stand-in together with device="cpu"; serving code leaves it None)"""
        s.shadow, s.rf, s.lay, s.rb, s.layers, s.wait, s.nslot = shadow, rf, rf.lay, rf.rb, layers, wait_for_slot, nslot
        dev = torch.device(device) if isinstance(device, (str, torch.device)) else \
            torch.device("cuda", torch.cuda.current_device() if device is None else device)
        s.pool = SlotPool(nslot, s.rb, dev)
        s.eng = engine if engine is not None else rf.engine(n_host, qd, dev.index, alt_path=alt_path or "", qd_alt=qd_alt)
        s.port = {L: Port(mb) for L, (_, mb, _) in layers.items()}
        s.rows = Rows(layers, s.lay, s.pool.base or 256)
        s.by_key = {}                                             # (L, E) -> its one outstanding Op
        s.by_tag = {}                                             # engine tag -> Op, for ops in state ISSUED
        s.queue = []                             # keys of QUEUED upgrades, in arrival order
        s.count = collections.Counter()
        s.next_tag = 0
        s.lat = []                                                # end-to-end seconds of every landed upgrade
        s.recent = collections.deque(maxlen=4096)                 # (read seconds, copy seconds) of the latest upgrades
        s.marks = {}                                              # io_stats(): caller name -> counters at its previous call
        s.tier_n = s.eng.tier_load([rf.rec(L, E) for L, E in tier]) if tier else 0

    # ---- the reference's attribute surface, derived from the op objects: `ops`, `wait_apply` and `up_tag` are read-only views
    # built on every access (changing the returned dict changes nothing); `pend` is the live queue
    slots = property(lambda s: s.pool.mem)
    slot0 = property(lambda s: s.pool.base)
    free = property(lambda s: s.pool.free)
    slot_of = property(lambda s: s.pool.owner)
    pend = property(lambda s: s.queue)       # the live queue of upgrades waiting for a slot (callers may remove from it, as the reference's do)
    ops = property(lambda s: {t: (*o.key, o.level, o.seq) for t, o in s.by_tag.items()})
    wait_apply = property(lambda s: {o.key: (o.level, o.seq) for o in s.by_key.values() if o.state is State.WRITTEN})
    up_tag = property(lambda s: {o.key: t for t, o in s.by_tag.items() if o.level == 4})
    n_landed = property(lambda s: s.count["landed"])
    n_cancel = property(lambda s: s.count["cancelled"])
    n_refused = property(lambda s: s.count["refused"])
    n_failed = property(lambda s: s.count["failed"])
    n_waited = property(lambda s: s.count["waited"])

    def addr(s, slot):
        return s.pool.addr(slot)

    def busy(s):
        return bool(s.by_key)

    def quiet(s):
        """nothing in the engine and nothing waiting for a mailbox (upgrades may still wait for a slot)"""
        return all(o.state is State.QUEUED for o in s.by_key.values())

    def close(s):
        s.eng.close()

    # ---- issuing
    def _row(s, L, E, level, slot=None):
        key = (L, E)
        return s.rows.low(key) if level == 2 or s.shadow else s.rows.high(key, s.pool.addr(slot))

    def _to_engine(s, op):
        L, E = op.key
        port = s.port[L]
        s.next_tag += 1
        op.tag, op.seq, op.state = s.next_tag, port.next_seq(E), State.ISSUED
        s.by_tag[op.tag] = op
        if op.level == 4:
            slot = s.pool.owner[op.key]
            s.eng.upgrade(op.tag, s.rf.rec(L, E), s.pool.addr(slot), port.stage(E), s._row(L, E, 4, slot), port.seq(E), op.seq)
        else:
            s.eng.post(op.tag, port.stage(E), s._row(L, E, 2), port.seq(E), op.seq)

    @staticmethod
    def _tell(sched, what, L, E, **kw):
        if sched is None:
            return
        fn = getattr(sched, what, None)
        if fn is None and what == "cancelled":                    # a scheduler without that hook hears of a failure
            fn = sched.failed
        fn(L, E, **kw)

    def apply(s, ups, downs, sched=None):
        for key in map(tuple, downs):
            op = Op(key, 2, State.ISSUED)
            s.by_key[key] = op
            s._to_engine(op)
        for key in map(tuple, ups):
            if s.pool.free:
                s.pool.take(key)
                op = Op(key, 4, State.ISSUED)
                s.by_key[key] = op
                s._to_engine(op)
            elif s.wait:
                s.by_key[key] = Op(key, 4, State.QUEUED)
                s.queue.append(key)
                s.count["waited"] += 1
            else:
                s.count["refused"] += 1
                s._tell(sched, "failed", *key)

    # ---- progress
    def _engine_report(s, op, t_read, t_e2e, sched):
        """one finished engine op: cancelled, failed, or its device writes are done"""
        L, E = op.key
        if t_read <= CANCELLED_BELOW or t_read < 0:
            if op.level == 2:
                # the level-4 row is still live and points into the slot: keep slot and books, post the row again
                if op.reposts >= REPOST_LIMIT:
                    # raised by poll() once the whole batch of reports has been handled, so that no other report of the batch is
                    # lost; the op stays in by_key (the level-4 row is live and owns its slot: the expert takes no further op)
                    return f"the engine failed to post the level-2 row of layer {L} expert {E} {op.reposts + 1} times"
                op.reposts += 1
                s.count["reposted"] += 1
                s._to_engine(op)
                return
            cancelled = t_read <= CANCELLED_BELOW
            s.count["cancelled" if cancelled else "failed"] += 1
            s.pool.give_back(op.key)
            del s.by_key[op.key]
            if cancelled:
                s._tell(sched, "cancelled", L, E)
            else:
                s._tell(sched, "failed", L, E, read_error=True)   # the read failed: its row was never posted
            return
        s.port[L].mb.hseq[E] = op.seq
        op.state = State.WRITTEN
        if op.level == 4:
            s.count["landed"] += 1
            s.lat.append(t_e2e)
            s.recent.append((t_read, t_e2e - t_read))

    def _mailbox_applied(s, op, sched):
        L, E = op.key
        del s.by_key[op.key]
        if op.level == 4:
            s._tell(sched, "landed", L, E)
        else:
            s.pool.give_back(op.key)                              # only now: no kernel reads the slot through the old row any more
            s._tell(sched, "released", L, E)

    def poll(s, sched=None, issue=True):
        fatal = []
        for tag, _hit, t_read, t_e2e in s.eng.poll():
            why = s._engine_report(s.by_tag.pop(tag), t_read, t_e2e, sched)
            if why:
                fatal.append(why)
        for op in [o for o in s.by_key.values() if o.state is State.WRITTEN]:
            if s.port[op.key[0]].applied[op.key[1]] == op.seq:
                s._mailbox_applied(op, sched)
        while issue and s.queue and s.pool.free:
            op = s.by_key[s.queue.pop(0)]
            s.pool.take(op.key)
            s._to_engine(op)
        if fatal:
            raise RuntimeError("; ".join(fatal))

    def cancel_up(s, L, E, sched=None):
        """drop an upgrade of (L, E) that has not started: still waiting for a slot here -> dropped now (True, and
        sched.cancelled now); queued in the engine -> cancel requested (True; poll() reports it, or it completes normally
        if it had started); otherwise False"""
        op = s.by_key.get((L, E))
        if op is None or op.level != 4:
            return False
        if op.state is State.QUEUED:
            s.queue.remove(op.key)
            del s.by_key[op.key]
            s.count["cancelled"] += 1
            s._tell(sched, "cancelled", L, E)
            return True
        if op.state is State.ISSUED:
            s.eng.cancel(op.tag)
            return True
        return False

    # ---- reporting
    def io_stats(s, name="default"):
        """I/O figures over the interval since this caller's (name) previous io_stats() call (first call: since start)"""
        e = s.eng.stats()
        scalars = dict(landed=s.count["landed"], ssd=e["bytes_read"], tier=e["tier_bytes"], lru=e["host_hits"], tier_hits=e["tier_hits"],
                       upgrades=e["upgrades"])
        drives = {k: np.asarray(e[k], np.float64) for k in ("drive_bytes", "drive_reads", "drive_read_s")}
        before = s.marks.get(name)
        s.marks[name] = (e["now"], scalars, drives)
        if before is None:
            before = (e["now"] - 1e-9, dict.fromkeys(scalars, 0), {k: np.zeros_like(v) for k, v in drives.items()})
        dt = max(e["now"] - before[0], 1e-9)
        d = {k: scalars[k] - before[1][k] for k in scalars}
        dd = {k: drives[k] - before[2][k] for k in drives}
        gbps = lambda nbytes: nbytes / dt / 1e9
        share = lambda hits: hits / d["upgrades"] if d["upgrades"] > 0 else None
        pct = lambda a, q: float(np.percentile(a, q)) * 1e3
        out = dict(dt_s=dt, delivered_GBps=gbps(d["landed"] * s.rb), ssd_GBps=gbps(d["ssd"]), tier_GBps=gbps(d["tier"]),
                   drive_GBps=[gbps(b) for b in dd["drive_bytes"]],
                   drive_read_ms=[sec / n * 1e3 if n else None for sec, n in zip(dd["drive_read_s"], dd["drive_reads"])],
                   drive_inflight=list(e["drive_inflight"]), drive_qd=list(e["drive_qd"]), tier_recs=e["tier_recs"], tier_state=e["tier_state"],
                   tier_hit_share=share(d["tier_hits"]), host_lru_hit_share=share(d["lru"]),
                   eng_waiting=e["waiting"], eng_reading=e["reading"], eng_copying=e["copying"], slot_wait=len(s.queue),
                   ops_outstanding=len(s.by_tag), free_slots=len(s.pool.free), cancelled=s.count["cancelled"],
                   ssd_cum=int(scalars["ssd"]), tier_cum=int(scalars["tier"]), landed_cum=int(scalars["landed"]),
                   op_p50_ms=None, op_p99_ms=None)
        if s.recent:
            rc = np.array(s.recent)
            total = rc.sum(1)
            out.update(op_p50_ms=pct(total, 50), op_p99_ms=pct(total, 99), rd_p50_ms=pct(rc[:, 0], 50), rd_p99_ms=pct(rc[:, 0], 99),
                       cp_p50_ms=pct(rc[:, 1], 50), cp_p99_ms=pct(rc[:, 1], 99))
        return out

    def check_invariants(s, sched=None, max_bytes=None):
        """Slot-integrity probe after the reference's sm120/serve/nq_slotcheck.py:11-21; synchronises the device and
        reads records from the rank's file. Keys (L, E) in transit (any outstanding op) are skipped.
          B  slot bytes == the expert's record in the file          T  table row == the level-4 row built for the slot
          O  a level-4 row points into the pool at the slot its key owns (level-2 rows equal the level-2 row)
          K  slot_of injective, no owned slot in the free list, the free list without duplicates
          S  (with sched) scheduler state UP <=> key resident and not in transit
        max_bytes: compare at most this many leading bytes of each record (None = all). Raises AssertionError."""
        torch.cuda.synchronize(s.pool.mem.device)
        pool = s.pool
        owned = list(pool.owner.values())
        assert len(set(owned)) == len(owned), "K: two keys own one slot"
        assert not set(owned) & set(pool.free), "K: an owned slot is in the free list"
        assert len(set(pool.free)) == len(pool.free), "K: a slot is twice in the free list"
        lo, hi = pool.base, pool.base + pool.n * pool.rb
        n = s.rb if max_bytes is None else min(s.rb, max_bytes)
        with open(s.rf.path, "rb") as f:
            for L, (layer, _, experts) in s.layers.items():
                table = layer.table.cpu().numpy()
                for E in experts:
                    key = (L, E)
                    if key in s.by_key:
                        continue
                    slot = pool.owner.get(key)
                    if slot is None or s.shadow:
                        assert (table[E] == s.rows.low(key)).all(), f"T: row of {key} is not its level-2 row"
                    else:
                        assert (table[E] == s.rows.high(key, pool.addr(slot))).all(), f"T: row of {key} is not the level-4 row of slot {slot}"
                        for w in np.nonzero(s.rows.at[key][2])[0]:
                            a = int(table[E][w])
                            assert lo <= a < hi and (a - lo) // pool.rb == slot, f"O: word {w} of the row of {key} leaves slot {slot}"
                    if slot is not None:
                        f.seek(s.rf.rec(L, E) * s.rb)
                        rec = np.frombuffer(f.read(n), np.uint8)
                        assert (pool.mem[slot, :n].cpu().numpy() == rec).all(), f"B: slot {slot} differs from the record of {key}"
                    if sched is not None:
                        up = int(sched.state[sched.li[L], E]) == 2
                        assert up == (slot is not None), f"S: scheduler state of {key} is {int(sched.state[sched.li[L], E])}, slot {slot}"
