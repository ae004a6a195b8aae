"""Per-rank executor: carries out level ops (upgrades to level 4, downgrades to level 2) on one rank's layers.

Host-side mirror of the reference's streaming/executor.py (`RankExecutor`, :38-165): one pool of device slots (one
refinement record each) for all layers of the rank, one upgrade engine (stream_engine.Engine, native) on the rank's
record file, one Mailbox per layer whose apply() runs at the start of that layer's call.

    ex = RankExecutor(rankfile, layers={L: (MoELayer, Mailbox, experts{E: resident expert})}, nslot, n_host, qd)
    ex.apply(ups, downs, sched)   issue ops without waiting; an upgrade with no free slot waits (first in, first out) for
                                  the next slot a downgrade frees; with wait_for_slot=False it is refused (sched.failed)
    ex.poll(sched)                after a layer call: ops the mailbox applied -> sched.landed / sched.released and slot
                                  release (issue=False: do not start waiting upgrades, e.g. during graph capture)
    ex.cancel_up(L, E)            best-effort skip of a stale upgrade (reference :120-135)
    ex.io_stats()                 I/O figures since the caller's previous call (reference :136-160)
    shadow=True                   every read, copy and mailbox op happens but the posted row stays the level-2 row

Invariants, as the reference's (:13-15): one outstanding op per expert; a slot is reused only after the level-2 row that
replaced it was applied; a failed read never posts its row, so its expert stays at level 2.

Left out (the reference's prefill-borrow and slot-lending extensions, :166-271, belong to its serving integration).
"""
import collections

import numpy as np
import torch

from . import p4rec
from .moe import entry, validate_row


class RankExecutor:
    def __init__(s, rf, layers, nslot, n_host=64, qd=8, device=None, wait_for_slot=True, shadow=False, alt_path=None, qd_alt=0, tier=None,
                 engine=None):
        """engine: an object with the Engine interface to use instead of `rf.engine(...)` (tests of the bookkeeping pass a
        host-only stand-in together with device="cpu"; serving code leaves it None)"""
        s.shadow, s.rf, s.lay, s.rb, s.layers = shadow, rf, rf.lay, rf.rb, layers
        dev = torch.device(device) if isinstance(device, (str, torch.device)) else \
            torch.device("cuda", torch.cuda.current_device() if device is None else device)
        s.slots = torch.empty(nslot, s.rb, dtype=torch.uint8, device=dev)
        s.free = list(range(nslot))[::-1]
        s.slot_of = {}
        s.eng = engine if engine is not None else rf.engine(n_host, qd, dev.index, alt_path=alt_path or "", qd_alt=qd_alt)
        s.tag, s.ops = 0, {}                                  # tag -> (L, E, level, seq)
        s.up_tag, s.wait_apply, s.pend = {}, {}, []           # wait_apply: device writes done, not yet applied by the mailbox
        s.n_cancel = s.n_landed = s.n_refused = s.n_failed = s.n_waited = 0
        s.lat = []
        s.lat_w, s.lat_rc = collections.deque(maxlen=4096), collections.deque(maxlen=4096)
        s._prev = {}
        s.wait, s.nslot = wait_for_slot, nslot
        s.tier_n = s.eng.tier_load([rf.rec(L, E) for L, E in tier]) if tier else 0
        s.slot0 = s.slots.data_ptr()
        s.ah = {L: MB.applied_host.numpy() for L, (_, MB, _) in layers.items()}
        s.pp = {L: (MB.stage.data_ptr(), MB.stage.stride(0) * 8, MB.seq.data_ptr()) for L, (_, MB, _) in layers.items()}
        s.rc = {(L, E): s._mkrows(L, E) for L, (_, _, exs) in layers.items() for E in exs}

    def _mkrows(s, L, E):
        """(level-2 row, level-4 row with the record at address 0, per-word factor of the slot address) as numpy int64"""
        M, _, exs = s.layers[L]
        ex = exs[E]
        keep = ex.signs
        if hasattr(ex, "sc"):
            ex.signs = ex.sc[2]
        try:
            r2 = entry(ex, 2)
        finally:
            ex.signs = keep
        z, o = p4rec.row(ex, s.lay, 0, entry), p4rec.row(ex, s.lay, 1, entry)
        probe = z + (o - z) * (s.slot0 or 256)
        validate_row(r2, M.H, M.I)
        validate_row(probe, M.H, M.I)
        M.rare_rows |= bool(r2[4] or r2[8] or r2[19])
        return r2.numpy().copy(), z.numpy().copy(), (o - z).numpy().copy()

    def _row(s, L, E, level, slot=None):
        r2, z, m = s.rc[L, E]
        if level == 2 or s.shadow:
            return r2
        return z + m * (s.slot0 + slot * s.rb)

    def addr(s, slot):
        return s.slot0 + slot * s.rb

    def apply(s, ups, downs, sched=None):
        for L, E in downs:
            MB = s.layers[L][1]
            st, sb, sq = s.pp[L]
            s.tag += 1
            q = MB.hseq[E] + 1
            s.eng.post(s.tag, st + sb * E, s._row(L, E, 2), sq + 4 * E, q)
            s.ops[s.tag] = (L, E, 2, q)
        for L, E in ups:
            if not s.free:
                if s.wait:
                    s.pend.append((L, E)); s.n_waited += 1
                else:
                    s.n_refused += 1
                    if sched is not None:
                        sched.failed(L, E)
                continue
            MB = s.layers[L][1]
            st, sb, sq = s.pp[L]
            sl = s.free.pop()
            s.slot_of[L, E] = sl
            s.tag += 1
            q = MB.hseq[E] + 1
            s.eng.upgrade(s.tag, s.rf.rec(L, E), s.addr(sl), st + sb * E, s._row(L, E, 4, sl), sq + 4 * E, q)
            s.ops[s.tag] = (L, E, 4, q)
            s.up_tag[L, E] = s.tag

    def poll(s, sched=None, issue=True):
        for tag, hit, trd, te2e in s.eng.poll():
            L, E, level, q = s.ops.pop(tag)
            if level == 4:
                s.up_tag.pop((L, E), None)
            if trd <= -1e8:                                   # cancelled before it started
                s.n_cancel += 1
                s.free.append(s.slot_of.pop((L, E)))
                if sched is not None:
                    (getattr(sched, "cancelled", None) or sched.failed)(L, E)
                continue
            if trd < 0:                                       # the read failed: its row was never posted
                s.n_failed += 1
                s.free.append(s.slot_of.pop((L, E)))
                if sched is not None:
                    sched.failed(L, E, read_error=True)
                continue
            s.layers[L][1].hseq[E] = q
            s.wait_apply[L, E] = (level, q)
            if level == 4:
                s.lat.append(te2e); s.lat_w.append(te2e); s.lat_rc.append((trd, te2e - trd)); s.n_landed += 1
        for (L, E), (level, q) in list(s.wait_apply.items()):
            if s.ah[L][E] != q:
                continue
            del s.wait_apply[L, E]
            if level == 4:
                if sched is not None:
                    sched.landed(L, E)
            else:
                s.free.append(s.slot_of.pop((L, E)))
                if sched is not None:
                    sched.released(L, E)
        if issue and s.pend and s.free:
            n = min(len(s.pend), len(s.free))
            go, s.pend = s.pend[:n], s.pend[n:]
            s.apply(go, [], sched)

    def cancel_up(s, L, E, sched=None):
        """drop an upgrade of (L, E) that has not started: still waiting for a slot here -> dropped now (True, and
        sched.cancelled now); queued in the engine -> cancel requested (True; poll() reports it, or it completes normally
        if it had started); otherwise False"""
        k = (L, E)
        if k in s.pend:
            s.pend.remove(k); s.n_cancel += 1
            if sched is not None:
                (getattr(sched, "cancelled", None) or sched.failed)(L, E)
            return True
        t = s.up_tag.get(k)
        if t is None:
            return False
        s.eng.cancel(t)
        return True

    def io_stats(s, name="default"):
        """I/O figures over the interval since this caller's (name) previous io_stats() call (first call: since start)"""
        e = s.eng.stats()
        t = e["now"]
        c = dict(t=t, landed=s.n_landed, ssd=e["bytes_read"], tier=e["tier_bytes"], hits=e["host_hits"], th=e["tier_hits"], ups=e["upgrades"],
                 db=list(e["drive_bytes"]), dr=list(e["drive_reads"]), ds=list(e["drive_read_s"]))
        nd = len(c["db"])
        p = s._prev.get(name) or dict(t=t - 1e-9, landed=0, ssd=0, tier=0, hits=0, th=0, ups=0, db=[0] * nd, dr=[0] * nd, ds=[0.0] * nd)
        s._prev[name] = c
        dt = max(t - p["t"], 1e-9)
        dups = max(c["ups"] - p["ups"], 0)
        lat = np.array(s.lat_w) if s.lat_w else None
        ddr = [a - b for a, b in zip(c["dr"], p["dr"])]
        out = dict(dt_s=dt,
                   delivered_GBps=(c["landed"] - p["landed"]) * s.rb / dt / 1e9,
                   ssd_GBps=(c["ssd"] - p["ssd"]) / dt / 1e9,
                   drive_GBps=[(a - b) / dt / 1e9 for a, b in zip(c["db"], p["db"])],
                   drive_read_ms=[(a - b) / n * 1e3 if n else None for a, b, n in zip(c["ds"], p["ds"], ddr)],
                   drive_inflight=list(e["drive_inflight"]), drive_qd=list(e["drive_qd"]),
                   tier_GBps=(c["tier"] - p["tier"]) / dt / 1e9, tier_recs=e["tier_recs"], tier_state=e["tier_state"],
                   tier_hit_share=(c["th"] - p["th"]) / dups if dups else None,
                   host_lru_hit_share=(c["hits"] - p["hits"]) / dups if dups else None,
                   eng_waiting=e["waiting"], eng_reading=e["reading"], eng_copying=e["copying"], slot_wait=len(s.pend),
                   ops_outstanding=len(s.ops), free_slots=len(s.free), cancelled=s.n_cancel,
                   ssd_cum=int(c["ssd"]), tier_cum=int(c["tier"]), landed_cum=int(c["landed"]),
                   op_p50_ms=float(np.percentile(lat, 50)) * 1e3 if lat is not None else None,
                   op_p99_ms=float(np.percentile(lat, 99)) * 1e3 if lat is not None else None)
        if s.lat_rc:
            a = np.array(s.lat_rc) * 1e3
            out.update(rd_p50_ms=float(np.percentile(a[:, 0], 50)), rd_p99_ms=float(np.percentile(a[:, 0], 99)),
                       cp_p50_ms=float(np.percentile(a[:, 1], 50)), cp_p99_ms=float(np.percentile(a[:, 1], 99)))
        return out

    def check_invariants(s, sched=None, max_bytes=None):
        """Slot-integrity probe after the reference's sm120/serve/nq_slotcheck.py:11-21; synchronises the device and
        reads records from the rank's file. Keys (L, E) in transit (an op in flight or a row not yet applied) are skipped.
          B  slot bytes == the expert's record in the file          T  table row == the level-4 row built for the slot
          O  a level-4 row points into the pool at the slot its key owns (level-2 rows equal the level-2 row)
          K  slot_of injective, no owned slot in the free list, the free list without duplicates
          S  (with sched) scheduler state UP <=> key resident and not in transit
        max_bytes: compare at most this many leading bytes of each record (None = all). Raises AssertionError."""
        torch.cuda.synchronize(s.slots.device)
        transit = {(o[0], o[1]) for o in s.ops.values()} | set(s.wait_apply) | set(s.pend)
        owned = list(s.slot_of.values())
        assert len(set(owned)) == len(owned), "K: two keys own one slot"
        assert not set(owned) & set(s.free), "K: an owned slot is in the free list"
        assert len(set(s.free)) == len(s.free), "K: a slot is twice in the free list"
        lo, hi = s.slot0, s.slot0 + s.nslot * s.rb
        n = s.rb if max_bytes is None else min(s.rb, max_bytes)
        with open(s.rf.path, "rb") as f:
            for L, (M, _, exs) in s.layers.items():
                table = M.table.cpu().numpy()
                for E in exs:
                    k = (L, E)
                    if k in transit:
                        continue
                    r2, z, m = s.rc[k]
                    sl = s.slot_of.get(k)
                    if sl is None or s.shadow:
                        assert (table[E] == r2).all(), f"T: row of {k} is not its level-2 row"
                    else:
                        assert (table[E] == z + m * s.addr(sl)).all(), f"T: row of {k} is not the level-4 row of slot {sl}"
                        for w in np.nonzero(m)[0]:
                            a = int(table[E][w])
                            assert lo <= a < hi and (a - lo) // s.rb == sl, f"O: word {w} of the row of {k} leaves slot {sl}"
                    if sl is not None:
                        f.seek(s.rf.rec(L, E) * s.rb)
                        rec = np.frombuffer(f.read(n), np.uint8)
                        assert (s.slots[sl, :n].cpu().numpy() == rec).all(), f"B: slot {sl} differs from the record of {k}"
                    if sched is not None:
                        up = int(sched.state[sched.li[L], E]) == 2
                        assert up == (sl is not None), f"S: scheduler state of {k} is {int(sched.state[sched.li[L], E])}, slot {sl}"

    def busy(s):
        return bool(s.ops or s.wait_apply or s.pend)

    def quiet(s):
        return not s.ops and not s.wait_apply

    def close(s):
        s.eng.close()
