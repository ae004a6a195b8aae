"""The record upgrade engine (csrc/nq_stream.hip through its C ABI) and the per-rank executor on top of it.

Engine checks follow the reference's streaming/smoke_fault.py (every op completes, a failed op's seq is never written, a
landed op's slot bytes equal the file's) on a synthetic record file; the executor check follows streaming/smoke_stream.py
(a layer served through upgrades / downgrades equals the layer whose table holds the applied levels) on repacked shards."""
import os
import time

import numpy as np
import pytest
import torch

from nestquant_amd import moe as M, nqload, repack, resident
from nestquant_amd.executor import RankExecutor
from nestquant_amd.stream_engine import Engine, RankFile
from tests.shards import synth_layer, write_layer

pytestmark = pytest.mark.gpu
DEV = "cuda"
RB = 64 * 1024


def record_file(tmp_path, n, name="rec.bin", seed=5):
    data = np.random.default_rng(seed).integers(0, 256, n * RB, dtype=np.uint8)
    path = str(tmp_path / name)
    data.tofile(path)
    return path, torch.from_numpy(data).view(n, RB)


class Bench:
    """device memory the ops write to: a slot, a stage row and a seq word per op"""

    def __init__(s, n):
        s.slots = torch.zeros(n, RB, dtype=torch.uint8, device=DEV)
        s.stage = torch.zeros(n, 20, dtype=torch.int64, device=DEV)
        s.seq = torch.zeros(n, dtype=torch.int32, device=DEV)

    def upgrade(s, eng, i, rec, tag=None, seq=None):
        eng.upgrade(i if tag is None else tag, rec, s.slots[i].data_ptr(), s.stage[i].data_ptr(), torch.full((20,), i + 1, dtype=torch.int64),
                    s.seq.data_ptr() + 4 * i, i + 1 if seq is None else seq)


def drain(eng, n, limit=60.0):
    done, t0 = {}, time.time()
    while len(done) < n and time.time() - t0 < limit:
        for tag, hit, trd, te2e in eng.poll():
            assert tag not in done
            done[tag] = (hit, trd, te2e)
        time.sleep(0.001)
    assert len(done) == n, f"{len(done)} of {n} ops completed"
    return done


def test_upgrades_land_in_order_with_the_file_bytes_and_cache_hits(tmp_path):
    n = 24
    path, data = record_file(tmp_path, 40)
    recs = [int(r) for r in np.random.default_rng(0).choice(40, n, replace=False)]
    b = Bench(2 * n)
    eng = Engine(path, RB, 32, 4, 0)
    try:
        for i, r in enumerate(recs):
            b.upgrade(eng, i, r)
        done = drain(eng, n)
        assert all(trd >= 0 and te2e >= trd and not hit for hit, trd, te2e in done.values())
        torch.cuda.synchronize()
        assert torch.equal(b.slots[:n].cpu(), data[recs])
        assert b.seq[:n].tolist() == list(range(1, n + 1))
        assert torch.equal(b.stage[:n].cpu(), torch.arange(1, n + 1).view(n, 1).expand(n, 20))
        # the same records again: all still held by the 32 host entries, so no drive read
        for i, r in enumerate(recs):
            b.upgrade(eng, n + i, r)
        again = drain(eng, n)
        assert all(hit for hit, _, _ in again.values())
        torch.cuda.synchronize()
        assert torch.equal(b.slots[n:].cpu(), data[recs])
        st = eng.stats()
        assert (st["upgrades"], st["host_hits"], st["bytes_read"], st["drive_reads"]) == (2 * n, n, n * RB, [n])
        assert st["posts"] == st["queued"] == st["reading"] == st["copying"] == st["waiting"] == 0
    finally:
        eng.close()
    with pytest.raises(RuntimeError):
        eng.poll()


def test_more_records_than_host_entries_replaces_the_least_recently_used(tmp_path):
    path, data = record_file(tmp_path, 12)
    b = Bench(16)
    eng = Engine(path, RB, 4, 2, 0)
    try:
        order = [0, 1, 2, 3, 0, 4, 0, 1]            # 4 entries: reading 4 replaces record 1 (0 was used again), so 1 is read twice
        hits = []
        for i, r in enumerate(order):
            b.upgrade(eng, i, r)
            hits.append(drain(eng, 1)[i][0])
        assert hits == [False, False, False, False, True, False, True, False]
        torch.cuda.synchronize()
        assert torch.equal(b.slots[:len(order)].cpu(), data[order])
    finally:
        eng.close()


def test_row_only_ops_between_upgrades_of_one_expert(tmp_path):
    path, data = record_file(tmp_path, 4)
    b = Bench(1)
    eng = Engine(path, RB, 4, 2, 0)
    try:
        # upgrade, downgrade, upgrade of the same expert, one outstanding op at a time as the executor keeps it (ops start in
        # arrival order, but an upgrade's writes follow its read, so the caller orders the ops of one expert)
        for tag, (rec, val) in enumerate([(2, 11), (None, 12), (3, 13)]):
            row = torch.full((20,), val, dtype=torch.int64)
            if rec is None:
                eng.post(tag, b.stage[0].data_ptr(), row, b.seq.data_ptr(), val)
            else:
                eng.upgrade(tag, rec, b.slots[0].data_ptr(), b.stage[0].data_ptr(), row, b.seq.data_ptr(), val)
            hit, trd, te2e = drain(eng, 1)[tag]
            assert (trd == 0.0) == (rec is None) and te2e >= trd        # a row-only op has no read time
            torch.cuda.synchronize()
            assert int(b.seq[0]) == val and b.stage[0].tolist() == [val] * 20
            assert torch.equal(b.slots[0].cpu(), data[3 if tag == 2 else 2])
        assert eng.stats()["posts"] == 1
        with pytest.raises(RuntimeError, match="row"):
            eng.post(9, b.stage[0].data_ptr(), torch.zeros(19, dtype=torch.int64), b.seq.data_ptr(), 1)
    finally:
        eng.close()


def test_failed_reads_never_write_their_row(tmp_path):
    n = 40
    path, data = record_file(tmp_path, n)
    b = Bench(n)
    eng = Engine(path, RB, 8, 4, 0)
    try:
        eng.set_fault(fail_ppm=500000)
        for i in range(n):
            b.upgrade(eng, i, i)
        done = drain(eng, n)
        torch.cuda.synchronize()
        ok = [t for t, (_, trd, _) in done.items() if trd >= 0]
        bad = [t for t, (_, trd, _) in done.items() if trd < 0]
        assert len(ok) >= 5 and len(bad) >= 5 and eng.stats()["fault_injected"] == len(bad)
        assert all(done[t][2] == -1.0 and not done[t][0] for t in bad)
        sq = b.seq.cpu()
        assert all(int(sq[t]) == 0 for t in bad) and all(int(sq[t]) == t + 1 for t in ok)
        assert not b.stage[bad].any() and not b.slots[bad].any()
        assert torch.equal(b.slots[ok].cpu(), data[ok])
    finally:
        eng.close()


def test_a_record_beyond_the_end_of_the_file_fails_cleanly(tmp_path):
    path, data = record_file(tmp_path, 4)
    b = Bench(2)
    eng = Engine(path, RB, 4, 2, 0)
    try:
        b.upgrade(eng, 0, 7)                                         # short read (0 bytes)
        b.upgrade(eng, 1, 1)
        done = drain(eng, 2)
        assert done[0][1] == -1.0 and done[0][2] == -1.0 and done[1][1] >= 0
        torch.cuda.synchronize()
        assert b.seq.tolist() == [0, 2] and torch.equal(b.slots[1].cpu(), data[1])
    finally:
        eng.close()


def test_a_slow_drive_spaces_reads_and_waiting_ops_can_be_cancelled(tmp_path):
    n = 8
    path, data = record_file(tmp_path, n)
    b = Bench(n)
    eng = Engine(path, RB, 8, 4, 0)
    try:
        eng.set_fault(read_ms=50.0)
        t0 = time.time()
        for i in range(n):
            b.upgrade(eng, i, i)
        time.sleep(0.02)
        eng.cancel(6); eng.cancel(7); eng.cancel(0)                   # 0 has started: completes normally
        done = drain(eng, n)
        dt = time.time() - t0
        assert dt >= 0.05 * (n - 3) * 0.9, dt
        assert done[6][1] == done[6][2] == -1e9 and done[7][1] == -1e9 and done[0][1] >= 0
        torch.cuda.synchronize()
        assert b.seq.tolist() == [1, 2, 3, 4, 5, 6, 0, 0]
        assert eng.stats()["cancelled"] == 2 and not b.slots[6:].any()
    finally:
        eng.close()


def test_ram_tier_serves_its_records_without_the_drive_and_can_be_dropped(tmp_path):
    path, data = record_file(tmp_path, 16)
    b = Bench(12)
    eng = Engine(path, RB, 4, 2, 0)
    try:
        assert eng.tier_load([3, 5, 9, 11]) == 4
        with pytest.raises(RuntimeError, match="tier"):
            eng.tier_load([1])
        for i, r in enumerate([3, 5, 9, 11]):
            b.upgrade(eng, i, r)
        done = drain(eng, 4)
        st = eng.stats()
        assert all(h for h, _, _ in done.values()) and st["tier_hits"] == 4 and st["tier_bytes"] == 4 * RB and st["bytes_read"] == 0
        assert st["tier_state"] == 1 and st["tier_recs"] == 4
        b.upgrade(eng, 4, 2)                                          # not in the tier: from the drive
        assert not drain(eng, 1)[4][0]
        eng.tier_drop()
        t0 = time.time()
        while eng.stats()["tier_state"] != 3 and time.time() - t0 < 10:
            time.sleep(0.002)
        assert eng.stats()["tier_state"] == 3 and eng.stats()["tier_recs"] == 0
        b.upgrade(eng, 5, 9)                                          # a former tier record now comes from the drive
        assert not drain(eng, 1)[5][0]
        torch.cuda.synchronize()
        assert torch.equal(b.slots[:6].cpu(), data[[3, 5, 9, 11, 2, 9]])
    finally:
        eng.close()


def test_two_drives_share_the_reads(tmp_path):
    n = 32
    path, data = record_file(tmp_path, n)
    alt, _ = record_file(tmp_path, n, name="copy.bin")
    b = Bench(n)
    eng = Engine(path, RB, 16, 2, 0, alt_path=alt, qd_alt=3)
    try:
        for i in range(n):
            b.upgrade(eng, i, i)
        drain(eng, n)
        torch.cuda.synchronize()
        st = eng.stats()
        assert st["drives"] == 2 and st["drive_qd"] == [2, 3] and sum(st["drive_reads"]) == n and st["drive_inflight"] == [0, 0]
        assert sum(st["drive_bytes"]) == n * RB == st["bytes_read"]
        assert torch.equal(b.slots.cpu(), data)
    finally:
        eng.close()
    short = str(tmp_path / "short.bin")
    open(short, "wb").write(b"\0" * RB)
    with pytest.raises(RuntimeError, match="size differs"):
        Engine(path, RB, 16, 2, 0, alt_path=short)


def test_close_with_ops_still_queued_returns_and_later_calls_raise(tmp_path):
    path, data = record_file(tmp_path, 16)
    b = Bench(16)
    eng = Engine(path, RB, 4, 2, 0)
    eng.set_fault(read_ms=200.0)                                      # at most two reads start before close()
    for i in range(16):
        b.upgrade(eng, i, i)
    time.sleep(0.01)
    t0 = time.time()
    eng.close()
    assert time.time() - t0 < 5.0
    eng.close()                                                       # a second close is a no-op
    torch.cuda.synchronize()
    sq = b.seq.cpu()
    landed = [i for i in range(16) if int(sq[i])]
    assert len(landed) <= 2 and all(int(sq[i]) == i + 1 and torch.equal(b.slots[i].cpu(), data[i]) for i in landed)
    for call in (eng.poll, eng.stats, lambda: eng.cancel(1), lambda: b.upgrade(eng, 0, 0)):
        with pytest.raises(RuntimeError, match="closed"):
            call()


def test_uploads_from_pinned_memory_on_an_engine_without_a_file():
    src = torch.randint(0, 256, (3, RB), dtype=torch.uint8).pin_memory()
    b = Bench(2)
    eng = Engine("", 0, 0, 4, 0)
    try:
        row = torch.full((20,), 7, dtype=torch.int64)
        # three spans into one slot, out of order and of different sizes, then row and seq
        spans = [(src[0].data_ptr(), b.slots[0].data_ptr() + 4096, 8192), (src[1].data_ptr() + 512, b.slots[0].data_ptr(), 4096),
                 (src[2].data_ptr(), b.slots[0].data_ptr() + 32768, RB - 32768)]
        eng.upload(1, spans, b.stage[0].data_ptr(), row, b.seq.data_ptr(), 5)
        eng.post(2, b.stage[1].data_ptr(), row * 2, b.seq.data_ptr() + 4, 9)
        done = drain(eng, 2)
        assert not done[1][0] and done[1][1] == 0.0 and done[1][2] >= 0
        torch.cuda.synchronize()
        got = b.slots[0].cpu()
        assert torch.equal(got[4096:12288], src[0][:8192]) and torch.equal(got[:4096], src[1][512:4608])
        assert torch.equal(got[32768:], src[2][:RB - 32768]) and not got[12288:32768].any()
        assert b.seq.tolist() == [5, 9] and b.stage[0].tolist() == [7] * 20 and b.stage[1].tolist() == [14] * 20
        st = eng.stats()
        assert (st["uploads"], st["upload_bytes"], st["posts"], st["upgrades"], st["drives"]) == (1, 8192 + 4096 + RB - 32768, 1, 0, 0)
        with pytest.raises(RuntimeError, match="without a record file"):
            b.upgrade(eng, 0, 0)
        with pytest.raises(RuntimeError, match="without a record file"):
            eng.tier_load([0, 1])                                         # no drive to read a tier from (once a division by zero)
        with pytest.raises(RuntimeError, match="spans"):
            eng.upload(3, [(src.data_ptr(), b.slots[0].data_ptr(), 16)] * 9, b.stage[0].data_ptr(), row, b.seq.data_ptr(), 6)
        with pytest.raises(RuntimeError, match="span 0"):
            eng.upload(3, [(src.data_ptr(), b.slots[0].data_ptr(), 0)], b.stage[0].data_ptr(), row, b.seq.data_ptr(), 6)
    finally:
        eng.close()


class Sched:
    """records the executor's callbacks"""

    def __init__(s):
        s.log = []

    def landed(s, L, E): s.log.append(("landed", L, E))
    def released(s, L, E): s.log.append(("released", L, E))
    def failed(s, L, E, read_error=False): s.log.append(("failed", L, E, read_error))
    def cancelled(s, L, E): s.log.append(("cancelled", L, E))


@pytest.mark.parametrize("in_call", [False, True], ids=["mailbox_launch", "mailbox_in_call"])
def test_executor_serves_a_layer_through_upgrades_and_downgrades(tmp_path, in_call):
    """in_call: the step is served(..., mailbox=mb) instead of mb.apply(); served(...).
    shards -> repack -> RankFile + resident planes -> RankExecutor: after every step the served layer equals, bitwise,
    the layer whose rows were set directly to the levels the mailbox has applied; slots are reused only after the
    downgrade was applied; with two slots for three wanted experts the third upgrade waits for a slot"""
    root, out = str(tmp_path / "fit"), str(tmp_path / "out")
    ids, L, rank, tp, topk, B = (0, 3, 4, 6), 7, 2, 4, 2, 4
    man, parts = synth_layer(seed=91, H=256, res_K=2.3125, var=True, rg=1, rd=2, experts=ids, had_dn=512)
    write_layer(root, L, man, parts, "safetensors")
    repack.repack(root, out, tp=tp, layers=[L], dev=DEV, ne=8, log=lambda s: None)
    RL = nqload.RankLayer(root, L, rank, tp, dev=DEV)
    H, I = RL.H, RL.I
    direct = M.MoELayer(8, H, I, Bmax=B, topk=topk)

    def set_direct(levels):
        for E in ids:
            row = M.entry(RL.ex[E], levels[E])
            row[9] = RL.ex[E].sc[levels[E]].data_ptr()
            direct.table[E].copy_(row.to(DEV))

    rf = RankFile(out, rank)
    got, h, i = resident.load(f"{out}/res/rank{rank}/L{L}.pt", DEV)
    served = M.MoELayer(8, H, I, Bmax=B, topk=topk)
    for E in ids:
        served.set(E, got[E], 2)
    mb = M.Mailbox(served)
    ex = RankExecutor(rf, {L: (served, mb, {E: got[E] for E in ids})}, nslot=2, n_host=4, qd=2, device=0)
    sched = Sched()
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(B, H, generator=g) * 0.5).half().to(DEV)
    sel = torch.stack([torch.tensor(ids)[torch.randperm(len(ids), generator=g)[:topk]] for _ in range(B)]).to(DEV)
    rw = torch.softmax(torch.randn(B, topk, generator=g), -1).half().to(DEV)
    levels = {E: 2 for E in ids}

    def step():
        """one layer call as the serving loop makes it; returns the output and updates `levels` from the callbacks"""
        if in_call:
            y = served(x, sel, rw, mailbox=mb).clone()
        else:
            mb.apply()
            y = served(x, sel, rw).clone()
        torch.cuda.synchronize()
        n = len(sched.log)
        ex.poll(sched)
        for ev in sched.log[n:]:
            if ev[0] == "landed":
                levels[ev[2]] = 4
            elif ev[0] == "released":
                levels[ev[2]] = 2
        return y

    def settle(cond, limit=20.0):
        t0 = time.time()
        while not cond() and time.time() - t0 < limit:
            y = step()
            time.sleep(0.002)
        assert cond(), (levels, sched.log, ex.ops, ex.wait_apply, ex.pend, ex.free, ex.eng.stats())

    def check():
        # a layer call with nothing in flight: the table holds exactly `levels`
        y = step()
        set_direct(levels)
        want = direct(x, sel, rw).clone()
        torch.cuda.synchronize()
        assert [int(served.table[E, 0]) for E in ids] == [levels[E] for E in ids]
        assert torch.isfinite(want).all() and torch.equal(y, want)
        ex.check_invariants()

    try:
        check()
        ex.apply([(L, 0), (L, 4), (L, 6)], [], sched)                 # two slots: expert 6 waits
        assert ex.n_waited == 1 and ex.pend == [(L, 6)] and ex.busy()
        settle(lambda: levels[0] == 4 and levels[4] == 4 and not ex.ops and not ex.wait_apply)
        assert levels[6] == 2 and ex.pend == [(L, 6)] and not ex.free
        check()
        rec = torch.from_numpy(np.fromfile(rf.path, dtype=np.uint8, count=rf.rb, offset=rf.rec(L, 4) * rf.rb))
        assert torch.equal(ex.slots[ex.slot_of[L, 4]].cpu(), rec)
        slot0 = ex.slot_of[L, 0]
        ex.apply([], [(L, 0)], sched)                                  # frees a slot; the waiting upgrade takes it
        settle(lambda: levels[0] == 2 and levels[6] == 4 and not ex.busy())
        assert ex.slot_of == {(L, 4): ex.slot_of[L, 4], (L, 6): slot0} and ex.quiet()
        check()
        assert ("released", L, 0) in sched.log and sched.log.index(("released", L, 0)) < sched.log.index(("landed", L, 6))
        # refused instead of waiting
        ex.wait = False
        ex.apply([(L, 3)], [], sched)
        assert sched.log[-1] == ("failed", L, 3, False) and ex.n_refused == 1
        # a failed read leaves the expert at level 2 and gives the slot back
        ex.apply([], [(L, 4)], sched)
        settle(lambda: levels[4] == 2 and not ex.busy())
        ex.eng.set_fault(fail_ppm=1000000)
        ex.apply([(L, 3)], [], sched)
        settle(lambda: sched.log[-1] == ("failed", L, 3, True))
        assert len(ex.free) == 1 and ex.n_failed == 1 and (L, 3) not in ex.slot_of
        ex.eng.set_fault()
        check()
        # the probe has teeth: a flipped slot byte and a foreign table row are both found
        sl6 = ex.slot_of[L, 6]
        ex.slots[sl6, 100] ^= 1
        with pytest.raises(AssertionError, match="B: slot"):
            ex.check_invariants()
        ex.slots[sl6, 100] ^= 1
        keep = served.table[6].clone()
        served.table[6, 2] += ex.rb
        with pytest.raises(AssertionError, match="T: row"):
            ex.check_invariants()
        served.table[6].copy_(keep)
        ex.check_invariants()
        st = ex.io_stats()
        assert st["landed_cum"] == 3 and st["free_slots"] == 1 and st["ops_outstanding"] == 0 and st["op_p50_ms"] > 0
    finally:
        ex.close()


@pytest.mark.parametrize("in_call", [False, True], ids=["mailbox_launch", "mailbox_in_call"])
def test_scheduler_executor_and_layer_in_one_serving_loop(tmp_path, in_call):
    """in_call: the step is served(..., mailbox=mb) instead of mb.apply(); served(...).
    the reference's serving step (sm120/serve/nq_vllm.py:546-574 with streaming/smoke_sched.py's loop): mailbox, layer
    call with the hits export, counts -> Scheduler.step -> RankExecutor.apply, poll after the call. Routing favours two
    experts at a time and then moves on; whenever nothing is in flight the table's levels are the scheduler's, and the layer
    equals, bitwise, a layer set directly to those levels"""
    from nestquant_amd.scheduler import Scheduler
    root, out = str(tmp_path / "fit"), str(tmp_path / "out")
    ids, L, rank, tp, topk, B = (0, 1, 3, 4, 6, 7), 5, 1, 4, 2, 1
    man, parts = synth_layer(seed=17, H=256, res_K=2.25, experts=ids)
    write_layer(root, L, man, parts, "safetensors")
    repack.repack(root, out, tp=tp, layers=[L], dev=DEV, ne=8, log=lambda s: None)
    RL = nqload.RankLayer(root, L, rank, tp, dev=DEV)
    H, I = RL.H, RL.I
    rf = RankFile(out, rank)
    got, _, _ = resident.load(f"{out}/res/rank{rank}/L{L}.pt", DEV)
    served, direct = M.MoELayer(8, H, I, Bmax=B, topk=topk), M.MoELayer(8, H, I, Bmax=B, topk=topk)
    hits = torch.zeros(8, dtype=torch.int32).pin_memory()
    served.hits_ptr = hits.data_ptr()
    for E in ids:
        served.set(E, got[E], 2)
    mb = M.Mailbox(served)
    ex = RankExecutor(rf, {L: (served, mb, {E: got[E] for E in ids})}, nslot=2, n_host=4, qd=2, device=0)
    S = Scheduler([L], {L: []}, {L: []}, rf.rb, NE=8, n_float=2, half_life=16, refresh=4, cap_GBps=1e3, tok_per_s=1.0, slots=2)
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(B, H, generator=g) * 0.5).half().to(DEV)
    rw = torch.tensor([[0.625, 0.375]]).half().to(DEV)
    seen_sets, checked = set(), 0
    try:
        for t in range(240):
            pair = [(0, 1), (3, 4), (6, 7), (4, 0)][(t // 60) % 4]
            sel = torch.tensor([pair], device=DEV)
            prev = hits.clone()
            if in_call:
                y = served(x, sel, rw, mailbox=mb).clone()
            else:
                mb.apply()
                y = served(x, sel, rw).clone()
            torch.cuda.synchronize()
            ex.poll(S)
            counts = (hits - prev).numpy().astype(np.float64)[None]
            assert counts.sum() == topk and counts[0, list(pair)].tolist() == [1, 1]
            if ex.quiet() and not ex.pend:
                lv = S.level()[0]
                assert [int(served.table[E, 0]) for E in ids] == [int(lv[E]) for E in ids]
                assert sorted(E for (_, E) in ex.slot_of) == [E for E in ids if lv[E] == 4]
                for E in ids:
                    row = M.entry(RL.ex[E], int(lv[E]))
                    row[9] = RL.ex[E].sc[int(lv[E])].data_ptr()
                    direct.table[E].copy_(row.to(DEV))
                want = direct(x, sel, rw).clone()
                torch.cuda.synchronize()
                assert torch.equal(y, want)
                seen_sets.add(tuple(E for E in ids if lv[E] == 4)); checked += 1
                if checked % 16 == 0:
                    ex.check_invariants(S)
            ups, downs = S.step(counts, ntok=B)
            ex.apply(ups, downs, S)
            time.sleep(0.001)
        assert checked >= 100 and {(0, 1), (3, 4), (6, 7), (0, 4)} <= seen_sets, (checked, seen_sets)
        assert S.stats["ups"] >= 8 and S.stats["downs"] >= 6 and ex.n_failed == 0
    finally:
        ex.close()
