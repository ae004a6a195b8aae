"""Bookkeeping of executor.RankExecutor on the host alone: a stand-in engine whose ops the test completes by hand, a
stand-in mailbox whose `applied_host` the test advances. The rules are the reference's (streaming/executor.py:13-15,71-135):
one slot per upgraded expert, a slot returns to the pool only when the downgrade's row was applied, a waiting upgrade takes
the next free slot in arrival order, refused / failed / cancelled upgrades give their slot back and tell the scheduler."""
import types

import numpy as np
import torch

from nestquant_amd import p4rec
from nestquant_amd.executor import RankExecutor
from nestquant_amd.moe import entry
from tests.test_formats import _lr_expert

H, I, L, NE = 256, 128, 4, 6


class FakeEngine:
    def __init__(s):
        s.q, s.done, s.cancels, s.closed = {}, [], [], False

    def upgrade(s, tag, rec, slot, stage, row, seqp, seq):
        s.q[tag] = dict(kind=4, rec=rec, slot=slot, stage=stage, row=np.array(row), seqp=seqp, seq=seq)

    def post(s, tag, stage, row, seqp, seq):
        s.q[tag] = dict(kind=2, stage=stage, row=np.array(row), seqp=seqp, seq=seq)

    def cancel(s, tag):
        s.cancels.append(tag)

    def finish(s, tag, trd=0.001):
        s.q.pop(tag)
        s.done.append((tag, False, trd, trd + 0.002 if trd >= 0 else (-1.0 if trd > -1e8 else trd)))

    def poll(s):
        d, s.done = s.done, []
        return d

    def stats(s):
        return dict(now=1.0 + len(s.q), bytes_read=0, tier_bytes=0, host_hits=0, tier_hits=0, upgrades=0, drive_bytes=[0], drive_reads=[0],
                    drive_read_s=[0.0], drive_inflight=[0], drive_qd=[2], tier_recs=0, tier_state=0, waiting=0, reading=0, copying=0)

    def close(s):
        s.closed = True


class Log:
    def __init__(s): s.ev = []
    def landed(s, L, E): s.ev.append(("landed", E))
    def released(s, L, E): s.ev.append(("released", E))
    def failed(s, L, E, read_error=False): s.ev.append(("failed", E, read_error))
    def cancelled(s, L, E): s.ev.append(("cancelled", E))


def make(nslot=2, **kw):
    exs = {E: _lr_expert(H, I, 20 + E, 1, 1, rk=(3, 9)) for E in range(NE)}
    lay = p4rec.layout(exs[0], H, I)
    rf = types.SimpleNamespace(lay=lay, rb=lay["rec_bytes"], rec=lambda L_, E: (L_ - 3) * NE + E)
    layer = types.SimpleNamespace(H=H, I=I, rare_rows=False)
    mb = types.SimpleNamespace(stage=torch.zeros(NE, 20, dtype=torch.int64), seq=torch.zeros(NE, dtype=torch.int32),
                               applied_host=torch.zeros(NE, dtype=torch.int32), hseq=[0] * NE)
    eng = FakeEngine()
    ex = RankExecutor(rf, {L: (layer, mb, exs)}, nslot, device="cpu", engine=eng, **kw)
    return ex, eng, mb, exs, lay


def test_rows_slots_and_the_order_of_release():
    ex, eng, mb, exs, lay = make()
    log = Log()
    ex.apply([(L, 1), (L, 3), (L, 5)], [], log)
    assert sorted(eng.q) == [1, 2] and ex.pend == [(L, 5)] and ex.n_waited == 1 and not ex.free
    op = eng.q[1]
    assert op["rec"] == NE + 1 and op["slot"] == ex.addr(ex.slot_of[L, 1]) and op["seq"] == 1
    assert op["stage"] == mb.stage.data_ptr() + 160 * 1 and op["seqp"] == mb.seq.data_ptr() + 4 * 1
    want = p4rec.row(exs[1], lay, op["slot"], entry).numpy()             # the level-4 row points into the slot
    assert (op["row"] == want).all() and op["row"][0] == 4 and op["row"][2] == op["slot"] + lay["seg"]["gu.p4"][0]
    eng.finish(1); eng.finish(2)
    ex.poll(log)
    assert log.ev == [] and set(ex.wait_apply) == {(L, 1), (L, 3)} and mb.hseq[1] == 1 and ex.busy() and not ex.quiet()
    mb.applied_host[1] = 1                                               # the mailbox kernel ran
    ex.poll(log)
    assert log.ev == [("landed", 1)] and (L, 3) in ex.wait_apply
    mb.applied_host[3] = 1
    ex.poll(log)
    assert log.ev[-1] == ("landed", 3) and ex.quiet() and ex.busy()      # expert 5 still waits for a slot
    # downgrade of 1: its slot is free only after the level-2 row was applied; then the waiting upgrade takes it
    slot1 = ex.slot_of[L, 1]
    ex.apply([], [(L, 1)], log)
    down = eng.q[3]
    assert down["kind"] == 2 and down["seq"] == 2 and down["row"][0] == 2 and (down["row"] == entry(exs[1], 2).numpy()).all()
    eng.finish(3, trd=0.0)
    ex.poll(log)
    assert not ex.free and ex.pend == [(L, 5)] and (L, 1) in ex.slot_of
    mb.applied_host[1] = 2
    ex.poll(log)
    assert log.ev[-1] == ("released", 1) and (L, 1) not in ex.slot_of and ex.slot_of[L, 5] == slot1 and not ex.pend
    assert eng.q[4]["kind"] == 4 and eng.q[4]["slot"] == ex.addr(slot1)
    ex.close()
    assert eng.closed


def test_refused_failed_and_cancelled_upgrades_return_their_slot():
    ex, eng, mb, exs, lay = make(nslot=1, wait_for_slot=False)
    log = Log()
    ex.apply([(L, 0), (L, 2)], [], log)
    assert log.ev == [("failed", 2, False)] and ex.n_refused == 1 and list(eng.q) == [1]
    eng.finish(1, trd=-5.0)                                              # the read failed
    ex.poll(log)
    assert log.ev[-1] == ("failed", 0, True) and ex.free == [0] and not ex.slot_of and ex.n_failed == 1 and mb.hseq[0] == 0
    ex.apply([(L, 2)], [], log)
    assert ex.cancel_up(L, 2, log) and eng.cancels == [2] and not ex.cancel_up(L, 4, log)
    eng.finish(2, trd=-1e9)                                              # the engine dropped it before it started
    ex.poll(log)
    assert log.ev[-1] == ("cancelled", 2) and ex.free == [0] and ex.n_cancel == 1 and not ex.busy()
    # an upgrade still waiting for a slot is cancelled here, without the engine
    ex.wait = True
    ex.apply([(L, 4), (L, 5)], [], log)
    assert ex.pend == [(L, 5)] and ex.cancel_up(L, 5, log) and log.ev[-1] == ("cancelled", 5) and not ex.pend and ex.n_cancel == 2
    # poll(issue=False) leaves waiting upgrades alone
    ex.apply([(L, 5)], [], log)
    eng.finish(3, trd=-5.0)
    ex.poll(log, issue=False)
    assert ex.free == [0] and ex.pend == [(L, 5)]
    ex.poll(log)
    assert not ex.free and ex.slot_of == {(L, 5): 0}


def test_a_failed_downgrade_keeps_its_slot_and_is_posted_again():
    """the engine reports an op whose copies failed with t_read < 0 whatever its kind; for a downgrade the level-4 row is
    still live and points into the slot, so the slot stays owned, the scheduler hears nothing, and the row is posted again"""
    import pytest
    ex, eng, mb, exs, lay = make(nslot=1)
    log = Log()
    ex.apply([(L, 1)], [], log)
    eng.finish(1); ex.poll(log); mb.applied_host[1] = 1; ex.poll(log)
    assert log.ev == [("landed", 1)] and ex.slot_of == {(L, 1): 0}
    ex.apply([], [(L, 1)], log)
    eng.finish(2, trd=-5.0)                                              # the row copy failed
    ex.poll(log)
    assert log.ev == [("landed", 1)] and ex.slot_of == {(L, 1): 0} and not ex.free and ex.n_failed == 0
    assert list(eng.q) == [3] and eng.q[3]["kind"] == 2 and eng.q[3]["seq"] == 2 and ex.count["reposted"] == 1
    eng.finish(3, trd=0.0); ex.poll(log); mb.applied_host[1] = 2; ex.poll(log)
    assert log.ev[-1] == ("released", 1) and ex.free == [0] and not ex.busy()
    # an engine that keeps failing surfaces as an error, not as a silent loop
    ex.apply([(L, 1)], [], log)
    eng.finish(4); ex.poll(log); mb.applied_host[1] = 3; ex.poll(log)
    ex.apply([], [(L, 1)], log)
    with pytest.raises(RuntimeError, match="failed to post"):
        for tag in range(5, 12):
            eng.finish(tag, trd=-5.0)
            ex.poll(log)
    assert ex.slot_of == {(L, 1): 0}


def test_a_fatal_report_does_not_lose_the_rest_of_its_batch():
    """the report that exhausts a downgrade's reposts and the completion of another expert's upgrade arrive in one poll(): the
    error is raised after the whole batch has been handled, so the upgrade is in the books and lands"""
    import pytest
    from nestquant_amd import executor as EX
    ex, eng, mb, exs, lay = make(nslot=2)
    log = Log()
    ex.apply([(L, 1)], [], log)
    eng.finish(1); ex.poll(log); mb.applied_host[1] = 1; ex.poll(log)
    ex.apply([], [(L, 1)], log)
    tag = 2
    for _ in range(EX.REPOST_LIMIT):                                     # every repost fails too
        eng.finish(tag, trd=-5.0); ex.poll(log); tag += 1
    ex.apply([(L, 5)], [], log)                                          # tag + 1: an upgrade of another expert
    eng.finish(tag, trd=-5.0); eng.finish(tag + 1)                       # both reports in the next poll
    with pytest.raises(RuntimeError, match="failed to post"):
        ex.poll(log)
    assert ex.wait_apply == {(L, 5): (4, 1)} and ex.n_landed == 1 + 1    # the upgrade's report was handled
    mb.applied_host[5] = 1; ex.poll(log)
    assert log.ev[-1] == ("landed", 5) and ex.slot_of[L, 1] == 0 and (L, 5) in ex.slot_of


def test_shadow_posts_level_2_rows_and_io_stats_reports_intervals():
    ex, eng, mb, exs, lay = make(shadow=True)
    ex.apply([(L, 1)], [])
    assert eng.q[1]["kind"] == 4 and eng.q[1]["row"][0] == 2            # the read and the copy happen, the row stays level 2
    eng.finish(1, trd=0.004)
    ex.poll()
    st = ex.io_stats()
    assert st["landed_cum"] == 1 and st["ops_outstanding"] == 0 and st["free_slots"] == 1 and st["slot_wait"] == 0
    assert abs(st["op_p50_ms"] - 6.0) < 1e-6 and abs(st["rd_p50_ms"] - 4.0) < 1e-6 and abs(st["cp_p50_ms"] - 2.0) < 1e-6
    assert st["delivered_GBps"] > 0 and ex.io_stats()["delivered_GBps"] == 0       # second call: nothing since the first


def test_rank_file_index_and_row_arguments(tmp_path):
    import json
    import numpy as np
    from nestquant_amd import stream_engine as SE
    idx = dict(format="nq-p4rec-v1", tp=4, rank=2, L0=3, NE=256, rec_bytes=8192, seg={"gu.p4": [0, 4096], "gu.d4": [4096, 256]}, layers={})
    (tmp_path / "rank2.json").write_text(json.dumps(idx))
    rf = SE.RankFile(str(tmp_path), 2)
    assert rf.path == f"{tmp_path}/rank2.bin" and rf.rb == 8192 and rf.lay == dict(seg=idx["seg"], rec_bytes=8192)
    assert rf.rec(3, 0) == 0 and rf.rec(5, 17) == 2 * 256 + 17                     # ((L - L0) * NE + E), streaming/stream_engine.py:21
    assert SE.mod().Engine is SE.Engine
    # a row is int64[20] from a CPU tensor, a numpy array or a list; anything else is refused as the reference's binding does
    for row in (torch.arange(20), np.arange(20, dtype=np.int64), list(range(20))):
        assert list(SE._row_array(row)) == list(range(20))
    for bad in (torch.arange(19), torch.arange(20, dtype=torch.int32), list(range(21))):
        try:
            SE._row_array(bad)
        except RuntimeError as e:
            assert "int64 cpu [20]" in str(e)
        else:
            raise AssertionError("accepted a malformed row")
