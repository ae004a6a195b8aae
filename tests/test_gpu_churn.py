"""Plane churn: promotions / demotions issued on a side stream race graph replays of [mailbox, layer]; every replay must
equal the float64 oracle of the level state it actually applied, every swapped expert must dequantise bit-exactly, and the
slot / table invariants must hold (reference sm120/levelswitch_mbox.py, sm120/serve/nq_slotcheck.py)."""
import random
import time

import numpy as np
import pytest
import torch

from nestquant_amd import churn as CH, format as F, moe as M
from oracle import nq_oracle as O
from tests.util import oracle_plane, rel_err, same_f16

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_slot_layout_and_rows():
    lay = CH.SlotLayout(6144, 2048)
    p = lay.parts
    assert p["gu.p3"] == (0, 3145728) and p["gu.p4"] == (3145728, 3145728) and p["dn.p3"][0] == 6291456
    assert p["gu.d3"][1] == 49152 and p["dn.d4"][1] == 24576 and lay.bytes % 256 == 0
    assert sum(n for _, n in lay.spans(2, 3)) == 4718592 + 73728                # P3 + d3 of one expert: 4 718 592 + 73 728 bytes at H 6144, I 2048
    assert sum(n for _, n in lay.spans(3, 4)) == 4718592 + 73728
    assert lay.spans(2, 4) == [(0, lay.bytes)] and lay.bytes >= 2 * (4718592 + 73728)


@pytest.mark.parametrize("in_call", [False, True], ids=["mailbox_launch", "mailbox_in_call"])
@pytest.mark.parametrize("native", [False, True], ids=["torch_copies", "engine_uploads"])
def test_churn_racing_graph_replays(native, in_call):
    """in_call: the replayed step is L(..., mailbox=MB) instead of MB.apply(); L(...). Every expert has a sign vector of its own
    per level (as served experts do: the level-2 and level-4 rows name different vectors), so a call whose parts disagreed
    about a row's level would rotate with the wrong vector and miss the oracle of either state."""
    H, I, NE, NSLOT, B, K = 512, 256, 8, 3, 4, 4
    ex = {e: F.Expert(H, I, seed=70 + e, dev="cpu", nested=True, var=(e == 2)) for e in range(NE)}
    planes = {e: (oracle_plane(x.gu), oracle_plane(x.dn)) for e, x in ex.items()}
    gs = torch.Generator().manual_seed(700)
    signs = {}
    for e, x in ex.items():
        x.sc = {2: x.signs}
        for lv in (3, 4):
            x.sc[lv] = (torch.randint(0, 2, x.signs.shape, generator=gs) * 2 - 1).half()
        for lv in (2, 3, 4):
            signs[e, lv] = x.sc[lv].numpy()
    for x in ex.values():
        x.gu.to(DEV); x.dn.to(DEV); x.signs = x.signs.to(DEV)
        x.sc = {lv: (x.signs if lv == 2 else v.to(DEV)) for lv, v in x.sc.items()}
        x.gu.slot = x.gu.nested_plane(); x.dn.slot = x.dn.nested_plane()
    L = M.MoELayer(NE, H, I, Bmax=B, topk=K)
    MB = M.Mailbox(L)
    X = CH.ChurnExecutor(L, MB, ex, NSLOT, native=native)
    for e in range(NE):
        L.table[e].copy_(X.row(e, 2))
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(B, H, generator=g) * 0.05).half().to(DEV)
    sel = torch.stack([torch.randperm(NE, generator=g)[:K] for _ in range(B)]).to(DEV)
    rw = torch.rand(B, K, generator=g).half().to(DEV)
    # float64 oracle output of every (expert, level) on these tokens, combined per level state
    xn = x.cpu().numpy()
    dense = {(e, lv): (O.dense_W(planes[e][0], lv, nested=True).astype(np.float32), O.dense_W(planes[e][1], lv, nested=True).astype(np.float32))
             for e in range(NE) for lv in (2, 3, 4)}
    yel = {k: O.expert_forward(xn, *w, signs[k], dtype=np.float64) for k, w in dense.items()}

    def ref(level):
        y = np.zeros((B, H))
        for b in range(B):
            for k in range(K):
                e = int(sel[b, k])
                y[b] += float(rw[b, k]) * yel[(e, level[e])][b]
        return y

    s = torch.cuda.Stream()
    step = (lambda: L(x, sel, rw, mailbox=MB)) if in_call else (lambda: (MB.apply(), L(x, sel, rw)))
    with torch.cuda.stream(s):
        for _ in range(2):
            step()
    torch.cuda.synchronize()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr, stream=s):
        step()
    junk = torch.randint(0, 256, (X.lay.bytes,), dtype=torch.uint8).pin_memory()
    rng = random.Random(1)
    nops, worst, changed = 0, 0.0, 0
    for st in range(80):
        prev = dict(X.level)
        for _ in range(rng.randint(0, 2)):                       # scheduler: new ops on the side stream, no host sync
            e = rng.randrange(NE)
            if not X.idle(e):
                continue
            lv = X.level[e]
            if lv == 2 or (lv == 3 and rng.random() < 0.5):
                nops += X.promote(e, rng.choice([3, 4]) if lv == 2 else 4)
            else:
                nops += X.demote(e, rng.choice([2, 3]) if lv == 4 else 2)
        gr.replay()
        torch.cuda.synchronize()                                 # (sync only to check this replay's output)
        out = L.out[:B].cpu().numpy()
        free_before = set(X.free)
        for e in X.poll():
            row = L.table[e].clone()
            lv = X.level[e]
            for proj, pl in ((0, planes[e][0]), (1, planes[e][1])):
                W = M.dequant(row, proj, H, I).cpu().numpy()
                assert same_f16(W, O.dense_W(pl, lv, nested=True)) == 0, (st, e, lv, proj)
        for sl in set(X.free) - free_before:                     # released slots are scribbled at once: stale use would show
            with torch.cuda.stream(X.side):
                X.slots[sl].copy_(junk, non_blocking=True)
            if native:
                X.side.synchronize()                             # the engine's uploads run on its own stream, not X.side
        err = rel_err(out, ref(X.level))
        worst = max(worst, err)
        assert err < 5e-5, (st, err, X.level)
        if X.level != prev and any(X.level[e] != prev[e] for e in set(sel.flatten().tolist())):
            changed += 1
            assert rel_err(out, ref(prev)) > 1e-3                # the stale state would be far off: the check has teeth
        if st % 10 == 9:
            X.check_invariants()
    torch.cuda.synchronize()
    X.check_invariants()
    # the engine's ops land a thread hop later than copies issued from this thread, so fewer experts are idle when picked
    assert nops > (20 if native else 30) and changed > (5 if native else 10) and X.bytes_copied > 0
    if native:
        for _ in range(2000):                                    # the engine reports an op a moment after its copies completed
            X.poll()
            if len(X.lat) == nops:
                break
            time.sleep(0.001)
        st_ = X.eng.stats()
        assert st_["upload_bytes"] == X.bytes_copied and st_["uploads"] + st_["posts"] == nops and len(X.lat) == nops
    X.close()
    print(f"ops {nops}, refused {X.n_refused}, state changes seen {changed}, worst rel err {worst:.2e}")


def test_refusals():
    H, I = 256, 256
    ex = {e: F.Expert(H, I, seed=e, dev=DEV, nested=True, gen_dev=DEV) for e in range(3)}
    L = M.MoELayer(3, H, I, Bmax=1, topk=2); MB = M.Mailbox(L)
    X = CH.ChurnExecutor(L, MB, ex, nslots=1)
    for e in range(3):
        L.table[e].copy_(X.row(e, 2))
    assert X.promote(0, 4) and not X.promote(0, 3)               # one outstanding op per expert
    assert not X.promote(1, 3)                                   # pool full: refused, expert stays at level 2
    MB.apply(); torch.cuda.synchronize()
    assert X.poll() == [0] and X.level == {0: 4, 1: 2, 2: 2}
    assert X.demote(0, 2)
    assert not X.promote(1, 3)                                   # the slot is not reusable before the level-2 row is applied
    MB.apply(); torch.cuda.synchronize(); X.poll()
    assert X.promote(1, 3)
    MB.apply(); torch.cuda.synchronize(); X.poll()
    X.check_invariants()
    with pytest.raises(AssertionError):
        X.promote(1, 3)
