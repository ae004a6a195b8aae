"""A layer served from the on-disk formats (resident file + level-4 records in a slot pool, promoted through the mailbox)
gives bitwise the outputs of the same experts set into a layer directly, in the decode path and in prefill."""
import json
import os
import types

import numpy as np
import pytest
import torch

from nestquant_amd import format as F, moe as M, nqload, p4rec, repack, resident
from tests.shards import synth_layer, write_layer
from tests.test_formats import _lr_expert, _rank_layer
from tests.util import O, oracle_plane, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_layer_from_resident_file_and_record_slots(tmp_path):
    H, I, E, topk, B = 256, 512, 6, 3, 4
    ranks = [(0, 0), (2, 1), (4, 4), (1, 0), (0, 3), (2, 2)]
    exs = [_lr_expert(H, I, 40 + e, *ranks[e], rk=(3, 9)) for e in range(E)]
    exs[0].lr = exs[0].lr4 = None
    levels = [2, 4, 4, 2, 4, 0]
    for x in exs:
        x.gu.to(DEV); x.dn.to(DEV); x.signs = x.signs.to(DEV); x.sc = {k: v.to(DEV) for k, v in x.sc.items()}
        x.lr, x.lr4 = (None, None) if x.lr is None else (x.lr.to(DEV), x.lr4.to(DEV))
        x.had_dn = 512

    # direct layer: rows straight from the experts' own tensors (level-4 rows with the level-4 scale vector)
    direct = M.MoELayer(E, H, I, Bmax=B, topk=topk)
    for e in range(E):
        row = M.entry(exs[e], levels[e])
        if levels[e] == 4:
            row[9] = exs[e].sc[4].data_ptr()
        M.validate_row(row, H, I)
        direct.table[e].copy_(row.to(DEV))

    # served layer: resident file -> level-2 rows; records -> pinned staging -> slots on a side stream -> mailbox
    path = str(tmp_path / "L7.pt")
    resident.save(_rank_layer(exs[:5], list(range(5)), H, I, had_dn=512), path)          # expert 5 is absent (level 0)
    got, h, i = resident.load(path, DEV)
    assert (h, i) == (H, I)
    lay = p4rec.layout(exs[1], H, I)
    served = M.MoELayer(E, H, I, Bmax=B, topk=topk)
    for e in range(5):
        served.set(e, got[e], 2)
    mb = M.Mailbox(served)
    pool = torch.zeros(3, lay["rec_bytes"], dtype=torch.uint8, device=DEV)
    stage = torch.empty(3, lay["rec_bytes"], dtype=torch.uint8).pin_memory()
    side = torch.cuda.Stream()
    for slot, e in enumerate(e for e in range(5) if levels[e] == 4):
        p4rec.pack_into(exs[e], lay, stage[slot])
        with torch.cuda.stream(side):
            pool[slot].copy_(stage[slot], non_blocking=True)
        mb.post(e, p4rec.row(got[e], lay, pool[slot].data_ptr(), M.entry), side)
    side.synchronize()

    g = torch.Generator().manual_seed(9)
    x = (torch.randn(B, H, generator=g) * 0.5).half().to(DEV)
    sel = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(B)]).to(DEV)
    rw = torch.softmax(torch.randn(B, topk, generator=g), -1).half().to(DEV)
    mb.apply()
    y = served(x, sel, rw).clone()
    want = direct(x, sel, rw).clone()
    torch.cuda.synchronize()
    assert all(mb.done(e) for e in range(E))
    assert [int(v) for v in served.table[:, 0].cpu()] == levels
    assert torch.isfinite(want).all() and want.abs().max() > 0
    assert torch.equal(y, want)
    # level 2 everywhere differs (the records matter), and prefill agrees bitwise too
    assert not torch.equal(served(x, sel, rw, force_level=2), want)
    T = 40
    xt = (torch.randn(T, H, generator=g) * 0.5).half().to(DEV)
    st = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(DEV)
    wt = torch.softmax(torch.randn(T, topk, generator=g), -1).half().to(DEV)
    assert torch.equal(served.prefill(xt, st, wt), direct.prefill(xt, st, wt))


@pytest.mark.parametrize("base_K,res_K,container", [(2, 2.25, "safetensors"), (1.75, 2.5625, "pt")])
def test_layer_from_production_shards_matches_the_oracle(tmp_path, base_K, res_K, container):
    """shard files -> nqload.RankLayer (rank 1 of 4) -> table rows -> decode path and prefill, against the oracle's layer over
    the oracle's dense decode of the loaded planes, with the low-rank factors taken from the shards themselves"""
    Hh, topk, B = 256, 2, 3
    ids = (4, 9, 17)
    man, parts = synth_layer(seed=71, H=Hh, res_K=res_K, base_K=base_K, var=True, rg=2, rd=1, experts=ids, had_dn=512)
    write_layer(str(tmp_path), 3, man, parts, container)
    RL = nqload.RankLayer(str(tmp_path), 3, rank=1, tp=4, dev=DEV)
    H, I = RL.H, RL.I
    assert (H, I, RL.had_dn) == (Hh, 512, 512)
    levels = [2, 4, 4]
    layer = M.MoELayer(len(ids), H, I, Bmax=B, topk=topk)
    for e, E in enumerate(ids):
        row = M.entry(RL.ex[E], levels[e])
        if levels[e] == 4:
            row[9] = RL.ex[E].sc[4].data_ptr()
        M.validate_row(row, H, I)
        layer.table[e].copy_(row.to(DEV))
    layer.rare_rows = base_K != 2
    # dequant of a loaded projection is bit-exact against the oracle's decode of the same planes
    for e, E in enumerate(ids):
        for proj, p in ((0, RL.ex[E].gu), (1, RL.ex[E].dn)):
            got = M.dequant(layer.table[e], proj, H, I, levels[e]).cpu().numpy()
            assert np.array_equal(got.view(np.uint16), O.dense_W(oracle_plane(p), levels[e]).astype(np.float16).view(np.uint16))

    def lr_of(e):
        a = RL.art(ids[e])
        f = lambda t: t.numpy().astype(np.float16)
        return dict(Vg=f(a["gate"]["base"]["lr"]["V"]), U2g=f(a["gate"]["base"]["lr"]["U2"]), U2u=f(a["up"]["base"]["lr"]["U2"]),
                    U4g=f(a["gate"]["p4"]["lr"]["U4"]), U4u=f(a["up"]["p4"]["lr"]["U4"]), Vd=f(a["down"]["base"]["lr"]["V"]),
                    U2d=f(a["down"]["base"]["lr"]["U2"]), U4d=f(a["down"]["p4"]["lr"]["U4"]))

    dense = lambda e: (O.dense_W(oracle_plane(RL.ex[ids[e]].gu), levels[e]).astype(np.float32),
                       O.dense_W(oracle_plane(RL.ex[ids[e]].dn), levels[e]).astype(np.float32))
    signs = lambda e: RL.ex[ids[e]].sc[levels[e]].cpu().numpy()
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(B, H, generator=g) * 0.5).half()
    sel = torch.stack([torch.randperm(len(ids), generator=g)[:topk] for _ in range(B)])
    rw = torch.softmax(torch.randn(B, topk, generator=g), -1).half()
    want = O.moe_forward(dense, levels, signs, x.numpy(), sel.numpy(), rw.numpy(), dtype=np.float64, had_dn=512, lr=lr_of)
    y = layer(x.to(DEV), sel.to(DEV), rw.to(DEV)).cpu().numpy()
    assert np.isfinite(y).all() and rel_err(y, want) < 1e-3
    no_lr = O.moe_forward(dense, levels, signs, x.numpy(), sel.numpy(), rw.numpy(), dtype=np.float64, had_dn=512)
    assert rel_err(no_lr, want) > 1e-2                  # the low-rank plane matters in this layer
    T = 24
    xt = (torch.randn(T, H, generator=g) * 0.5).half()
    st = torch.stack([torch.randperm(len(ids), generator=g)[:topk] for _ in range(T)])
    wt = torch.softmax(torch.randn(T, topk, generator=g), -1).half()
    want = O.moe_forward(dense, levels, signs, xt.numpy(), st.numpy(), wt.numpy(), dtype=np.float64, had_dn=512, lr=lr_of)
    assert rel_err(layer.prefill(xt.to(DEV), st.to(DEV), wt.to(DEV)).cpu().numpy(), want) < 1e-3


def test_layer_served_from_repacked_files_equals_the_shards_served_directly(tmp_path):
    """shards -> repack -> (resident file, record file, index) -> level-2 rows + records read into pinned staging, copied into
    slots on a side stream and promoted through the mailbox: bitwise the layer whose rows point at the loaded planes"""
    root, out = str(tmp_path / "fit"), str(tmp_path / "out")
    ids, L, rank, tp, topk, B = (0, 3, 4, 6), 7, 2, 4, 2, 4
    man, parts = synth_layer(seed=91, H=256, res_K=2.3125, var=True, rg=1, rd=2, experts=ids, had_dn=512)
    write_layer(root, L, man, parts, "safetensors")
    assert repack.repack(root, out, tp=tp, layers=[L], dev=DEV, ne=8, log=lambda s: None) == [(L, r) for r in range(tp)]
    RL = nqload.RankLayer(root, L, rank, tp, dev=DEV)
    H, I = RL.H, RL.I
    levels = {0: 4, 3: 2, 4: 4, 6: 4}
    direct = M.MoELayer(8, H, I, Bmax=B, topk=topk)
    for E in ids:
        row = M.entry(RL.ex[E], levels[E])
        if levels[E] == 4:
            row[9] = RL.ex[E].sc[4].data_ptr()
        M.validate_row(row, H, I)
        direct.table[E].copy_(row.to(DEV))

    with open(f"{out}/rank{rank}.json") as f:
        idx = json.load(f)
    lay = dict(seg={k: tuple(v) for k, v in idx["seg"].items()}, rec_bytes=idx["rec_bytes"])
    got, h, i = resident.load(f"{out}/res/rank{rank}/L{L}.pt", DEV)
    assert (h, i) == (H, I) and got[0].had_dn == 512
    served = M.MoELayer(8, H, I, Bmax=B, topk=topk)
    for E in ids:
        served.set(E, got[E], 2)
    mb = M.Mailbox(served)
    up = [E for E in ids if levels[E] == 4]
    pool = torch.zeros(len(up), idx["rec_bytes"], dtype=torch.uint8, device=DEV)
    stage = torch.empty(len(up), idx["rec_bytes"], dtype=torch.uint8).pin_memory()
    side = torch.cuda.Stream()
    fd = os.open(f"{out}/rank{rank}.bin", os.O_RDONLY)
    try:
        for slot, E in enumerate(up):
            repack.read_record(fd, idx, L, E, stage[slot])
            with torch.cuda.stream(side):
                pool[slot].copy_(stage[slot], non_blocking=True)
            mb.post(E, p4rec.row(got[E], lay, pool[slot].data_ptr(), M.entry), side)
    finally:
        os.close(fd)
    side.synchronize()
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(B, H, generator=g) * 0.5).half().to(DEV)
    sel = torch.stack([torch.tensor(ids)[torch.randperm(len(ids), generator=g)[:topk]] for _ in range(B)]).to(DEV)
    rw = torch.softmax(torch.randn(B, topk, generator=g), -1).half().to(DEV)
    mb.apply()
    y = served(x, sel, rw).clone()
    want = direct(x, sel, rw).clone()
    torch.cuda.synchronize()
    assert [int(served.table[E, 0]) for E in ids] == [levels[E] for E in ids]
    assert torch.isfinite(want).all() and want.abs().max() > 0 and torch.equal(y, want)
    assert not torch.equal(served(x, sel, rw, force_level=2), want)
