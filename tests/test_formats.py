"""Serving on-disk formats: the level-4 record (p4rec) and the resident file (resident).

The record layout is pinned by the byte figures the reference publishes for its tensor-parallel-4 artifact
(sm120/NQ_RES_V2.md:63-68: H 6144, I 512, residual codes 3 / 9 -> segment offsets and lengths, rec_bytes 2,854,912).
No sample record or resident file ships with the reference, so beyond those figures the formats are checked through
round trips of this build's own files; byte-level interchange with a file written by the reference is unpinned."""
import json
import os
import types

import numpy as np
import pytest
import torch

from nestquant_amd import format as F, moe as M, p4rec, resident


def test_record_layout_matches_published_figures():
    want = {"gu.p4": (0, 1769472), "gu.d4": (1769472, 12288), "dn.p4": (1781760, 1007620), "dn.d4": (2789632, 6144),
            "lr4": (2795776, 57344)}
    lay = p4rec.layout_of(p4rec.seg_bytes(6144, 512, rk_gu=3, rk_dn=9))
    assert lay["seg"] == want and lay["rec_bytes"] == 2854912
    # the same from an expert's planes (only the sizes matter)
    plane = lambda nbytes: types.SimpleNamespace(p4=torch.empty(nbytes // 4, dtype=torch.int32), d4=torch.empty(0, dtype=torch.int32))
    ex = types.SimpleNamespace(gu=plane(1769472), dn=plane(1007620), lr4=None)
    ex.gu.d4 = torch.empty(12288 // 4, dtype=torch.int32); ex.dn.d4 = torch.empty(6144 // 4, dtype=torch.int32)
    assert p4rec.layout(ex, 6144, 512) == lay
    # a rank's record file: 75 layers x 256 experts (54.8 GB)
    assert 75 * 256 * lay["rec_bytes"] == 54814310400


@pytest.mark.parametrize("rk", [(0, 0), (3, 9), (6, 1), (4, 7)])
def test_layout_invariants(rk):
    H, I = 256, 128
    lay = p4rec.layout_of(p4rec.seg_bytes(H, I, *rk))
    end = 0
    for name in p4rec.SEGS:
        off, n = lay["seg"][name]
        assert off % p4rec.SEG_ALIGN == 0 and off >= end and off - end < p4rec.SEG_ALIGN
        end = off + n
    assert lay["rec_bytes"] % p4rec.ALIGN == 0 and 0 <= lay["rec_bytes"] - end < p4rec.ALIGN + p4rec.SEG_ALIGN
    ex = F.Expert(H, I, seed=3, dev="cpu", rk_gu=rk[0], rk_dn=rk[1])
    assert p4rec.layout(ex, H, I) == lay


def _lr_expert(H, I, seed, rg, rd, rk=(0, 0), var=True):
    ex = F.Expert(H, I, seed=seed, dev="cpu", rk_gu=rk[0], rk_dn=rk[1], var=var)
    g = torch.Generator().manual_seed(1000 + seed)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.05).half()
    ex.set_lr(r(rg, H), r(rg, I), r(rg, I), r(rg, I), r(rg, I), r(rd, I), r(rd, H), r(rd, H))
    sc4 = ex.signs * (0.5 + torch.rand(ex.signs.numel(), generator=g)).half()
    ex.sc = {2: ex.signs, 4: sc4}
    return ex


def test_pack_places_every_plane_and_zeroes_the_rest():
    H, I = 256, 128
    ex = _lr_expert(H, I, 5, 2, 3, rk=(3, 9))
    lay = p4rec.layout(ex, H, I)
    rec = np.frombuffer(p4rec.pack(ex, lay), np.uint8)
    assert rec.size == lay["rec_bytes"]
    covered = np.zeros(rec.size, bool)
    for name, t in (("gu.p4", ex.gu.p4), ("gu.d4", ex.gu.d4), ("dn.p4", ex.dn.p4), ("dn.d4", ex.dn.d4), ("lr4", ex.lr4)):
        off, n = lay["seg"][name]
        raw = t.contiguous().view(torch.uint8).numpy().reshape(-1)
        assert raw.size <= n and np.array_equal(rec[off:off + raw.size], raw), name
        covered[off:off + raw.size] = True
    assert not rec[~covered].any()
    # lr4 = U4_g | U4_u | U4_d at the expert's own ranks, the segment sized for RMAX
    assert ex.lr4.numel() == 2 * (2 * I) + 3 * H and lay["seg"]["lr4"][1] == p4rec.RMAX * (2 * I + H) * 2
    # pack_into a larger, dirty buffer gives the same record and leaves the tail alone
    buf = torch.full((lay["rec_bytes"] + 64,), 0xA5, dtype=torch.uint8)
    p4rec.pack_into(ex, lay, buf)
    assert np.array_equal(buf[: lay["rec_bytes"]].numpy(), rec) and bool((buf[lay["rec_bytes"]:] == 0xA5).all())
    with pytest.raises(ValueError):
        p4rec.pack_into(ex, lay, torch.empty(lay["rec_bytes"] - 1, dtype=torch.uint8))
    with pytest.raises(ValueError, match="do not fit"):
        p4rec.pack(_lr_expert(H, I, 5, 0, 0, rk=(4, 4)), lay)           # wider residual code than the layout's


def test_row_points_level_4_fields_into_the_slot():
    H, I = 256, 128
    ex = _lr_expert(H, I, 6, 1, 1)
    lay = p4rec.layout(ex, H, I)
    base = M.entry(ex, 4)
    slot = 0x7F0000000000
    r = p4rec.row(ex, lay, slot, M.entry)
    s = lay["seg"]
    assert [int(r[i]) for i in (2, 3, 6, 7, 15)] == [slot + s[k][0] for k in p4rec.SEGS]
    assert int(r[9]) == ex.sc[4].data_ptr() and int(r[0]) == 4
    keep = [i for i in range(F.TBL_W) if i not in (2, 3, 6, 7, 9, 15)]
    assert torch.equal(r[keep], base[keep])
    plain = F.Expert(H, I, seed=7, dev="cpu")                             # no low-rank plane, no per-level scales
    r = p4rec.row(plain, lay, slot, M.entry)
    assert int(r[15]) == 0 and int(r[9]) == plain.signs.data_ptr()


def _rank_layer(exs, ids, H, I, had_dn=128):
    return types.SimpleNamespace(L=7, rank=1, tp=4, H=H, I=I, experts=ids, ex=dict(zip(ids, exs)), had_dn=had_dn)


def test_resident_round_trip(tmp_path):
    H, I = 256, 128
    ranks = [(0, 0), (2, 3), (4, 4)]
    exs = [_lr_expert(H, I, 10 + i, *ranks[i], rk=(3, 9)) for i in range(3)]
    exs[0].lr = None
    ids = [5, 9, 2]
    path = str(tmp_path / "L7.pt")
    resident.save(_rank_layer(exs, ids, H, I), path)
    d = torch.load(path, weights_only=True)
    assert d["format"] == "nq-res-v1" and "bk_gu" not in d and "in_had_down" not in d
    assert d["lr"].shape == (3, resident.lr_len(H, I, 4, 4)) and d["lr"].dtype == torch.float16
    assert d["gu_base"].dtype == torch.int32 and d["gu_var"].dtype == torch.uint8 and d["sc4"].shape == (3, 3 * H + 3 * I)
    got, h, i = resident.load(path, "cpu")
    assert (h, i) == (H, I) and list(got) == ids
    for e, x in zip(ids, exs):
        y = got[e]
        for p, q in ((x.gu, y.gu), (x.dn, y.dn)):
            assert torch.equal(p.base, q.base) and torch.equal(p.var, q.var) and (p.rk, 0) == (q.rk, q.bk)
            assert q.p4 is None and q.d4 is None and q.flags is None
        assert torch.equal(y.sc[2], x.sc[2]) and torch.equal(y.sc[4], x.sc[4]) and y.signs is y.sc[2]
        assert (y.rg, y.rd, y.had_dn) == (x.rg, x.rd, 128)
        if x.rg + x.rd:
            assert torch.equal(y.lr, x.lr) and y.lr4 is not None
        else:
            assert y.lr is None and y.lr4 is None
        # level-2 row of the loaded expert: same fields as the original's, at the new addresses
        r = M.entry(y, 2)
        assert int(r[0]) == 2 and int(r[1]) == y.gu.base.data_ptr() and int(r[2]) == 0 and int(r[16]) == x.rg and int(r[19]) == 0


def test_resident_optional_keys_and_refusals(tmp_path):
    H, I = 256, 512
    exs = [_lr_expert(H, I, 20, 1, 1)]
    p1 = str(tmp_path / "a.pt")
    resident.save(_rank_layer(exs, [0], H, I, had_dn=512), p1)
    assert torch.load(p1, weights_only=True)["in_had_down"] == 512
    assert resident.load(p1, "cpu")[0][0].had_dn == 512
    # Hadamard width from the rank's index when the file has no key of its own
    root = tmp_path / "art"
    (root / "res" / "rank1").mkdir(parents=True)
    p2 = str(root / "res" / "rank1" / "L7.pt")
    resident.save(_rank_layer(exs, [0], H, I), p2)
    assert resident.load(p2, "cpu")[0][0].had_dn == 128            # no index file
    resident._rank_layers.cache_clear()
    (root / "rank1.json").write_text(json.dumps({"layers": {"7": {"in_had_down": 512}, "8": {}}}))
    assert resident.load(p2, "cpu")[0][0].had_dn == 512
    # base codes other than 0 -> v2 with per-expert lists; the loaded expert carries them into table word 19
    exs[0].gu.bk = 1
    p3 = str(tmp_path / "b.pt")
    resident.save(_rank_layer(exs, [0], H, I), p3)
    d = torch.load(p3, weights_only=True)
    assert d["format"] == "nq-res-v2" and d["bk_gu"] == [1] and d["bk_dn"] == [0]
    y = resident.load(p3, "cpu")[0][0]
    assert y.gu.bk == 1 and int(M.entry(y, 2)[19]) == 1
    exs[0].gu.bk = 0
    # not a resident file / a file that would need unpickling of objects
    p4 = str(tmp_path / "c.pt")
    torch.save({"format": "something-else"}, p4)
    with pytest.raises(ValueError, match="not a resident file"):
        resident.load(p4, "cpu")
    torch.save({"format": "nq-res-v1", "obj": types.SimpleNamespace(a=1)}, p4)
    with pytest.raises(Exception, match="(?i)weights_only|unsupported|allowed"):
        resident.load(p4, "cpu")
    assert not os.path.exists(p1 + ".tmp")
