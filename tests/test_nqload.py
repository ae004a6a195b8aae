"""The production shard loader (nestquant_amd/nqload.py) against the reference's own loader and against the format's
definition.

tests/golden/shards_{a,b}.npz hold what the reference's sm120/nqload.py (group_art + kernel_expert on the CPU) made of the
seeded synthetic layers of tests/shards.py: every plane, block word, variant byte, scale vector and low-rank buffer must
come out bit for bit. The second half checks the loader against the format's words rather than against another loader:
a unit's place in the files, lane l of a ring = the stream's bits [l * bits, (l + 1) * bits), files and containers."""
import os

import numpy as np
import pytest
import torch

from nestquant_amd import format as F, nqload as NL, resident
from tests.shards import NSH, synth_layer, write_layer

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("name", ["a", "b"])
def test_loader_matches_the_reference_loader(name):
    z = np.load(os.path.join(GOLD, f"shards_{name}.npz"))
    kw = dict(seed=int(z["seed"]), H=int(z["H"]), res_K=float(z["res_K"]), base_K=float(z["base_K"]), var=bool(z["var"]),
              rg=int(z["rg"]), rd=int(z["rd"]))
    man, parts = synth_layer(**kw)
    ex, scales, Q = NL.kernel_expert(NL.group_art(parts, man, 0, [2, 3]), dev="cpu")
    assert Q == (None, None, None)
    assert (ex.H, ex.I, ex.rg, ex.rd) == (kw["H"], int(z["I"]), kw["rg"], kw["rd"]) and ex.I == 512
    for pn, p in (("gu", ex.gu), ("dn", ex.dn)):
        assert (p.rk, p.bk) == (int(z[f"{pn}_rk"]), int(z[f"{pn}_bk"]))
        for k in ("base", "p4", "d4", "var"):
            got = getattr(p, k).numpy()
            assert got.dtype == z[f"{pn}_{k}"].dtype and np.array_equal(got, z[f"{pn}_{k}"]), (pn, k)
        assert p.base.numel() * 4 == p.z["base"] and p.p4.numel() * 4 == p.z["p4"] and p.d4.numel() * 4 == p.z["d4"]
    for lv in (2, 4):
        assert np.array_equal(ex.sc[lv].numpy().view(np.uint16), z[f"sc{lv}"])
        assert torch.equal(scales(lv), ex.sc[lv])
    assert ex.signs is ex.sc[2]
    if kw["rg"] + kw["rd"]:
        assert np.array_equal(ex.lr.numpy().view(np.uint16), z["lr"]) and np.array_equal(ex.lr4.numpy().view(np.uint16), z["lr4"])
        assert ex.lr.numel() == resident.lr_len(ex.H, ex.I, ex.rg, ex.rd)
    else:
        assert ex.lr is None and ex.lr4 is None
    assert NL.p4_bytes(ex) == int(z["p4_bytes"])


def test_unit_order_is_shard_major_then_strip_then_chunk():
    # gate / up: shards of 16 strips; inside, strips in order, each with all its chunks
    tk, tn = 3, 48
    want = [a * tn + c for c in range(tn) for a in range(tk)]
    assert NL.unit_order(tk, tn, "n").tolist() == want
    # down: shards of 2 chunks; inside, strips in order, each with the shard's two chunks
    tk, tn = 6, 5
    want = [a * tn + c for s in range(3) for c in range(tn) for a in (2 * s, 2 * s + 1)]
    assert NL.unit_order(tk, tn, "k").tolist() == want
    # the kernels' order: unit = strip * tk + chunk
    flat = NL.unit_order(tk, tn, "k")[NL.record_order(tk, tn, "k")]
    assert flat.tolist() == [a * tn + c for c in range(tn) for a in range(tk)]


def _streams_of(words, bits):
    """ring streams of record words by the format's definition, bit by bit: ring r of a unit is the concatenation of its four
    lanes' records, lane 0 first, written LSB first"""
    w = words.numpy().astype(np.uint64)
    out = np.zeros(w.shape[0] * bits // 8, np.uint8)
    pos = 0
    for rec in w:
        for b in range(bits):
            if (int(rec[b // 32]) >> (b % 32)) & 1:
                out[pos >> 3] |= 1 << (pos & 7)
            pos += 1
    return torch.from_numpy(out)


@pytest.mark.parametrize("base_K,res_K", [(2, 2.3125), (1.75, 2.25)])
def test_planes_written_unit_by_unit_come_back(base_K, res_K):
    """a down projection (the sharded-over-chunks case, where storage and kernel order differ most) built from known record
    words: each unit's streams go to the place the format gives it, the loader must return the words in the kernels' order"""
    H, g = 128, 2                                        # two shards: 4 chunks x 8 strips = 32 units
    tk, tn = 2 * g, H // 16
    bk, rk = F.RK_OF[base_K], F.RK_OF[res_K]
    gen = torch.Generator().manual_seed(77)

    def words(bits):
        w = torch.randint(0, 2**32, (tk * tn * 32, (bits + 31) // 32), generator=gen, dtype=torch.int64)
        if bits % 32:
            w[:, -1] &= (1 << (bits % 32)) - 1
        return w

    bw, rw = words(F.rbits(bk)), words(F.rbits(rk))      # kernel order: record = (strip * tk + chunk) * 32 + ring * 4 + lane
    word = torch.randint(0, 2**16, (tk * tn,), generator=gen, dtype=torch.int64)
    var = torch.randint(0, 256, (tk * tn,), generator=gen, dtype=torch.int64)
    shards = []
    for s in range(g):
        base, p4, wd, vr = [], [], [], []
        for c in range(tn):                              # the shard's storage order: strip, then its two chunks
            for a in (2 * s, 2 * s + 1):
                u = c * tk + a
                base.append(_streams_of(bw[32 * u: 32 * u + 32], F.rbits(bk)))
                p4.append(_streams_of(rw[32 * u: 32 * u + 32], F.rbits(rk)))
                wd.append(int(word[u]))
                vr += [(int(var[u]) >> r) & 1 for r in range(8)]
        shards.append(dict(base=torch.cat(base), p4=torch.cat(p4), word=torch.tensor(wd, dtype=torch.int32),
                           var=torch.tensor(vr, dtype=torch.uint8)))
    meta = dict(k=128 * tk, n=H, tk=tk, tn=tn, shard_axis="k", res_rule=dict(kind="uniform", K=res_K), base_K=base_K, base_var="sign")
    P = dict(base=dict(shards=[d["base"] for d in shards], var=[d["var"] for d in shards]),
             p4=dict(shards=[d["p4"] for d in shards], word=[d["word"] for d in shards]), meta=meta)
    p, Q = NL.repack(P, dev="cpu")
    assert Q is None and (p.N, p.K, p.rk, p.bk) == (H, 128 * tk, rk, bk)
    assert torch.equal(p.bw, bw) and torch.equal(p.p4w, rw)
    assert torch.equal(F.unpack_words(p.p4, tk * tn * 32, F.rbits(rk)), rw)
    if bk == 0:
        assert torch.equal(p.base.long() & 0xFFFFFFFF, bw.reshape(-1))
    else:
        assert torch.equal(F.unpack_words(p.base, tk * tn * 32, F.rbits(bk)), bw)
    assert torch.equal(p.d4.long() & 0xFFFF, word) and torch.equal(p.Mb, word & 255) and torch.equal(p.Nn, word >> 8)
    assert torch.equal(p.var.long(), var)


def _same_expert(a, b):
    for pa, pb in ((a.gu, b.gu), (a.dn, b.dn)):
        assert (pa.N, pa.K, pa.rk, pa.bk) == (pb.N, pb.K, pb.rk, pb.bk)
        for k in ("base", "p4", "d4", "var"):
            assert torch.equal(getattr(pa, k), getattr(pb, k)), k
    assert all(torch.equal(a.sc[lv], b.sc[lv]) for lv in (2, 4)) and (a.rg, a.rd) == (b.rg, b.rd)
    assert (a.lr is None and b.lr is None) or (torch.equal(a.lr, b.lr) and torch.equal(a.lr4, b.lr4))


@pytest.mark.parametrize("container", ["pt", "safetensors"])
def test_rank_layer_from_files(tmp_path, container):
    man, parts = synth_layer(seed=31, H=128, res_K=2.25, var=True, rg=1, rd=2, experts=(3, 11, 12), had_dn=512)
    write_layer(str(tmp_path), 5, man, parts, container)
    RL = NL.RankLayer(str(tmp_path), 5, rank=3, tp=4, dev="cpu")
    assert RL.ss == [6, 7] and RL.experts == [3, 11, 12] and (RL.H, RL.I, RL.had_dn) == (128, 512, 512)
    assert sorted(RL.parts) == [6, 7] and list(RL.parts[6]) == [3, 11, 12]
    for E in RL.experts:
        _same_expert(RL.ex[E], NL.kernel_expert(NL.group_art(parts, man, E, [6, 7]), dev="cpu")[0])
        assert RL.ex[E].had_dn == 512
    # the shards differ from each other and the experts too: the group and the id matter
    assert not torch.equal(RL.ex[3].gu.base, RL.ex[11].gu.base)
    assert not torch.equal(RL.ex[3].gu.base, NL.kernel_expert(NL.group_art(parts, man, 3, [4, 5]), dev="cpu")[0].gu.base)
    want = max(NL.p4_bytes(x) for x in RL.ex.values())
    assert RL.slot_bytes() == (want + 255) // 256 * 256 and RL.slot_bytes(4096) % 4096 == 0
    # a subset of the experts, another degree: tp = 2 gives I = 1024; tp = 8 would give I = 256, below the rotation's width
    one = NL.RankLayer(str(tmp_path), 5, rank=1, tp=2, experts={11}, dev="cpu")
    assert one.experts == [11] and one.I == 1024 and one.ss == [4, 5, 6, 7]
    assert torch.equal(one.ex[11].gu.d4[32: 48], RL.ex[11].gu.d4[: 16])     # gate's strips of shard 6: third in one group, first in the other
    with pytest.raises(ValueError, match="in_had_down"):
        NL.RankLayer(str(tmp_path), 5, rank=6, tp=8, experts={11}, dev="cpu")
    # what a resident file keeps of the rank's layer loads back
    path = str(tmp_path / "res.pt")
    resident.save(RL, path)
    got, H, I = resident.load(path, "cpu")
    assert (H, I) == (128, 512) and sorted(got) == [3, 11, 12]
    for E in RL.experts:
        assert torch.equal(got[E].gu.base, RL.ex[E].gu.base) and torch.equal(got[E].dn.var, RL.ex[E].dn.var)
        assert torch.equal(got[E].sc[4], RL.ex[E].sc[4]) and torch.equal(got[E].lr, RL.ex[E].lr) and got[E].had_dn == 512


def test_whole_layer_as_one_group_matches_the_sizes_of_the_format(tmp_path):
    man, parts = synth_layer(seed=8, H=128, res_K=2.3125, var=False)
    ex = NL.kernel_expert(NL.group_art(parts, man, 0, list(range(NSH))), dev="cpu")[0]
    assert (ex.H, ex.I) == (128, 2048) and ex.gu.var is None and ex.dn.var is None
    assert ex.gu.N == 4096 and ex.gu.base.numel() * 4 == 4096 * 128 // 4
    assert ex.gu.p4.numel() * 4 == F.proj_sizes(4096, 128, None, 7)["p4"]
    assert ex.sc[2].numel() == 3 * 128 + 3 * 2048 and ex.lr is None and ex.rg == ex.rd == 0


def test_loader_refuses_what_the_kernels_do_not_serve(tmp_path):
    man, parts = synth_layer(seed=9, H=128, res_K=2.25, shards=[0, 1])
    art = NL.group_art(parts, man, 0, [0, 1])
    with pytest.raises(NotImplementedError, match="moe.dequant"):
        NL.repack(art["gate"], dev="cpu", want_Q=True)
    bad = dict(art["gate"], meta=dict(art["gate"]["meta"], res_rule=dict(kind="pos", K=2, K_hi=3, frac=0.5)))
    with pytest.raises(NotImplementedError, match="residual rule"):
        NL.repack(bad, dev="cpu")
    bad = dict(art["gate"], meta=dict(art["gate"]["meta"], res_rule=dict(kind="uniform", K=2.75)))
    with pytest.raises(ValueError, match="no window code"):
        NL.repack(bad, dev="cpu")
    bad = dict(art["gate"], meta=dict(art["gate"]["meta"], base_var="sg4"))
    with pytest.raises(NotImplementedError, match="sign variant"):
        NL.repack(bad, dev="cpu")
    g, _ = NL.repack(art["gate"], dev="cpu")
    other = dict(art["up"], meta=dict(art["up"]["meta"], res_rule=dict(kind="uniform", K=2)))
    other["p4"] = dict(other["p4"], shards=[t[: t.numel() * 128 // 144] for t in other["p4"]["shards"]])
    u, _ = NL.repack(other, dev="cpu")
    with pytest.raises(ValueError, match="share"):
        NL.cat_proj(g, u, dev="cpu")
    with pytest.raises(ValueError, match="must divide"):
        NL.RankLayer(str(tmp_path), 0, rank=0, tp=3)
    write_layer(str(tmp_path), 0, dict(man, format="something-else"), parts)
    with pytest.raises(ValueError, match="nestquant-v1"):
        NL.RankLayer(str(tmp_path), 0, rank=0, tp=4, dev="cpu")
    assert NL.had_width({}) == 128 and NL.had_width(dict(config=dict(in_had_down=512))) == 512
    assert NL.layer_dir(str(tmp_path), 0) == f"{tmp_path}/L0" and NL.layer_dir(str(tmp_path), 9) == f"{tmp_path}/layers/L9"
