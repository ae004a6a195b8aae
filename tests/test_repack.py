"""Shards -> record file + index + resident files (nestquant_amd/repack.py, the reference's streaming/repack.py), on the CPU."""
import json
import os

import numpy as np
import pytest
import torch

from nestquant_amd import nqload, p4rec, repack as RP, resident
from tests.shards import synth_layer, write_layer


def _layers(root, specs):
    for L, kw in specs.items():
        man, parts = synth_layer(**kw)
        write_layer(root, L, man, parts, "pt" if L % 2 else "safetensors")


def test_repack_writes_records_index_and_resident_files(tmp_path):
    root, out = str(tmp_path / "fit"), str(tmp_path / "out")
    ids = (1, 5, 6)
    _layers(root, {3: dict(seed=3, H=128, res_K=2.25, rg=2, rd=1, experts=ids), 4: dict(seed=4, H=128, res_K=2.25, rg=0, rd=0, experts=ids)})
    lines = []
    done = RP.repack(root, out, tp=2, layers=[3, 4, 5], dev="cpu", ne=8, log=lines.append)
    assert done == [(3, 0), (3, 1), (4, 0), (4, 1)] and any("L5: not fitted" in s for s in lines)
    for r in range(2):
        with open(f"{out}/rank{r}.json") as f:
            idx = json.load(f)
        assert idx["format"] == "nq-p4rec-v1" and (idx["tp"], idx["rank"], idx["L0"], idx["NE"]) == (2, r, 3, 8)
        assert sorted(idx["layers"]) == ["3", "4"] and idx["layers"]["3"]["experts"] == list(ids)
        assert idx["layers"]["3"]["rg"] == {"1": 2, "5": 2, "6": 2} and idx["layers"]["4"]["rd"] == {"1": 0, "5": 0, "6": 0}
        assert idx["rec_bytes"] % 4096 == 0 and list(idx["seg"]) == list(p4rec.SEGS)
        size = os.path.getsize(f"{out}/rank{r}.bin")
        assert size == (1 * 8 + 6 + 1) * idx["rec_bytes"]            # last record: layer 4, expert 6
        fd = os.open(f"{out}/rank{r}.bin", os.O_RDONLY)
        try:
            buf = torch.empty(idx["rec_bytes"] + 16, dtype=torch.uint8)
            for L in (3, 4):
                RL = nqload.RankLayer(root, L, r, 2, dev="cpu")
                lay = p4rec.layout(RL.ex[1], RL.H, RL.I)
                assert lay["rec_bytes"] == idx["rec_bytes"] and {k: list(v) for k, v in lay["seg"].items()} == idx["seg"]
                for E in ids:
                    rec = RP.read_record(fd, idx, L, E, buf)
                    assert rec.numel() == idx["rec_bytes"] and rec.numpy().tobytes() == p4rec.pack(RL.ex[E], lay)
                    assert RP.record_offset(idx, L, E) == ((L - 3) * 8 + E) * idx["rec_bytes"]
                got, H, I = resident.load(f"{out}/res/rank{r}/L{L}.pt", "cpu")
                assert (H, I) == (128, 1024) and sorted(got) == list(ids)
                for E in ids:
                    assert torch.equal(got[E].gu.base, RL.ex[E].gu.base) and torch.equal(got[E].dn.base, RL.ex[E].dn.base)
                    assert torch.equal(got[E].sc[2], RL.ex[E].sc[2]) and (got[E].rg, got[E].rd) == (RL.ex[E].rg, RL.ex[E].rd)
            with pytest.raises(KeyError):
                RP.read_record(fd, idx, 3, 2, buf)                       # an id the layer does not hold
            with pytest.raises(KeyError):
                RP.read_record(fd, idx, 5, 1, buf)
            with pytest.raises(ValueError):
                RP.read_record(fd, idx, 3, 1, buf[: 100])
        finally:
            os.close(fd)
    # a second run has nothing to do; a layer that arrives later is added without touching the others
    before = {r: open(f"{out}/rank{r}.bin", "rb").read() for r in range(2)}
    assert RP.repack(root, out, tp=2, layers=[3, 4], dev="cpu", ne=8, log=lines.append) == []
    _layers(root, {5: dict(seed=5, H=128, res_K=2.25, experts=(0, 7))})
    assert RP.repack(root, out, tp=2, layers=[3, 4, 5], dev="cpu", ne=8, log=lines.append) == [(5, 0), (5, 1)]
    for r in range(2):
        now = open(f"{out}/rank{r}.bin", "rb").read()
        assert now[: len(before[r])] == before[r] and len(now) > len(before[r])
        with open(f"{out}/rank{r}.json") as f:
            idx = json.load(f)
        assert sorted(idx["layers"]) == ["3", "4", "5"] and idx["layers"]["5"]["experts"] == [0, 7]
    # a layer with another residual code has another record layout: refused, the files stay as they are
    _layers(root, {6: dict(seed=6, H=128, res_K=2.5625, experts=(0,))})
    with pytest.raises(ValueError, match="record layout"):
        RP.repack(root, out, tp=2, layers=[6], dev="cpu", ne=8, log=lines.append)
    with pytest.raises(ValueError, match="outside"):
        RP.repack(root, str(tmp_path / "o2"), tp=2, layers=[5], dev="cpu", ne=4, log=lines.append)       # expert 7 >= NE


def test_slot_size_override_and_command_line(tmp_path, capsys):
    root, out = str(tmp_path / "fit"), str(tmp_path / "out")
    _layers(root, {3: dict(seed=13, H=128, res_K=2.25, experts=(0, 2))})
    RL = nqload.RankLayer(root, 3, 0, 4, dev="cpu")
    lay = p4rec.layout(RL.ex[0], RL.H, RL.I)
    big = lay["rec_bytes"] + 8192
    RP.repack(root, out, tp=4, layers=[3], rec_bytes=big, dev="cpu", log=lambda s: None)
    with open(f"{out}/rank0.json") as f:
        idx = json.load(f)
    assert idx["rec_bytes"] == big and idx["NE"] == 256 and idx["L0"] == 3
    raw = np.fromfile(f"{out}/rank0.bin", np.uint8)
    rec = raw[2 * big: 3 * big]
    want = np.frombuffer(p4rec.pack(RL.ex[2], lay), np.uint8)
    assert np.array_equal(rec[: want.size], want) and not rec[want.size:].any()
    assert RP.parse_layers("7") == [7] and RP.parse_layers("3-6") == [3, 4, 5, 6]
    assert RP.main([]) == 2 and "rank{r}.bin" in capsys.readouterr().out
