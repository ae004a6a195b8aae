"""Resident planes of one layer of one tensor-parallel rank: the file that holds everything the GPU keeps for the whole
run (formats nq-res-v1 / nq-res-v2).

Host-side mirror of the reference's streaming/resident.py (`save` :19, `load` :33, `had_width` :46): same key names,
shapes and dtypes, so a file written by either side loads on the other. One file per (rank, layer); a torch.save'd dict

    format      'nq-res-v1', or 'nq-res-v2' when some expert has a base window code other than 0
    L rank tp   layer index, rank, tensor-parallel degree          H I       hidden size, this rank's intermediate size
    experts     expert ids, in the order of the stacked tensors
    rk_gu rk_dn residual window code per expert                    rg rd     low-rank ranks per expert (0..RMAX)
    gu_base dn_base [E, n] int32   2-bit base planes               gu_var dn_var [E, units] uint8  variant bits
    sc2 sc4     [E, 3H + 3I] fp16  sign / scale vectors of levels 2 and 4
    lr          [E, lr_len(H, I, RMAX, RMAX)] fp16, per expert V_g | U2_g | U2_u | V_d | U2_d at its own ranks, zero padded
    bk_gu bk_dn (v2 only) base window code per expert              in_had_down (only when not 128) Hadamard width of the
                                                                   down projection's input

The residual planes, their block words and the U4 factors are not here: they are the expert's record (p4rec.py) and a
loaded expert has p4 = d4 = None, so its level-2 row comes from moe.entry(ex, 2) and its level-4 row from
p4rec.row(ex, lay, slot_ptr, moe.entry).

Files are read with torch.load(weights_only=True): the dict holds tensors, lists, ints and strings only, so nothing in a
file is executed. v2 files load with each projection's `bk`; the kernels serve base codes 0 and 1, and the table-row
check refuses any other, loudly, when such an expert is set into a layer.
"""
import functools
import json
import os

import torch

RMAX = 4
FORMATS = ("nq-res-v1", "nq-res-v2")
_STACKED = ("gu_base", "gu_var", "dn_base", "dn_var", "sc2", "sc4", "lr")


def lr_len(H, I, rg, rd):
    """fp16 elements of the resident low-rank buffer at ranks rg, rd"""
    return rg * (H + 2 * I) + rd * (I + H)


def save(RL, path):
    """RL: a rank's layer (attributes L, rank, tp, H, I, experts = ids, ex = {id: expert}, optional had_dn); each expert
    has gu / dn with base, var, rk (and bk), sc = {2: ..., 4: ...}, rg, rd and lr (or None)"""
    ids = list(RL.experts)
    exs = [RL.ex[e] for e in ids]
    H, I = RL.H, RL.I
    stack = lambda get: torch.stack([get(x).detach().cpu() for x in exs])
    lr = torch.zeros(len(ids), lr_len(H, I, RMAX, RMAX), dtype=torch.float16)
    for i, x in enumerate(exs):
        if getattr(x, "lr", None) is not None:
            lr[i, : x.lr.numel()] = x.lr.detach().cpu()
    bk = lambda p: int(getattr(p, "bk", 0) or 0)
    d = {"format": FORMATS[0], "L": RL.L, "rank": RL.rank, "tp": RL.tp, "H": H, "I": I, "experts": ids,
         "rk_gu": [int(x.gu.rk) for x in exs], "rk_dn": [int(x.dn.rk) for x in exs],
         "rg": [int(x.rg) for x in exs], "rd": [int(x.rd) for x in exs],
         "gu_base": stack(lambda x: x.gu.base), "gu_var": stack(lambda x: x.gu.var),
         "dn_base": stack(lambda x: x.dn.base), "dn_var": stack(lambda x: x.dn.var),
         "sc2": stack(lambda x: x.sc[2]), "sc4": stack(lambda x: x.sc[4]), "lr": lr}
    bk_gu, bk_dn = [bk(x.gu) for x in exs], [bk(x.dn) for x in exs]
    if any(bk_gu) or any(bk_dn):
        d.update(format=FORMATS[1], bk_gu=bk_gu, bk_dn=bk_dn)
    w = int(getattr(RL, "had_dn", 128) or 128)
    if w != 128:
        d["in_had_down"] = w
    tmp = path + ".tmp"
    torch.save(d, tmp)
    os.replace(tmp, path)


class ResidentProj:
    """resident half of one projection: base plane and variant bits; p4 / d4 come from a record slot"""

    def __init__(s, base, var, rk, bk):
        s.base, s.var, s.rk, s.bk = base, var, rk, bk
        s.p4 = s.d4 = s.flags = s.fl = None


class ResidentExpert:
    """expert as loaded from a resident file: the fields moe.entry and p4rec.row read"""

    def __init__(s, gu, dn, H, I, rg, rd, sc2, sc4, lr, lr4, had_dn):
        s.gu, s.dn, s.H, s.I, s.rg, s.rd = gu, dn, H, I, rg, rd
        s.sc = {2: sc2, 4: sc4}
        s.signs = sc2
        s.lr, s.lr4, s.had_dn = lr, lr4, had_dn


def load(path, dev="cuda"):
    """-> ({expert id: ResidentExpert}, H, I), the stacked tensors moved to `dev` once and sliced per expert"""
    d = torch.load(path, map_location="cpu", mmap=True, weights_only=True)
    if not isinstance(d, dict) or d.get("format") not in FORMATS:
        raise ValueError(f"{path}: not a resident file (format {d.get('format') if isinstance(d, dict) else type(d)})")
    H, I = int(d["H"]), int(d["I"])
    ids = list(d["experts"])
    for k in _STACKED:
        if d[k].shape[0] != len(ids):
            raise ValueError(f"{path}: {k} holds {d[k].shape[0]} experts, the id list {len(ids)}")
    t = {k: d[k].to(dev) for k in _STACKED}
    zeros = [0] * len(ids)
    bk_gu, bk_dn = d.get("bk_gu", zeros), d.get("bk_dn", zeros)
    width = had_width(path, d)
    u4_stub = torch.zeros(1, dtype=torch.float16, device=dev)    # level-2 rows never read U4; level-4 rows take it from the slot
    out = {}
    for i, e in enumerate(ids):
        rg, rd = int(d["rg"][i]), int(d["rd"][i])
        has_lr = rg + rd > 0
        out[e] = ResidentExpert(ResidentProj(t["gu_base"][i], t["gu_var"][i], int(d["rk_gu"][i]), int(bk_gu[i])),
                                ResidentProj(t["dn_base"][i], t["dn_var"][i], int(d["rk_dn"][i]), int(bk_dn[i])),
                                H, I, rg, rd, t["sc2"][i], t["sc4"][i],
                                t["lr"][i, : lr_len(H, I, rg, rd)] if has_lr else None, u4_stub if has_lr else None, width)
    return out, H, I


def had_width(path, d):
    """in_had_down of a resident file: its own key when present, else the layer's entry in rank{r}.json three directories
    up (<root>/rank{r}.json for <root>/res/rank{r}/L{L}.pt), else 128"""
    if "in_had_down" in d:
        return int(d["in_had_down"])
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(path))))
    layers = _rank_layers(os.path.join(root, f"rank{d['rank']}.json"))
    return int(layers.get(str(d["L"]), {}).get("in_had_down", 128))


@functools.lru_cache(None)
def _rank_layers(index_path):
    if not os.path.exists(index_path):
        return {}
    with open(index_path) as f:
        return json.load(f)["layers"]
