"""Loader of the production shard format (nestquant-v1): <root>/L{L}/tp{s}.pt (or <root>/layers/L{L}/tp{s}.safetensors)
+ manifest.json -> experts in the kernels' plane layout.

Host-side mirror of the reference's sm120/nqload.py (group_art :19, repack :40, cat_proj :70, kernel_expert :80,
had_width :104, p4_bytes :108, layer_dir :113, load_part :118, RankLayer :130); same names and argument meaning, so code
written against the reference's loader reads the same here.

The format (reference threads/12-reference-encoder/nq_decode.py:1-40, nq_layer.py:107-132):
  a layer is cut into NSH = 8 shards of 256 intermediate channels; shard s holds, per expert and projection
      base  uint8   ring streams of the 2-bit base plane (K = proj_meta.base_K, default 2), LSB first in every byte, 8 rings of
                    4 lanes per 16 x 128 unit, the units of gate / up in (strip, chunk) order, those of down in (strip, chunk)
                    order inside the shard's two chunks
      p4    uint8   ring streams of the residual plane (uniform K = proj_meta.res_rule.K)
      word  int32   block word Mb | N << 8 per unit            var   uint8  sign variant of each ring (bit 0)
      suh2 svh2 suh4 svh4   fp16 input / output scale vectors of levels 2 and 4 (the shard's slice on the sharded side)
      lrV lrU2 lrU4         fp16 low-rank plane (optional; `lrV_from` = 'gate' when up shares gate's V)
  rank r of a tensor-parallel run of degree tp owns the shards [r * 8 / tp, (r + 1) * 8 / tp): unit order is shard-major,
  so the group is a self-contained expert of I = 256 * 8 / tp.

What the repack does: lane l of a ring owns the stream's bits [l * bits, (l + 1) * bits) (bits = record size of the window
code), so a unit's 32 records are its stream cut every `bits` bits; units are reordered from storage order to the kernels'
(strip-major, chunk-minor) and the record words packed into the sub-array layout of format.pack_words. No value is decoded
on the way: the kernels read what the file holds.

Files: tp{s}.pt is read with torch.load(weights_only=True) (the reference's own loader unpickles freely; a shard holds
dicts, strings and tensors only, so the restricted loader reads it, and a file it refuses is reported, not executed); the
safetensors container (reference threads/25-campaign/nq25_st.py:31-66) holds the same dict, its skeleton as JSON in the
metadata field `tree`.
"""
import json
import os
import struct
import types

import torch

from .format import RK_OF, RKP, lane_words_from_rings, pack_words, proj_sizes, rbits

PROJ = ("gate", "up", "down")
NSH = 8
SCALE_PLANE = {2: "base", 4: "p4"}
ST_FORMAT = "nestquant-v1-tp-safetensors"


def unit_order(tk, tn, shard_axis):
    """storage order of a projection's units (reference nq_decode.py:166-173): flat unit id a * tn + c (a = 128-column chunk,
    c = 16-row strip), shard-major, then strip, then chunk; a shard is 16 strips (axis 'n') or 2 chunks (axis 'k')"""
    a = torch.arange(tk).repeat_interleave(tn)
    c = torch.arange(tn).repeat(tk)
    shard = c // 16 if shard_axis == "n" else a // 2
    return torch.argsort((shard * tn + c) * tk + a)


def record_order(tk, tn, shard_axis):
    """perm with  kernel_units = storage_units[perm]: the kernels number units strip-major (unit = strip * tk + chunk)"""
    flat = unit_order(tk, tn, shard_axis)
    return torch.argsort((flat % tn) * tk + flat // tn)


def _cat(ts):
    return torch.cat([t.cpu() for t in ts]) if len(ts) else torch.zeros(0)


def group_art(parts, man, E, ss):
    """Expert E of the contiguous shard group ss as one artifact {proj: {base, p4, meta}} with the group's geometry.
    parts[s] = the loaded shard s (load_part); man = the layer's manifest."""
    g = len(ss)
    art = {}
    for pn in PROJ:
        meta = dict(man["proj_meta"][pn])
        ps = [parts[s][E][pn] for s in ss]
        along = lambda key: torch.cat([p[key] for p in ps])
        if pn == "down":                                 # sharded over its input columns: chunks
            meta.update(k=meta["k"] * g // NSH, tk=meta["tk"] * g // NSH)
            su = {2: along("suh2"), 4: along("suh4")}
            sv = {2: ps[0]["svh2"], 4: ps[0]["svh4"]}
        else:                                            # sharded over its output rows: strips
            meta.update(n=meta["n"] * g // NSH, tn=meta["tn"] * g // NSH)
            su = {2: ps[0]["suh2"], 4: ps[0]["suh4"]}
            sv = {2: along("svh2"), 4: along("svh4")}
        base = dict(shards=[p["base"] for p in ps], suh=su[2], svh=sv[2])
        if "var" in ps[0]:
            base["var"] = [p["var"] for p in ps]
        p4 = dict(shards=[p["p4"] for p in ps], word=[p["word"] for p in ps], suh=su[4], svh=sv[4])
        if "lrU2" in ps[0]:
            if pn == "down":                             # V sliced over the input, U whole in every shard
                V, U2, U4 = torch.cat([p["lrV"] for p in ps], 1), ps[0]["lrU2"], ps[0]["lrU4"]
            else:                                        # V whole (possibly kept by gate only), U sliced over the output
                V = parts[ss[0]][E][ps[0].get("lrV_from", pn)]["lrV"]
                U2, U4 = torch.cat([p["lrU2"] for p in ps], 1), torch.cat([p["lrU4"] for p in ps], 1)
            base["lr"] = dict(V=V, U2=U2)
            p4["lr"] = dict(U4=U4)
        art[pn] = dict(base=base, p4=p4, meta=meta)
    return art


def _code_of(K, what):
    K = float(K)
    if K not in RK_OF:
        raise ValueError(f"{what}: no window code for K = {K}")
    return RK_OF[K]


def repack(P, dev="cuda", want_Q=False):
    """one projection of an artifact -> (planes in the kernels' layout, None). The planes object has the fields of
    format.Proj that moe.entry, p4rec and resident read: N K rk bk z base p4 d4 var flags fl, and until kernel_expert drops
    them the unpacked record words bw / p4w that cat_proj joins.
    The reference returns the rotated dense matrices of its CPU decoder as second value when want_Q is set; here the dense
    check is moe.dequant on the loaded expert, so want_Q must stay False."""
    if want_Q:
        raise NotImplementedError("no host decoder in the product path: decode the loaded expert with moe.dequant instead")
    m = P["meta"]
    tk, tn = m["tk"], m["tn"]
    U = tk * tn
    rule = m["res_rule"]
    if rule["kind"] != "uniform":
        raise NotImplementedError(f"residual rule {rule['kind']!r}: the kernels take one window code per projection")
    rk = _code_of(rule["K"], "res_rule.K")
    bk = _code_of(m.get("base_K", 2), "base_K")
    perm = record_order(tk, tn, m["shard_axis"])

    def records(shards, code):
        bits = rbits(code)
        raw = _cat(shards).reshape(U, 32 * bits // 8)[perm]
        return lane_words_from_rings(raw, bits)

    p = types.SimpleNamespace(N=m["n"], K=m["k"], rk=rk, bk=bk, z=proj_sizes(m["n"], m["k"], None, rk, bk), flags=None, fl=None)
    p.bw = records(P["base"]["shards"], bk)
    if bk == 0:                                          # one uint4 per record: the words themselves
        w = p.bw.reshape(-1)
        p.base = torch.where(w >= 2**31, w - 2**32, w).to(torch.int32).to(dev)
    else:
        p.base = pack_words(p.bw, rbits(bk)).to(dev)
    p.p4w = records(P["p4"]["shards"], rk)
    p.p4 = pack_words(p.p4w, rbits(rk)).to(dev)
    word = _cat(P["p4"]["word"]).long()[perm]
    p.Mb, p.Nn = (word & 255).to(dev), ((word >> 8) & 255).to(dev)
    p.d4 = (p.Mb | (p.Nn << 8)).to(torch.int32)
    p.var = None
    if m.get("base_var"):
        if m["base_var"] != "sign":
            raise NotImplementedError(f"base variant set {m['base_var']!r}: the kernels know the sign variant only")
        v = _cat(P["base"]["var"]).long().reshape(U, 8)[perm]
        p.var = ((v & 1) << torch.arange(8)).sum(1).to(torch.uint8).to(dev)
    return p, None


def cat_proj(a, b, dev="cuda"):
    """gate and up stacked into one projection of 2I rows (gate's strips first)"""
    if a.rk != b.rk or a.bk != b.bk:
        raise ValueError("gate and up must share the residual and the base window code (one code per projection pair)")
    if (a.var is None) != (b.var is None):
        raise ValueError("gate and up must both carry sign variants or neither")
    p = types.SimpleNamespace(N=a.N + b.N, K=a.K, rk=a.rk, bk=a.bk, z=proj_sizes(a.N + b.N, a.K, None, a.rk, a.bk), flags=None, fl=None)
    p.bw = torch.cat([a.bw, b.bw])
    p.base = torch.cat([a.base, b.base]) if p.bk == 0 else pack_words(p.bw, rbits(p.bk)).to(dev)   # sub-arrays span all records
    p.p4w = torch.cat([a.p4w, b.p4w])
    p.p4 = pack_words(p.p4w, rbits(p.rk)).to(dev)
    p.Mb, p.Nn, p.d4 = torch.cat([a.Mb, b.Mb]), torch.cat([a.Nn, b.Nn]), torch.cat([a.d4, b.d4])
    p.var = None if a.var is None else torch.cat([a.var, b.var])
    return p


def kernel_expert(art, dev="cuda", want_Q=False):
    """artifact -> (ex, scales, (None, None, None)): ex has gu / dn planes, H, I, sc = {2, 4: [su_g | sv_g | sv_u | su_d |
    sv_o | su_u] fp16}, signs = sc[2], and the low-rank buffers lr = V_g | U2_g | U2_u | V_d | U2_d, lr4 = U4_g | U4_u | U4_d
    with ranks rg, rd (None / 0 without the plane); scales(level) rebuilds one scale vector."""
    g, _ = repack(art["gate"], dev, want_Q)
    u, _ = repack(art["up"], dev, want_Q)
    d, _ = repack(art["down"], dev, want_Q)
    ex = types.SimpleNamespace(gu=cat_proj(g, u, dev), dn=d, H=d.N, I=d.K, lr=None, lr4=None, rg=0, rd=0)
    for p in (ex.gu, ex.dn):
        del p.bw, p.p4w

    def lr_of(pn):                                       # a projection of rank 0 has no 'lr' entry
        P = art[pn]
        n, k = P["meta"]["n"], P["meta"]["k"]
        if "lr" not in P["base"]:
            z = lambda c: torch.zeros(0, c, dtype=torch.float16)
            return z(k), z(n), z(n)
        return P["base"]["lr"]["V"].cpu(), P["base"]["lr"]["U2"].cpu(), P["p4"]["lr"]["U4"].cpu()

    (Vg, U2g, U4g), (Vu, U2u, U4u), (Vd, U2d, U4d) = (lr_of(pn) for pn in PROJ)
    if not torch.equal(Vg, Vu):
        raise ValueError("gate and up must share the low-rank input directions V")
    ex.rg, ex.rd = Vg.shape[0], Vd.shape[0]
    flat = lambda *t: torch.cat([x.reshape(-1) for x in t]).half().contiguous().to(dev)
    if ex.rg + ex.rd:
        ex.lr, ex.lr4 = flat(Vg, U2g, U2u, Vd, U2d), flat(U4g, U4u, U4d)

    def scales(level):
        pl = SCALE_PLANE[level]
        s = lambda pn, key: art[pn][pl][key].half().to(dev)
        return torch.cat([s("gate", "suh"), s("gate", "svh"), s("up", "svh"), s("down", "suh"), s("down", "svh"), s("up", "suh")])

    ex.sc = {level: scales(level) for level in (2, 4)}
    ex.signs = ex.sc[2]
    return ex, scales, (None, None, None)


def had_width(man):
    """width of the Hadamard rotation of the down projection's input of a layer manifest; absent = 128"""
    return int(man.get("config", {}).get("in_had_down", 128))


def p4_bytes(ex):
    """bytes of the streamed level-4 part of one expert on one rank: residual planes + block words (+ U4 of the low-rank plane)"""
    b = sum(p.p4.numel() * 4 + p.d4.numel() * 4 for p in (ex.gu, ex.dn))
    return b + (0 if ex.lr4 is None else ex.lr4.numel() * 2)


def layer_dir(root, L):
    """<root>/L{L} (output of a fit) or <root>/layers/L{L} (published layout)"""
    d = f"{root}/L{L}"
    return d if os.path.exists(f"{d}/manifest.json") else f"{root}/layers/L{L}"


def _untree(node, tensor):
    if "D" in node:
        return {k: _untree(v, tensor) for k, v in node["D"]}
    if "T" in node:
        return tensor(node["T"])
    return node["V"]


def load_part(d, i):
    """shard i of the layer directory d: tp{i}.pt, else the safetensors container tp{i}.safetensors (the same dict:
    {expert id: {projection: {plane: tensor or value}}})"""
    pt = f"{d}/tp{i}.pt"
    if os.path.exists(pt):
        return torch.load(pt, map_location="cpu", weights_only=True)
    import safetensors.torch
    with open(f"{d}/tp{i}.safetensors", "rb") as f:      # one sequential read
        blob = f.read()
    n = struct.unpack("<Q", blob[:8])[0]
    meta = json.loads(blob[8:8 + n]).get("__metadata__", {})
    if meta.get("format") != ST_FORMAT:
        raise ValueError(f"{d}/tp{i}.safetensors: format {meta.get('format')!r}, expected {ST_FORMAT!r}")
    tensors = safetensors.torch.load(blob)
    return _untree(json.loads(meta["tree"]), tensors.__getitem__)


class RankLayer:
    """All experts (or the listed ones) of layer L for rank `rank` of a tensor-parallel run of degree tp.
    Attributes as the reference's: man, ss (shard ids), L rank tp, parts, experts (ids), ex {id: expert}, H, I, had_dn;
    the object is what resident.save takes."""

    def __init__(s, root, L, rank, tp=4, experts=None, dev="cuda"):
        if NSH % tp or not 0 <= rank < tp:
            raise ValueError(f"tp = {tp} must divide {NSH} and rank = {rank} lie below it")
        d = layer_dir(root, L)
        with open(f"{d}/manifest.json") as f:
            s.man = json.load(f)
        if s.man.get("format") != "nestquant-v1":
            raise ValueError(f"{d}/manifest.json: format {s.man.get('format')!r}, expected 'nestquant-v1'")
        g = NSH // tp
        s.ss = list(range(rank * g, (rank + 1) * g))
        s.L, s.rank, s.tp, s.dev = L, rank, tp, dev
        s.parts = {i: load_part(d, i) for i in s.ss}
        s.experts = [E for E in s.man["experts"] if experts is None or E in experts]
        s.ex = {E: kernel_expert(s.art(E), dev)[0] for E in s.experts}
        s.H, s.I = s.man["proj_meta"]["down"]["n"], s.man["proj_meta"]["down"]["k"] * g // NSH
        s.had_dn = had_width(s.man)
        if s.I % s.had_dn:
            raise ValueError(f"layer {L}: I = {s.I} is not a multiple of in_had_down = {s.had_dn}")
        for x in s.ex.values():
            x.had_dn = s.had_dn

    def art(s, E):
        return group_art(s.parts, s.man, E, s.ss)

    def slot_bytes(s, align=256):
        """size of a level-4 slot of this layer: the largest expert's streamed part, rounded up to `align`"""
        m = max(p4_bytes(e) for e in s.ex.values())
        return (m + align - 1) // align * align
