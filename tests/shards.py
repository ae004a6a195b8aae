"""Synthetic layers in the production shard format (nestquant-v1), for the loader's tests and for the script that writes its
golden fixtures: seeded random ring streams, block words, sign variants, scale vectors and low-rank factors with the shard
geometry of the format (8 shards of 256 intermediate channels; gate / up sharded over strips, down over chunks)."""
import json
import os

import torch

NSH = 8
I_ALL = 256 * NSH
RING_BITS = {2: 512, 1.75: 448, 2.25: 576, 2.3125: 592, 2.5625: 656, 2.5: 640, 3: 768}    # 4 lanes x record bits


def synth_layer(seed, H, res_K, base_K=2, var=True, rg=0, rd=0, experts=(0,), shards=range(NSH), had_dn=None):
    """-> (manifest dict, {shard id: {expert id: {projection: planes}}}) of a layer with hidden size H"""
    g = torch.Generator().manual_seed(seed)
    rnd_u8 = lambda n: torch.randint(0, 256, (n,), generator=g, dtype=torch.int64).to(torch.uint8)
    rnd_h = lambda *sh: ((torch.randint(0, 2, sh, generator=g) * 2 - 1) * (0.5 + torch.rand(*sh, generator=g))).half()
    geo = {"gate": dict(k=H, n=I_ALL, tk=H // 128, tn=I_ALL // 16, shard_axis="n"),
           "up": dict(k=H, n=I_ALL, tk=H // 128, tn=I_ALL // 16, shard_axis="n"),
           "down": dict(k=I_ALL, n=H, tk=I_ALL // 128, tn=H // 16, shard_axis="k")}
    meta = {}
    for pn, m in geo.items():
        m = dict(m, res_rule=dict(kind="uniform", K=res_K))
        if base_K != 2:
            m["base_K"] = base_K
        if var:
            m["base_var"] = "sign"
        if rg + rd:
            m["lr"] = dict(shared_V=True)
        meta[pn] = m
    man = dict(format="nestquant-v1", layer=0, experts=list(experts), tp=NSH, proj_meta=meta, config={})
    if had_dn:
        man["config"]["in_had_down"] = had_dn
    parts = {s: {} for s in shards}
    for E in experts:
        su = {pn: {lv: rnd_h(geo[pn]["k"]) for lv in (2, 4)} for pn in geo}
        sv = {pn: {lv: rnd_h(geo[pn]["n"]) for lv in (2, 4)} for pn in geo}
        Vg = (torch.randn(rg, H, generator=g) * 0.5).half()
        lr = {"gate": (Vg, rnd_h(rg, I_ALL) * 0.02, rnd_h(rg, I_ALL) * 0.02),
              "up": (Vg, rnd_h(rg, I_ALL) * 0.02, rnd_h(rg, I_ALL) * 0.02),
              "down": ((torch.randn(rd, I_ALL, generator=g) * 0.5).half(), rnd_h(rd, H) * 0.02, rnd_h(rd, H) * 0.02)}
        for s in range(NSH):                             # every shard is drawn, so a subset sees the same bytes as the whole
            ex = {}
            for pn, m in geo.items():
                units = 16 * m["tk"] if pn != "down" else 2 * m["tn"]
                Mb = torch.randint(120, 256, (units,), generator=g)
                N = torch.minimum((torch.rand(units, generator=g) * 0.8 * Mb).round().long(), 257 - Mb)
                d = dict(base=rnd_u8(units * 8 * RING_BITS[base_K] // 8), p4=rnd_u8(units * 8 * RING_BITS[res_K] // 8),
                         word=(Mb | (N << 8)).to(torch.int32))
                ks = slice(s * m["k"] // NSH, (s + 1) * m["k"] // NSH) if pn == "down" else slice(0, m["k"])
                ns = slice(0, m["n"]) if pn == "down" else slice(s * m["n"] // NSH, (s + 1) * m["n"] // NSH)
                d.update(suh2=su[pn][2][ks].clone(), svh2=sv[pn][2][ns].clone(), suh4=su[pn][4][ks].clone(), svh4=sv[pn][4][ns].clone())
                if var:
                    d["var"] = torch.randint(0, 2, (units * 8,), generator=g).to(torch.uint8)
                if rg + rd:
                    V, U2, U4 = lr[pn]
                    if pn == "down":
                        d.update(lrV=V[:, ks].clone(), lrU2=U2.clone(), lrU4=U4.clone())
                    else:
                        d.update(lrU2=U2[:, ns].clone(), lrU4=U4[:, ns].clone())
                        if pn == "up":
                            d["lrV_from"] = "gate"
                        else:
                            d["lrV"] = V.clone()
                ex[pn] = d
            if s in parts:
                parts[s][E] = ex
    return man, parts


def write_layer(root, L, man, parts, container="pt"):
    """the layer as files: <root>/L{L}/manifest.json + tp{s}.pt, or <root>/layers/L{L}/... + tp{s}.safetensors in the
    container whose metadata carries the dict's skeleton (tensors as {"T": key}, other values as {"V": value})"""
    d = f"{root}/L{L}" if container == "pt" else f"{root}/layers/L{L}"
    os.makedirs(d, exist_ok=True)
    with open(f"{d}/manifest.json", "w") as f:
        json.dump(man, f)
    for s, part in parts.items():
        if container == "pt":
            torch.save(part, f"{d}/tp{s}.pt")
            continue
        from safetensors.torch import save_file
        tensors = {}

        def tree(x, key):
            if isinstance(x, dict):
                return {"D": [[k, tree(v, f"{key}.{k}")] for k, v in x.items()]}
            if torch.is_tensor(x):
                tensors[key] = x.contiguous().clone()
                return {"T": key}
            return {"V": x}

        skeleton = {"D": [[E, tree(ex, f"E{E}")] for E, ex in part.items()]}
        save_file(tensors, f"{d}/tp{s}.safetensors",
                  metadata=dict(format="nestquant-v1-tp-safetensors", layer=str(L), shard=str(s), tp=str(NSH),
                                experts=",".join(str(E) for E in part), tree=json.dumps(skeleton, separators=(",", ":"))))
    return d
