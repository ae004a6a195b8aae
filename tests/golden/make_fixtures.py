"""Writes the golden fixtures of tests/golden/ by running the REFERENCE's own CPU decoder once, in the build container.

Run only where /root/reference exists:   python tests/golden/make_fixtures.py
It imports sm120/ref15_spec.py (numpy only) and sm120/moe.py (torch CPU; its `build` import is replaced by an empty
stub the way the reference's own sm120/verify_res2.py:9-15 does) and stores inputs + outputs as small .npz files.
The fixtures pin what closed forms cannot: lane-minor ring concatenation, bit order of the ring streams, the dense
row/column scatter, sub-array order and tail packing, the gate|up row order, and the layer math conventions.
Nothing here is read at test time except the .npz files it wrote.
"""
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/sm120"
OUT = os.path.dirname(os.path.abspath(__file__))


def load_reference():
    sys.modules["build"] = types.SimpleNamespace(get=lambda *a, **k: None, get_sal=lambda *a, **k: None)
    sys.path.insert(0, REF)
    import moe as R          # reference torch decoder (CPU)
    import ref15_spec as SP  # reference numpy bit-level spec
    # The reference's Proj.to() reads s.bw, which Proj.__init__ only sets for base codes != 0 (sm120/moe.py:84-88,105);
    # a class-level default lets its Expert constructor run for the K=2 base used everywhere here.
    R.Proj.bw = None
    return R, SP


def base_code(R):
    """7. base window code 1 (K = 1.75 base plane in the sub-array layout, table word 19): planes from the reference
    generator, dense decode by the reference at levels 2 and 4; residual codes 3 and 9 as in the build that uses it"""
    for rk, var in ((3, False), (9, True)):
        seed = 3000 + rk
        gen = torch.Generator().manual_seed(seed)
        p = R.Proj(32, 256, gen, None, rk, ("exh", 700 * rk + 3), var=var, bk=1)
        W2 = R.dense_W(p, 2, 4, torch.float16)
        W4 = R.dense_W(p, 4, 4, torch.float16)
        np.savez_compressed(os.path.join(OUT, f"proj_bk1_rk{rk}.npz"), seed=seed, N=32, K=256, rk=rk, bk=1, mbn_offset=700 * rk + 3,
                            base=p.base.numpy(), p4=p.p4.numpy(), d4=p.d4.numpy(), var=(p.var.numpy() if var else np.zeros(0, np.uint8)),
                            W2=W2.numpy().view(np.uint16), W4=W4.numpy().view(np.uint16))


def rings_of_two(R):
    """8. the same planes read as rings of G = 2 lanes (the reference kernel's second variant, sm120/nqmoe.cu:223-228):
    the reference's dense decode with G = 2 at levels 2 and 4"""
    for rk in (0, 7):
        seed = 4000 + rk
        gen = torch.Generator().manual_seed(seed)
        p = R.Proj(32, 256, gen, None, rk, ("exh", 500 * rk + 9))
        np.savez_compressed(os.path.join(OUT, f"proj_g2_rk{rk}.npz"), seed=seed, N=32, K=256, rk=rk, mbn_offset=500 * rk + 9,
                            W2=R.dense_W(p, 2, 2, torch.float16).numpy().view(np.uint16),
                            W4=R.dense_W(p, 4, 2, torch.float16).numpy().view(np.uint16))


def shard_loader():
    """9. the production shard loader (sm120/nqload.py: group_art + kernel_expert on the CPU): synthetic shards of
    tests/shards.py (seeded, so the fixture stores the outputs only), the group of rank 1 of 4 (shards 2, 3)"""
    sys.path.insert(0, os.path.dirname(os.path.dirname(OUT)))
    from tests.shards import synth_layer
    import nqload as NL          # imports the reference's nq_decode (torch only at import) and moe (stubbed build)
    cases = {"a": dict(seed=5101, H=128, res_K=2.25, base_K=2, var=True, rg=2, rd=1),
             "b": dict(seed=5102, H=128, res_K=2.5625, base_K=1.75, var=True, rg=0, rd=0)}
    for name, kw in cases.items():
        man, parts = synth_layer(**kw)
        ex = NL.kernel_expert(NL.group_art(parts, man, 0, [2, 3]), dev="cpu")[0]
        out = dict(I=ex.I, **{k: np.array(v) for k, v in kw.items()})
        for pn, p in (("gu", ex.gu), ("dn", ex.dn)):
            out.update({f"{pn}_base": p.base.numpy(), f"{pn}_p4": p.p4.numpy(), f"{pn}_d4": p.d4.numpy(), f"{pn}_var": p.var.numpy(),
                        f"{pn}_rk": p.rk, f"{pn}_bk": p.bk})
        out.update(sc2=ex.sc[2].numpy().view(np.uint16), sc4=ex.sc[4].numpy().view(np.uint16))
        if ex.lr is not None:
            out.update(lr=ex.lr.numpy().view(np.uint16), lr4=ex.lr4.numpy().view(np.uint16))
        out["p4_bytes"] = NL.p4_bytes(ex)
        np.savez_compressed(os.path.join(OUT, f"shards_{name}.npz"), **out)


def nested_interleaved():
    """10. two-plane level 4 with the planes interleaved bit by bit (stream bit 2 i = bit i of P3's lane record, bit 2 i + 1 =
    bit i of P4's): the reference's generic decode_unit with Kr = 2 over the interleaved lane records, and level 3 (Kr = (1, 0))
    over P3 alone from the same planes. The interleave is done here on Python integers, one record at a time. Needs only the
    reference's numpy spec."""
    sys.path.insert(0, REF)
    import ref15_spec as SP
    rng = np.random.default_rng(12)
    units = []
    for u in range(4):
        base = rng.integers(0, 2**32, (32, 4), dtype=np.uint64).astype(np.uint32)
        p3 = rng.integers(0, 2**32, (32, 2), dtype=np.uint64).astype(np.uint32)
        p4 = rng.integers(0, 2**32, (32, 2), dtype=np.uint64).astype(np.uint32)
        Mb3 = int(rng.integers(1, 256)); N3 = int(rng.integers(0, min(255, 257 - Mb3) + 1))
        Mb4 = int(rng.integers(120, 256)); N4 = int(rng.integers(0, 257 - Mb4 + 1))
        mixed = np.zeros((32, 4), np.uint32)
        for lane in range(32):
            a = int(p3[lane, 0]) | int(p3[lane, 1]) << 32
            b = int(p4[lane, 0]) | int(p4[lane, 1]) << 32
            v = 0
            for i in range(64):
                v |= ((a >> i) & 1) << (2 * i) | ((b >> i) & 1) << (2 * i + 1)
            mixed[lane] = [(v >> (32 * k)) & 0xFFFFFFFF for k in range(4)]
        bs = SP.rings_from_lane_words(base, 128)
        Q2, Q3 = SP.decode_unit(bs, SP.rings_from_lane_words(p3, 64), Mb3, N3, Kb=2, Kr=(1, 0))
        _, Q4 = SP.decode_unit(bs, SP.rings_from_lane_words(mixed, 128), Mb4, N4, Kb=2, Kr=2)
        units.append(dict(base=base, p3=p3, p4=p4, d3=Mb3 | N3 << 8, d4=Mb4 | N4 << 8,
                          U2=SP.to_unit(Q2).T.astype(np.float16).view(np.uint16),      # [16 rows, 128 cols]
                          U3=SP.to_unit(Q3).T.astype(np.float16).view(np.uint16),
                          U4=SP.to_unit(Q4).T.astype(np.float16).view(np.uint16)))
    np.savez_compressed(os.path.join(OUT, "nested_interleaved_units.npz"),
                        **{k: np.stack([np.asarray(u[k]) for u in units]) for k in units[0]})


def main():
    R, SP = load_reference()

    # 1. projections: planes from the reference generator, dense decode by the reference at levels 2 and 4
    for rk in (0, 3, 6, 7, 8, 9):
        for var in (False, True):
            if var and rk not in (0, 7):
                continue
            seed = 1000 + 10 * rk + int(var)
            gen = torch.Generator().manual_seed(seed)
            p = R.Proj(32, 256, gen, None, rk, ("exh", 4000 * rk + 17), var=var)
            W2 = R.dense_W(p, 2, 4, torch.float16)
            W4 = R.dense_W(p, 4, 4, torch.float16)
            np.savez_compressed(
                os.path.join(OUT, f"proj_rk{rk}_var{int(var)}.npz"), seed=seed, N=32, K=256, rk=rk,
                mbn_offset=4000 * rk + 17, base=p.base.numpy(), p4=p.p4.numpy(), d4=p.d4.numpy(),
                var=(p.var.numpy() if var else np.zeros(0, np.uint8)),
                W2=W2.numpy().view(np.uint16), W4=W4.numpy().view(np.uint16))

    # 2. nested levels through the reference's generic (KA, MASK) decoder: K=1 plane, and K=2 over P3 || P4
    rng = np.random.default_rng(7)
    units = []
    for u in range(4):
        base = rng.integers(0, 2**32, (32, 4), dtype=np.uint64).astype(np.uint32)
        p3 = rng.integers(0, 2**32, (32, 2), dtype=np.uint64).astype(np.uint32)
        p4 = rng.integers(0, 2**32, (32, 2), dtype=np.uint64).astype(np.uint32)
        Mb3, N3 = int(rng.integers(1, 256)), 0
        N3 = int(rng.integers(0, min(255, 257 - Mb3) + 1))
        Mb4 = int(rng.integers(120, 256)); N4 = int(rng.integers(0, 257 - Mb4 + 1))
        bs = SP.rings_from_lane_words(base, 128)
        r3 = SP.rings_from_lane_words(p3, 64)
        r4 = SP.rings_from_lane_words(np.concatenate([p3, p4], 1), 128)
        Q2, Q3 = SP.decode_unit(bs, r3, Mb3, N3, Kb=2, Kr=(1, 0))
        _, Q4 = SP.decode_unit(bs, r4, Mb4, N4, Kb=2, Kr=2)
        units.append(dict(base=base, p3=p3, p4=p4, d3=Mb3 | N3 << 8, d4=Mb4 | N4 << 8,
                          U2=SP.to_unit(Q2).T.astype(np.float16).view(np.uint16),      # [16 rows, 128 cols]
                          U3=SP.to_unit(Q3).T.astype(np.float16).view(np.uint16),
                          U4=SP.to_unit(Q4).T.astype(np.float16).view(np.uint16)))
    np.savez_compressed(os.path.join(OUT, "nested_units.npz"),
                        **{k: np.stack([np.asarray(u[k]) for u in units]) for k in units[0]})

    # 3. layer math: reference Expert.ref / moe_ref on CPU (H = I = 256, 4 experts, levels 2/4/4/0, var on expert 2)
    H = I = 256
    ex = [R.Expert(H, I, seed=300 + i, dev="cpu", rk_gu=(0, 3, 7, 0)[i], rk_dn=(0, 7, 0, 0)[i], var=(i == 2)) for i in range(4)]
    levels = [2, 4, 4, 0]
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(3, H, generator=g) * 0.05).half()
    sel = torch.tensor([[0, 1, 2, 3], [2, 0, 1, 3], [1, 2, 0, 3]])
    rw = (torch.rand(3, 4, generator=g) + 0.1)
    rw = (rw / rw.sum(1, keepdim=True)).half()
    rw[2, 1] = 0                                                     # a pick with zero weight is skipped
    y = R.moe_ref(ex, levels, x, sel, rw)
    y1 = ex[1].ref(x.float(), 4)
    np.savez_compressed(os.path.join(OUT, "layer_small.npz"), H=H, I=I, seeds=np.arange(300, 304), levels=np.array(levels),
                        rk_gu=np.array([0, 3, 7, 0]), rk_dn=np.array([0, 7, 0, 0]), var=np.array([0, 0, 1, 0]),
                        x=x.numpy().view(np.uint16), sel=sel.numpy(), rw=rw.numpy().view(np.uint16),
                        y=y.numpy(), y_expert1_level4=y1.numpy(), signs1=ex[1].signs.numpy().view(np.uint16))

    # 4. the reference's residual packer on every code (sub-array order and tail bits)
    g = torch.Generator().manual_seed(0)
    packs = {}
    for c in range(10):
        b = R.rbits(c); nw = (b + 31) // 32
        w = torch.randint(0, 2**32, (96, nw), generator=g, dtype=torch.int64)
        if b % 32:
            w[:, -1] &= (1 << (b % 32)) - 1
        packs[f"w{c}"] = w.numpy().astype(np.uint32)
        packs[f"p{c}"] = R.pack_words(w, b).numpy()
    np.savez_compressed(os.path.join(OUT, "pack_words.npz"), **packs)
    # 5. optional layer features of the reference's Expert.ref: Hadamard-512 on the down projection's input (in_had_down)
    #    and the low-rank plane (set_lr); H = 256, I = 512, 3 experts at levels 2 / 4 / 4
    H, I = 256, 512
    ex = [R.Expert(H, I, seed=700 + i, dev="cpu", rk_gu=(0, 7, 0)[i], rk_dn=(0, 0, 3)[i]) for i in range(3)]
    levels = [2, 4, 4]
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(2, H, generator=g) * 0.05).half()
    sel = torch.tensor([[0, 1, 2], [2, 1, 0]])
    rw = (torch.rand(2, 3, generator=g) + 0.1)
    rw = (rw / rw.sum(1, keepdim=True)).half()
    out = dict(H=H, I=I, seeds=np.arange(700, 703), levels=np.array(levels), rk_gu=np.array([0, 7, 0]), rk_dn=np.array([0, 0, 3]),
               x=x.numpy().view(np.uint16), sel=sel.numpy(), rw=rw.numpy().view(np.uint16))
    for e in ex:
        e.had_dn = 512
    out["y_had512"] = R.moe_ref(ex, levels, x, sel, rw).numpy()
    rg, rd = 2, 3
    names = ("Vg", "U2g", "U2u", "U4g", "U4u", "Vd", "U2d", "U4d")
    shapes = ((rg, H), (rg, I), (rg, I), (rg, I), (rg, I), (rd, I), (rd, H), (rd, H))
    for i, e in enumerate(ex):
        t = [(torch.randn(*sh, generator=g) * (0.5 if n[0] == "V" else 0.02)).half() for n, sh in zip(names, shapes)]
        e.set_lr(*t)
        for n, v in zip(names, t):
            out[f"lr{i}_{n}"] = v.numpy().view(np.uint16)
    out["y_had512_lr"] = R.moe_ref(ex, levels, x, sel, rw).numpy()
    for e in ex:
        e.had_dn = 128
    out["y_lr"] = R.moe_ref(ex, levels, x, sel, rw).numpy()
    np.savez_compressed(os.path.join(OUT, "layer_had512_lr.npz"), **out)
    # 6. mask mode: nm flagged chunks per strip (here 1 of 3), the residual plane compact over them, flags uniform over each
    #    group of 8 strips (two groups here); unflagged chunks decode at level 2
    for rk, var in ((0, False), (7, True)):
        gen = torch.Generator().manual_seed(2000 + rk)
        p = R.Proj(256, 384, gen, 1, rk, ("exh", 900 * rk + 5), var=var)
        W4 = R.dense_W(p, 4, 4, torch.float16)
        np.savez_compressed(os.path.join(OUT, f"mask_rk{rk}.npz"), seed=2000 + rk, N=256, K=384, nm=1, rk=rk, mbn_offset=900 * rk + 5,
                            var=int(var), flags=p.flags.numpy(), W4=W4.numpy().view(np.uint16))
    base_code(R)
    rings_of_two(R)
    shard_loader()
    nested_interleaved()
    print("fixtures written to", OUT)


if __name__ == "__main__":
    if sys.argv[1:] == ["base_code"]:            # only the fixtures of section 7
        base_code(load_reference()[0])
    elif sys.argv[1:] == ["rings_of_two"]:       # only the fixtures of section 8
        rings_of_two(load_reference()[0])
    elif sys.argv[1:] == ["shard_loader"]:       # only the fixtures of section 9
        load_reference(); shard_loader()
    elif sys.argv[1:] == ["nested_interleaved"]:  # only the fixture of section 10
        nested_interleaved()
    else:
        main()
