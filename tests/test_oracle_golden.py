"""Oracle and host format code against the golden fixtures written by tests/golden/make_fixtures.py
(outputs of the reference's own CPU decoder: sm120/moe.py dense_W / Expert.ref / moe_ref / pack_words and
sm120/ref15_spec.py decode_unit). CPU only."""
import glob
import os

import numpy as np
import pytest
import torch

from nestquant_amd import format as F
from oracle import nq_oracle as O
from tests.util import oracle_plane, rel_err, same_f16, u32

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
PROJ_FILES = sorted(glob.glob(os.path.join(GOLD, "proj_rk*_var*.npz")))


def test_fixture_inventory():
    assert len(PROJ_FILES) == 8 and len(glob.glob(os.path.join(GOLD, "proj_bk1_rk*.npz"))) == 2
    for f in ("nested_units.npz", "nested_interleaved_units.npz", "layer_small.npz", "pack_words.npz"):
        assert os.path.exists(os.path.join(GOLD, f))


@pytest.mark.parametrize("path", PROJ_FILES, ids=[os.path.basename(p)[:-4] for p in PROJ_FILES])
def test_dense_decode_matches_reference(path):
    z = np.load(path)
    N, K, rk = int(z["N"]), int(z["K"]), int(z["rk"])
    nrec = (N // 16) * (K // 128) * 32
    var = z["var"] if z["var"].size else None
    res = O.unpack_words(z["p4"], nrec, O.rbits(rk))
    p = O.Plane(N, K, u32(torch.from_numpy(z["base"])).reshape(-1, 4), rk=rk, res=res, d4=u32(torch.from_numpy(z["d4"])), var=var)
    W2 = O.dense_W(p, 2); W4 = O.dense_W(p, 4)
    assert same_f16(W2, z["W2"].view(np.float16)) == 0
    assert same_f16(W4, z["W4"].view(np.float16)) == 0
    # a decoder that ignored the residual plane, or the sign plane, must not pass by accident
    assert same_f16(W2, z["W4"].view(np.float16)) > 1000
    if var is not None:
        q = O.Plane(N, K, p.base, rk=rk, res=res, d4=p.d4, var=None)
        assert same_f16(O.dense_W(q, 2), z["W2"].view(np.float16)) > 1000


@pytest.mark.parametrize("path", PROJ_FILES, ids=[os.path.basename(p)[:-4] for p in PROJ_FILES])
def test_package_generator_reproduces_reference_planes(path):
    """nestquant_amd.format.Proj draws in the reference's order: same seed -> same planes, block words and signs"""
    z = np.load(path)
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = F.Proj(int(z["N"]), int(z["K"]), gen, None, int(z["rk"]), ("exh", int(z["mbn_offset"])), var=bool(z["var"].size))
    assert np.array_equal(p.base.numpy(), z["base"]) and np.array_equal(p.p4.numpy(), z["p4"])
    assert np.array_equal(p.d4.numpy(), z["d4"])
    if z["var"].size:
        assert np.array_equal(p.var.numpy(), z["var"])
    assert p.p4.numel() * 4 == F.proj_sizes(p.N, p.K, None, p.rk)["p4"]


def test_pack_words_matches_reference():
    z = np.load(os.path.join(GOLD, "pack_words.npz"))
    for c in range(10):
        w = z[f"w{c}"]; want = z[f"p{c}"]
        bits = O.rbits(c)
        assert np.array_equal(O.pack_words(w, bits).view(np.int32), want)
        got = F.pack_words(torch.from_numpy(w.astype(np.int64)), bits)
        assert np.array_equal(got.numpy(), want)
        assert np.array_equal(F.unpack_words(torch.from_numpy(want), 96, bits).numpy().astype(np.uint32), w)
        assert np.array_equal(O.unpack_words(want, 96, bits), w)


def test_nested_levels_match_reference_generic_decoder():
    """level 3 (K=1 plane) and nested level 4 (K=2 over P3 || P4) through the reference's decode_unit(Kr=(KA, MASK))"""
    z = np.load(os.path.join(GOLD, "nested_units.npz"))
    n = z["base"].shape[0]
    base = z["base"].reshape(n * 32, 4); p3 = z["p3"].reshape(n * 32, 2); p4 = z["p4"].reshape(n * 32, 2)
    p = O.Plane(16, 128 * n, base, p3=p3, d3=z["d3"].astype(np.uint32), p4n=p4, d4n=z["d4"].astype(np.uint32))
    for lv, key in ((2, "U2"), (3, "U3"), (4, "U4")):
        W = O.dense_W(p, lv, nested=True)
        for u in range(n):
            assert same_f16(W[:, 128 * u:128 * (u + 1)], z[key][u].view(np.float16)) == 0, (lv, u)
    assert same_f16(O.dense_W(p, 3, nested=True), O.dense_W(p, 4, nested=True)) > 1000


def test_interleaved_two_plane_level4_matches_reference_generic_decoder():
    """window code 12: level 4 over P3 and P4 interleaved bit by bit = the reference's decode_unit(Kr=2) over lane records that the
    fixture script interleaved on Python integers; level 3 over the same P3 as before; the interleave itself by its definition"""
    z = np.load(os.path.join(GOLD, "nested_interleaved_units.npz"))
    n = z["base"].shape[0]
    base = z["base"].reshape(n * 32, 4); p3 = z["p3"].reshape(n * 32, 2); p4 = z["p4"].reshape(n * 32, 2)
    p = O.Plane(16, 128 * n, base, p3=p3, d3=z["d3"].astype(np.uint32), p4n=p4, d4n=z["d4"].astype(np.uint32))
    for lv, key in ((2, "U2"), (3, "U3"), (4, "U4")):
        W = O.dense_W(p, lv, nested="interleave")
        for u in range(n):
            assert same_f16(W[:, 128 * u:128 * (u + 1)], z[key][u].view(np.float16)) == 0, (lv, u)
    assert same_f16(O.dense_W(p, 4, nested="interleave"), O.dense_W(p, 4, nested=True)) > 1000       # not the concatenated record
    il = O.interleave_words(p3, p4)
    as_int = lambda w: [sum(int(v) << (32 * i) for i, v in enumerate(r)) for r in w]
    for a, b, v in zip(as_int(p3[:9]), as_int(p4[:9]), as_int(il[:9])):
        assert all((v >> (2 * i)) & 1 == (a >> i) & 1 and (v >> (2 * i + 1)) & 1 == (b >> i) & 1 for i in range(64))
    t = F.interleave_words(torch.from_numpy(p3.astype(np.int64)), torch.from_numpy(p4.astype(np.int64)))
    assert np.array_equal(t.numpy().astype(np.uint32), il)
    # every 16-bit window of the 2-bits-per-step stream holds eight bits of each plane: state(j) of lane 0, read off the planes
    a, b = as_int(p3[:1])[0], as_int(p4[:1])[0]
    for j in (0, 5, 31, 40, 56):
        st = (as_int(il[:1])[0] >> (2 * j)) & 0xFFFF
        assert all((st >> (2 * m)) & 1 == (a >> (j + m)) & 1 and (st >> (2 * m + 1)) & 1 == (b >> (j + m)) & 1 for m in range(8))


def _small_layer():
    z = np.load(os.path.join(GOLD, "layer_small.npz"))
    H, I = int(z["H"]), int(z["I"])
    ex = [F.Expert(H, I, seed=int(z["seeds"][i]), dev="cpu", rk_gu=int(z["rk_gu"][i]), rk_dn=int(z["rk_dn"][i]),
                   var=bool(z["var"][i])) for i in range(4)]
    return z, H, I, ex


def test_expert_and_layer_math_match_reference():
    z, H, I, ex = _small_layer()
    levels = z["levels"].tolist()
    assert np.array_equal(ex[1].signs.numpy().view(np.uint16), z["signs1"])
    x = z["x"].view(np.float16); rw = z["rw"].view(np.float16); sel = z["sel"]

    def dense(e):
        return (O.dense_W(oracle_plane(ex[e].gu), levels[e]).astype(np.float32),
                O.dense_W(oracle_plane(ex[e].dn), levels[e]).astype(np.float32))

    y1 = O.expert_forward(x.astype(np.float32), *dense(1), ex[1].signs.numpy())
    assert rel_err(y1, z["y_expert1_level4"]) < 2e-6
    y = O.moe_forward(dense, levels, lambda e: ex[e].signs.numpy(), x, sel, rw)
    # row-by-row and batched fp32 matmuls differ in summation order; where that flips one of the fp16 activation
    # roundings an element moves by one fp16 ulp, so the layer bar is the reference's own kernel-vs-ref band (<= 1e-4)
    assert rel_err(y, z["y"]) < 1e-4
    # sensitivity: dropping the zero-weight rule or the level-0 rule, or swapping gate and up, must fail this bar
    Wgu, Wdn = dense(1)
    swapped = np.concatenate([Wgu[I:], Wgu[:I]])
    assert rel_err(O.expert_forward(x.astype(np.float32), swapped, Wdn, ex[1].signs.numpy()), z["y_expert1_level4"]) > 1e-2
    # distance to the pipeline without the two fp16 activation roundings stays inside the 1e-3 budget
    y_pure = O.moe_forward(dense, levels, lambda e: ex[e].signs.numpy(), x, sel, rw, round_acts=False)
    assert 0 < rel_err(y, y_pure) < 1e-3


LR_NAMES = ("Vg", "U2g", "U2u", "U4g", "U4u", "Vd", "U2d", "U4d")


def had512_lr_layer():
    """the optional-feature fixture: experts rebuilt from their seeds, low-rank tensors and expected outputs as stored"""
    z = np.load(os.path.join(GOLD, "layer_had512_lr.npz"))
    H, I = int(z["H"]), int(z["I"])
    ex = [F.Expert(H, I, seed=int(z["seeds"][i]), dev="cpu", rk_gu=int(z["rk_gu"][i]), rk_dn=int(z["rk_dn"][i])) for i in range(3)]
    lr = [{n: z[f"lr{i}_{n}"].view(np.float16) for n in LR_NAMES} for i in range(3)]
    return z, H, I, ex, lr


def test_had512_and_low_rank_plane_match_reference():
    """in_had_down = 512 and the low-rank plane (reference Expert.ref, sm120/moe.py:196-210), alone and together"""
    z, H, I, ex, lr = had512_lr_layer()
    levels = z["levels"].tolist()
    x = z["x"].view(np.float16); rw = z["rw"].view(np.float16); sel = z["sel"]

    def dense(e):
        return (O.dense_W(oracle_plane(ex[e].gu), levels[e]).astype(np.float32),
                O.dense_W(oracle_plane(ex[e].dn), levels[e]).astype(np.float32))

    sg = lambda e: ex[e].signs.numpy()
    y_h = O.moe_forward(dense, levels, sg, x, sel, rw, had_dn=512)
    y_hl = O.moe_forward(dense, levels, sg, x, sel, rw, had_dn=512, lr=lambda e: lr[e])
    y_l = O.moe_forward(dense, levels, sg, x, sel, rw, lr=lambda e: lr[e])
    assert rel_err(y_h, z["y_had512"]) < 1e-4
    assert rel_err(y_hl, z["y_had512_lr"]) < 1e-4
    assert rel_err(y_l, z["y_lr"]) < 1e-4
    # the three variants and the plain layer are far apart, so a dropped term or a wrong width fails the bars above
    y_0 = O.moe_forward(dense, levels, sg, x, sel, rw)
    for a, b in ((y_h, y_0), (y_l, y_0), (y_hl, y_h), (y_hl, y_l)):
        assert rel_err(a, b) > 1e-2
    # U4 terms count at level 4 only: expert 0 is at level 2
    lr_no4 = [dict(d) for d in lr]
    for n in ("U4g", "U4u", "U4d"):
        lr_no4[0][n] = np.zeros_like(lr[0][n])
    assert np.array_equal(O.moe_forward(dense, levels, sg, x, sel, rw, lr=lambda e: lr_no4[e]), y_l)


def mask_proj(rk):
    """the mask-mode fixture: the projection rebuilt from its seed, and the reference's level-4 dense decode of it"""
    z = np.load(os.path.join(GOLD, f"mask_rk{rk}.npz"))
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = F.Proj(int(z["N"]), int(z["K"]), gen, int(z["nm"]), rk, ("exh", int(z["mbn_offset"])), var=bool(z["var"]))
    return z, p


@pytest.mark.parametrize("rk", [0, 7])
def test_mask_mode_matches_reference(rk):
    """flags per strip, residual plane compact over the flagged chunks, the other chunks at level 2 (sm120/moe.py:134-155)"""
    z, p = mask_proj(rk)
    assert np.array_equal(p.flags.numpy(), z["flags"])             # same generator order as the reference's Proj
    assert p.p4w.shape[0] == p.z["nrec_r"] == 16 * 1 * 32 and p.d4.numel() == 16
    assert len(set(z["flags"][:8].tolist())) == 1 and len(set(z["flags"][8:].tolist())) == 1   # uniform over 8-strip groups
    P = oracle_plane(p)
    W4 = O.dense_W(P, 4)
    assert same_f16(W4, z["W4"].view(np.float16)) == 0
    # two of three chunks of every strip stay at level 2, the flagged one differs
    W2 = O.dense_W(P, 2)
    on = ((z["flags"][:, None] >> np.arange(3)[None]) & 1).astype(bool)
    for s_ in (0, 9):
        for c in range(3):
            blk = (slice(16 * s_, 16 * s_ + 16), slice(128 * c, 128 * c + 128))
            assert (same_f16(W4[blk], W2[blk]) == 0) == (not on[s_, c])


BK_FILES = sorted(glob.glob(os.path.join(GOLD, "proj_bk1_rk*.npz")))


@pytest.mark.parametrize("path", BK_FILES, ids=[os.path.basename(p)[:-4] for p in BK_FILES])
def test_base_code_1_matches_reference(path):
    """K = 1.75 base plane (window pattern (1, 0xEEEE), 112-bit records in the sub-array layout, table word 19) against the
    reference's dense decode (sm120/moe.py:138-140); the package's generator draws the same planes from the same seed"""
    z = np.load(path)
    N, K, rk = int(z["N"]), int(z["K"]), int(z["rk"])
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = F.Proj(N, K, gen, None, rk, ("exh", int(z["mbn_offset"])), var=bool(z["var"].size), bk=1)
    assert np.array_equal(p.base.numpy(), z["base"]) and np.array_equal(p.p4.numpy(), z["p4"]) and np.array_equal(p.d4.numpy(), z["d4"])
    assert p.base.numel() * 4 == F.proj_sizes(N, K, None, rk, 1)["base"] == (N // 16) * (K // 128) * 32 * 14
    op = oracle_plane(p)
    assert op.bk == 1 and op.base.shape == ((N // 16) * (K // 128) * 32, 4) and int(op.base[:, 3].max()) < 1 << 16
    W2 = O.dense_W(op, 2); W4 = O.dense_W(op, 4)
    assert same_f16(W2, z["W2"].view(np.float16)) == 0 and same_f16(W4, z["W4"].view(np.float16)) == 0
    # the two independent state walks agree on the 112-bit records, and reading them as K = 2 records is far off
    assert np.array_equal(O.lane_sums(op.base, 1), O.hash_sum(O.ring_states(op.base, 1)).reshape(-1, 64))
    wrong = O.Plane(N, K, np.concatenate([op.base, op.base], 0)[: op.base.shape[0]], rk=rk, res=op.res, d4=op.d4, var=op.var, bk=0)
    assert same_f16(O.dense_W(wrong, 2), z["W2"].view(np.float16)) > 1000


@pytest.mark.parametrize("rk", [0, 7])
def test_rings_of_two_lanes_match_reference(rk):
    """the same planes read as rings of G = 2 records: the reference's dense_W(p, level, G=2) at levels 2 and 4"""
    z = np.load(os.path.join(GOLD, f"proj_g2_rk{rk}.npz"))
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = oracle_plane(F.Proj(int(z["N"]), int(z["K"]), gen, None, rk, ("exh", int(z["mbn_offset"]))))
    assert same_f16(O.dense_W(p, 2, G=2), z["W2"].view(np.float16)) == 0
    assert same_f16(O.dense_W(p, 4, G=2), z["W4"].view(np.float16)) == 0
    # the G = 4 reading differs where a window crosses the end of a record whose ring neighbour changed (lanes 1 and 3)
    assert same_f16(O.dense_W(p, 4), z["W4"].view(np.float16)) > 100
