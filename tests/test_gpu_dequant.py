"""HIP decoder (nq_dequant / nq_pf_decode through the C ABI) against the oracle and the golden fixtures: bit-exact fp16,
+0 and -0 identified (the reference's own rule, sm120/verify_ext.py:55)."""
import glob
import os

import numpy as np
import pytest
import torch

from nestquant_amd import _lib, format as F, moe as M
from oracle import nq_oracle as O
from tests.util import oracle_plane, same_f16

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda"


class _Ex:
    """duck-typed expert with one real projection (the other side is a tiny dummy) for single-projection decodes"""

    def __init__(s, p, mode, H, I):
        s.H, s.I, s.nested = H, I, p.nested
        s.gu = s.dn = p
        s.signs = torch.zeros(8, dtype=torch.float16, device=DEV)
        s.mode = mode
        s.lr = None


def gpu_dense(p, level, N, K, mode=0, l4code=None):
    """decode projection p (already on the device) as gate|up (mode 0: N = 2I, K = H) or down (mode 1); l4code: the window code
    nested level 4 reads P3 and P4 with (default: concatenated)"""
    H, I = (K, N // 2) if mode == 0 else (N, K)
    ex = _Ex(p, mode, H, I)
    if l4code is not None:
        ex.l4code = l4code
    if p.nested:
        p.slot = p.nested_plane()
    row = M.entry(ex, level)
    M.validate_row(row, 128, 128)                                 # field checks only; a lone projection may be small
    W = M.dequant(row.to(DEV), mode, H, I)
    torch.cuda.synchronize()
    return W.cpu().numpy()


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "proj_rk*_var*.npz"))), ids=lambda p: os.path.basename(p)[:-4])
def test_golden_projections(path):
    z = np.load(path)
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = F.Proj(int(z["N"]), int(z["K"]), gen, None, int(z["rk"]), ("exh", int(z["mbn_offset"])), var=bool(z["var"].size)).to(DEV)
    for mode in (0, 1):
        assert same_f16(gpu_dense(p, 2, p.N, p.K, mode), z["W2"].view(np.float16)) == 0
        assert same_f16(gpu_dense(p, 4, p.N, p.K, mode), z["W4"].view(np.float16)) == 0


def test_golden_nested_units():
    z = np.load(os.path.join(GOLD, "nested_units.npz"))
    n = z["base"].shape[0]
    gen = torch.Generator().manual_seed(0)
    p = F.Proj(16, 128 * n, gen, nested=True)
    p.base = torch.from_numpy(z["base"].reshape(-1).view(np.int32).copy())
    p.p3 = F.pack_words(torch.from_numpy(z["p3"].reshape(-1, 2).astype(np.int64)), 64)
    p.p4n = F.pack_words(torch.from_numpy(z["p4"].reshape(-1, 2).astype(np.int64)), 64)
    p.d3 = torch.from_numpy(z["d3"].astype(np.int32)); p.d4n = torch.from_numpy(z["d4"].astype(np.int32))
    p.to(DEV)
    for lv, key in ((2, "U2"), (3, "U3"), (4, "U4")):
        W = gpu_dense(p, lv, 16, 128 * n, mode=1)
        for u in range(n):
            assert same_f16(W[:, 128 * u:128 * (u + 1)], z[key][u].view(np.float16)) == 0, (lv, u)


def test_golden_interleaved_nested_units():
    """window code 12 (P3 and P4 interleaved bit by bit) on the fixture the reference's generic decode_unit wrote; both dense
    decoders (stand-alone and the multi-expert prefill decode)"""
    z = np.load(os.path.join(GOLD, "nested_interleaved_units.npz"))
    n = z["base"].shape[0]
    gen = torch.Generator().manual_seed(0)
    p = F.Proj(16, 128 * n, gen, nested=True)
    p.base = torch.from_numpy(z["base"].reshape(-1).view(np.int32).copy())
    p.p3 = F.pack_words(torch.from_numpy(z["p3"].reshape(-1, 2).astype(np.int64)), 64)
    p.p4n = F.pack_words(torch.from_numpy(z["p4"].reshape(-1, 2).astype(np.int64)), 64)
    p.d3 = torch.from_numpy(z["d3"].astype(np.int32)); p.d4n = torch.from_numpy(z["d4"].astype(np.int32))
    p.to(DEV)
    for lv, key in ((2, "U2"), (3, "U3"), (4, "U4")):
        W = gpu_dense(p, lv, 16, 128 * n, mode=1, l4code=F.CODE_L4B)
        for u in range(n):
            assert same_f16(W[:, 128 * u:128 * (u + 1)], z[key][u].view(np.float16)) == 0, (lv, u)


@pytest.mark.parametrize("var", [False, True])
def test_interleaved_nested_projection_vs_oracle(var):
    """a projection of several strips and chunks at levels 3 and interleaved 4, sign plane on and off, against the numpy oracle"""
    gen = torch.Generator().manual_seed(31)
    p = F.Proj(64, 512, gen, None, 0, "rand", var=var, nested=True)
    op = oracle_plane(p)
    p.to(DEV)
    for mode in (0, 1):
        assert same_f16(gpu_dense(p, 4, 64, 512, mode=mode, l4code=F.CODE_L4B), O.dense_W(op, 4, nested="interleave")) == 0
        assert same_f16(gpu_dense(p, 3, 64, 512, mode=mode, l4code=F.CODE_L4B), O.dense_W(op, 3, nested=True)) == 0


@pytest.mark.parametrize("rk", range(10))
@pytest.mark.parametrize("var", [False, True])
def test_every_residual_code(rk, var):
    """4 strips x 4 chunks as the reference's verify_ext.py (a): every code, sign planes on and off"""
    gen = torch.Generator().manual_seed(rk)
    p = F.Proj(64, 512, gen, None, rk, ("exh", rk * 1000), var=var)
    op = oracle_plane(p)
    p.to(DEV)
    for lv in (2, 4):
        assert same_f16(gpu_dense(p, lv, 64, 512, mode=rk % 2), O.dense_W(op, lv)) == 0, (rk, var, lv)


def test_exhaustive_block_words():
    """every one of the 33149 valid (Mb, N) words goes through the device's constant computation"""
    seen = set()
    for i in range(17):
        gen = torch.Generator().manual_seed(900 + i)
        p = F.Proj(2048, 2048, gen, None, 0, ("exh", i * 2048))
        seen |= set((p.Mb * 256 + p.Nn).tolist())
        op = oracle_plane(p)
        p.to(DEV)
        assert same_f16(gpu_dense(p, 4, 2048, 2048, mode=1), O.dense_W(op, 4)) == 0, i
    assert len(seen) == 33149


def test_odd_unit_count_and_level0():
    gen = torch.Generator().manual_seed(5)
    p = F.Proj(48, 128, gen, None, 3, "rand", var=True)          # 3 units: the last wave decodes a single unit
    op = oracle_plane(p); p.to(DEV)
    assert same_f16(gpu_dense(p, 4, 48, 128, mode=1), O.dense_W(op, 4)) == 0
    assert same_f16(gpu_dense(p, 2, 48, 128, mode=1), O.dense_W(op, 2)) == 0
    ex = _Ex(p, 1, 48, 128)
    row = M.entry(ex, 0).to(DEV)
    out = torch.full((48, 128), float("nan"), dtype=torch.float16, device=DEV)
    M.dequant(row, 1, 48, 128, out=out)
    assert not out.any()                                          # level 0 decodes to zeros


def test_full_shape_nested_expert_and_pf_decode():
    """one full-size expert (H 6144, I 2048) at levels 2/3/4 and the multi-expert prefill decode on top of it"""
    H, I = 6144, 2048
    ex = F.Expert(H, I, seed=77, dev="cpu", nested=True)
    og, od = oracle_plane(ex.gu), oracle_plane(ex.dn)
    for p in (ex.gu, ex.dn):
        p.to(DEV); p.slot = p.nested_plane()
    ex.signs = ex.signs.to(DEV)
    want = {}
    for lv in (2, 3, 4):
        want[lv] = (O.dense_W(og, lv, nested=True), O.dense_W(od, lv, nested=True))
        assert same_f16(M.dense_W(ex, 0, lv).cpu().numpy(), want[lv][0]) == 0, lv
        assert same_f16(M.dense_W(ex, 1, lv).cpu().numpy(), want[lv][1]) == 0, lv
    table = torch.stack([M.entry(ex, lv) for lv in (4, 0, 2, 3)]).to(DEV)
    ids = torch.tensor([3, 1, 0], dtype=torch.int32, device=DEV)
    Wgu = torch.empty(3, 2 * I, H, dtype=torch.float16, device=DEV); Wdn = torch.empty(3, H, I, dtype=torch.float16, device=DEV)
    _lib.check(_lib.lib().nq_pf_decode(table.data_ptr(), ids.data_ptr(), 3, Wgu.data_ptr(), Wdn.data_ptr(), H, I,
                                       _lib.stream_ptr()))
    torch.cuda.synchronize()
    assert same_f16(Wgu[0].cpu().numpy(), want[3][0]) == 0 and same_f16(Wdn[0].cpu().numpy(), want[3][1]) == 0
    assert not Wgu[1].any() and not Wdn[1].any()
    assert same_f16(Wgu[2].cpu().numpy(), want[4][0]) == 0 and same_f16(Wdn[2].cpu().numpy(), want[4][1]) == 0


def test_bad_arguments_raise():
    row = torch.zeros(F.TBL_W, dtype=torch.int64, device=DEV)
    out = torch.empty(256, 256, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="whole 16x128 units"):
        M.dequant(row, 0, 100, 128, out=out)
    with pytest.raises(RuntimeError, match="proj"):
        _lib.check(_lib.lib().nq_dequant(row.data_ptr(), 2, 0, 128, 128, out.data_ptr(), None))


@pytest.mark.parametrize("rk", [0, 7])
def test_mask_mode_golden(rk):
    """mask mode (flags per strip, compact residual plane): the reference's own level-4 dense decode, both projections' row
    fields; nq_pf_decode takes the same path"""
    from tests.test_oracle_golden import mask_proj
    z, p = mask_proj(rk)
    p.to(DEV)
    want = z["W4"].view(np.float16)
    for mode in (0, 1):
        assert same_f16(gpu_dense(p, 4, p.N, p.K, mode), want) == 0
        assert same_f16(gpu_dense(p, 2, p.N, p.K, mode), O.dense_W(oracle_plane(p), 2)) == 0


def test_mask_mode_layer_decode_and_prefill():
    """a layer whose experts mix dense and masked residual planes: decode path and prefill against the float64 oracle"""
    from tests.test_gpu_moe import oracle_layer
    from tests.util import rel_err
    H, I, NE = 512, 256, 6
    ex = [F.Expert(H, I, seed=4100 + i, dev="cpu", nm_gu=(2 if i % 2 else None), nm_dn=(1 if i % 2 else None),
                   rk_gu=(0, 3, 7, 9, 0, 6)[i], rk_dn=(7, 0, 0, 3, 9, 8)[i], var=(i == 3)) for i in range(NE)]
    planes = [(oracle_plane(e.gu), oracle_plane(e.dn), False) for e in ex]
    signs = [e.signs.numpy() for e in ex]
    levels = [4, 4, 2, 4, 4, 4]
    for e in ex:
        e.gu.to(DEV); e.dn.to(DEV); e.signs = e.signs.to(DEV)
    L = M.MoELayer(NE, H, I, Bmax=4, topk=3)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    g = torch.Generator().manual_seed(3)
    for B in (1, 4):
        sel = torch.stack([torch.randperm(NE, generator=g)[:3] for _ in range(B)]).to(DEV)
        rw = (torch.rand(B, 3, generator=g) + 0.1).half().to(DEV)
        x = (torch.randn(B, H, generator=g) * 0.05).half().to(DEV)
        want = oracle_layer(planes, levels, signs, x, sel, rw)
        for cg, cd in (([1, 4, 2], [1, 4, 1]), ([1, 2, 4], [1, 4, 2])):
            y = L(x, sel, rw, cfg_gu=cg, cfg_dn=cd)
            torch.cuda.synchronize()
            assert rel_err(y.cpu().numpy(), want) < 5e-5, (B, cg, cd)
        assert rel_err(L.prefill(x, sel, rw).cpu().numpy(), want) < 5e-5, B
    # the dense decode used by prefill-with-scratch callers agrees with the oracle bit for bit
    for e in (1, 3):
        for proj, pl in ((0, planes[e][0]), (1, planes[e][1])):
            assert same_f16(M.dense_W(ex[e], proj, 4).cpu().numpy(), O.dense_W(pl, 4)) == 0


@pytest.mark.parametrize("rk", [3, 9])
def test_base_code_1_golden(rk):
    """K = 1.75 base plane (table word 19, 112-bit records in the sub-array layout): the reference's own dense decode at
    levels 2 and 4, through both projections' row fields"""
    z = np.load(os.path.join(GOLD, f"proj_bk1_rk{rk}.npz"))
    gen = torch.Generator().manual_seed(int(z["seed"]))
    p = F.Proj(int(z["N"]), int(z["K"]), gen, None, rk, ("exh", int(z["mbn_offset"])), var=bool(z["var"].size), bk=1).to(DEV)
    for mode in (0, 1):
        assert same_f16(gpu_dense(p, 2, p.N, p.K, mode), z["W2"].view(np.float16)) == 0
        assert same_f16(gpu_dense(p, 4, p.N, p.K, mode), z["W4"].view(np.float16)) == 0


def test_base_code_1_layer_decode_and_prefill():
    """a layer that mixes K = 2 and K = 1.75 base planes (one of the latter also in mask mode, one with a different code per
    projection): decode path at several k-splits, prefill and the dense decoders against the oracle"""
    from tests.test_gpu_moe import oracle_layer
    from tests.util import rel_err
    H, I, NE = 512, 256, 6
    bk = [(1, 1), (0, 0), (1, 0), (0, 1), (1, 1), (1, 1)]
    ex = [F.Expert(H, I, seed=5100 + i, dev="cpu", nm_gu=(2 if i == 4 else None), nm_dn=(1 if i == 4 else None),
                   rk_gu=(3, 0, 7, 9, 0, 3)[i], rk_dn=(9, 0, 0, 3, 9, 9)[i], var=(i in (0, 3)), bk_gu=bk[i][0], bk_dn=bk[i][1])
          for i in range(NE)]
    planes = [(oracle_plane(e.gu), oracle_plane(e.dn), False) for e in ex]
    signs = [e.signs.numpy() for e in ex]
    levels = [4, 4, 4, 4, 4, 2]
    for e in ex:
        e.gu.to(DEV); e.dn.to(DEV); e.signs = e.signs.to(DEV)
    assert M.bk_codes() == [3, 3]
    L = M.MoELayer(NE, H, I, Bmax=4, topk=3)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    assert int(L.table[2, 19]) == 1 and int(L.table[3, 19]) == 256 and int(L.table[0, 19]) == 257
    g = torch.Generator().manual_seed(4)
    for B in (1, 4):
        sel = torch.stack([torch.randperm(NE, generator=g)[:3] for _ in range(B)]).to(DEV)
        rw = (torch.rand(B, 3, generator=g) + 0.1).half().to(DEV)
        x = (torch.randn(B, H, generator=g) * 0.05).half().to(DEV)
        want = oracle_layer(planes, levels, signs, x, sel, rw)
        for cg, cd in (([1, 4, 2], [1, 4, 1]), ([1, 2, 4], [1, 4, 2]), ([1, 1, 1], [1, 2, 1])):
            y = L(x, sel, rw, cfg_gu=cg, cfg_dn=cd)
            torch.cuda.synchronize()
            assert rel_err(y.cpu().numpy(), want) < 5e-5, (B, cg, cd)
        assert rel_err(L.prefill(x, sel, rw).cpu().numpy(), want) < 5e-5, B
        want2 = oracle_layer(planes, [2] * NE, signs, x, sel, rw)
        assert rel_err(L(x, sel, rw, force_level=2).cpu().numpy(), want2) < 5e-5
    for e in (0, 2, 3, 4, 5):
        for proj, pl in ((0, planes[e][0]), (1, planes[e][1])):
            assert same_f16(M.dense_W(ex[e], proj, levels[e]).cpu().numpy(), O.dense_W(pl, levels[e])) == 0
    # other base codes are refused when a row is set
    bad = M.entry(ex[0], 4); bad[19] = 5
    with pytest.raises(RuntimeError, match="base codes"):
        M.validate_row(bad, H, I)
    # the layer object has seen rows that are not of the common kind, so its decode calls run the kernel with every decode
    # loop; told (wrongly) that all rows are common, the common kernel is loud about the rows it has no loop for: tokens that
    # picked a K=1.75 or mask-mode row come out NaN, the others are untouched
    assert L.rare_rows
    sel = torch.tensor([[1, 1, 1], [0, 1, 2]], device=DEV)
    rw = torch.tensor([[0.5, 0.25, 0.25], [0.3, 0.3, 0.4]], dtype=torch.float16, device=DEV)
    x = (torch.randn(2, H, generator=g) * 0.05).half().to(DEV)
    ref = L(x, sel, rw).clone()
    L.rare_rows = False
    y = L(x, sel, rw).clone()
    torch.cuda.synchronize()
    assert torch.equal(y[0], ref[0]) and bool(torch.isnan(y[1]).all()) and bool(torch.isfinite(ref).all())
    assert not L.cnt_gu.any() and not L.cnt_d.any()                  # the workspace contract holds on that path too
    L.rare_rows = True
    assert torch.equal(L(x, sel, rw), ref)
    # the same in prefill: a table handed over with the call is of unknown kind, so both kernel variants run and the result is
    # right whatever the layer object believes; a wrong "all rows common" makes the lone variant write NaN for the tiles it has
    # no loop for (never the stale contents of the shared scratch) and leaves the tokens of common rows alone
    T = 24
    selp = torch.stack([torch.randperm(NE, generator=g)[:3] for _ in range(T)]).to(DEV)
    selp[:4] = 1                                                     # four tokens that pick only the common expert 1
    rwp = (torch.rand(T, 3, generator=g) + 0.1).half().to(DEV)
    xp = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    want = L.prefill(xp, selp, rwp).clone()
    assert rel_err(want.cpu().numpy(), oracle_layer(planes, levels, signs, xp, selp, rwp)) < 5e-5
    L.rare_rows = False
    assert torch.equal(L.prefill(xp, selp, rwp, table=L.table.clone()), want)
    yp = L.prefill(xp, selp, rwp).clone()
    torch.cuda.synchronize()
    assert torch.equal(yp[:4], want[:4])
    rare = torch.tensor([bool(L.table[e, 19]) or bool(L.table[e, 4]) for e in range(NE)], device=DEV)
    hit = rare[selp].any(1)
    assert bool(hit.any()) and bool(torch.isnan(yp[hit]).any(1).all()) and torch.equal(yp[~hit], want[~hit])
    L.rare_rows = True
