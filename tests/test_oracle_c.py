"""The C oracle against the numpy oracle and the reference's golden fixtures (CPU only)."""
import glob
import os

import numpy as np
import pytest
import torch

from nestquant_amd import format as F
from oracle import nq_oracle as O, nq_oracle_c as OC
from tests.util import oracle_plane, same_f16, u32

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_scalar_pieces():
    L = OC.lib()
    assert [L.nqo_rbits(c) for c in range(13)] == [O.rbits(c) for c in range(13)]
    for c in range(13):
        assert [L.nqo_step_off(p, c) for p in range(0, 257, 3)] == O.step_off(np.arange(0, 257, 3), *O.RKP[c]).tolist()
    st = np.arange(0, 65536, 13)
    assert [L.nqo_hash_sum(int(s)) for s in st] == O.hash_sum(st).tolist()
    # fp16 conversion on every fp16 value and on ties / subnormals / overflow
    allh = np.arange(65536, dtype=np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    back = np.array([L.nqo_f32_to_f16(float(v)) for v in f[ok][::7]], np.uint16)
    assert np.array_equal(back, allh[ok][::7])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)])
    x = np.concatenate([x, np.float32([2**-25, 2**-25 * 1.0001, 2**-24 * 1.5, 65504, 65519.99, 65520, 1 + 2**-11, 1 + 3 * 2**-11])])
    want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.nqo_f32_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(np.array([L.nqo_f16_to_f32(int(h)) for h in allh[ok][::5]], np.float32), f[ok][::5])


def test_fold_constants_all_block_words():
    L = O.all_block_words()
    Ah, Ch = O.fold_consts(L[:, 0], L[:, 1])
    got = np.array([OC.fold_consts(m, n) for m, n in L[::3]], np.uint16)
    assert np.array_equal(got[:, 0], Ah.view(np.uint16)[::3]) and np.array_equal(got[:, 1], Ch.view(np.uint16)[::3])


@pytest.mark.parametrize("code", range(12))
def test_unpack_matches_numpy(code):
    rng = np.random.default_rng(code)
    bits = O.rbits(code); nw = (bits + 31) // 32
    w = rng.integers(0, 2**32, (160, nw), dtype=np.uint64).astype(np.uint32)
    if bits % 32:
        w[:, -1] &= np.uint32((1 << (bits % 32)) - 1)
    for split in ((False, True) if code == 11 else (False,)):
        assert np.array_equal(OC.unpack(O.pack_words(w, bits, split), 160, code, split), w)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "proj_rk*_var*.npz"))), ids=lambda p: os.path.basename(p)[:-4])
def test_golden_projections(path):
    z = np.load(path)
    N, K, rk = int(z["N"]), int(z["K"]), int(z["rk"])
    nrec = (N // 16) * (K // 128) * 32
    base = u32(torch.from_numpy(z["base"])).reshape(-1, 4)
    res = OC.unpack(z["p4"], nrec, rk)
    var = z["var"] if z["var"].size else None
    assert same_f16(OC.decode_proj(base, N, K, 2, var=var), z["W2"].view(np.float16)) == 0
    assert same_f16(OC.decode_proj(base, N, K, 4, rk, res, u32(torch.from_numpy(z["d4"])), var), z["W4"].view(np.float16)) == 0


def test_nested_levels_and_random_projection_vs_numpy():
    gen = torch.Generator().manual_seed(11)
    p = F.Proj(64, 384, gen, None, 7, "rand", var=True, nested=True)
    op = oracle_plane(p)
    assert same_f16(OC.decode_proj(op.base, 64, 384, 2, var=op.var), O.dense_W(op, 2)) == 0
    assert same_f16(OC.decode_proj(op.base, 64, 384, 4, 7, op.res, op.d4, op.var), O.dense_W(op, 4)) == 0
    assert same_f16(OC.decode_proj(op.base, 64, 384, 3, 10, op.p3, op.d3, op.var), O.dense_W(op, 3, nested=True)) == 0
    both = np.concatenate([op.p3, op.p4n], 1)
    assert same_f16(OC.decode_proj(op.base, 64, 384, 4, 11, both, op.d4n, op.var), O.dense_W(op, 4, nested=True)) == 0
    stored = np.concatenate([op.p3.reshape(-1), op.p4n.reshape(-1)])                  # the device layout: P3's records, then P4's
    mixed = OC.unpack(stored, op.p3.shape[0], 12, split=2)
    assert np.array_equal(mixed, O.interleave_words(op.p3, op.p4n))
    assert same_f16(OC.decode_proj(op.base, 64, 384, 4, 12, mixed, op.d4n, op.var), O.dense_W(op, 4, nested="interleave")) == 0
    W = O.dense_W(op, 4); x = np.random.default_rng(0).standard_normal(384).astype(np.float32)
    assert np.allclose(OC.matvec_f16(W, x), W.astype(np.float32) @ x, rtol=1e-4, atol=1e-3)
