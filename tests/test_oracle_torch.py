"""The torch-CPU restatement that bench.py times as the CPU baseline (oracle/nq_oracle_torch.py) against the numpy oracle,
which the golden fixtures of the reference's own decoder pin: dense weights bit for bit, layer output to fp32 rounding."""
import numpy as np
import torch

from nestquant_amd import format as F
from oracle import nq_oracle as O, nq_oracle_torch as OT
from tests.util import oracle_plane, rel_err, same_f16


def test_dense_weights_equal_the_numpy_oracle_bitwise():
    for seed, rk, nested, var in ((1, 0, False, False), (2, 7, False, True), (3, 3, True, False), (4, 9, True, True)):
        ex = F.Expert(256, 128, seed=seed, dev="cpu", rk_gu=rk, rk_dn=rk, nested=nested, var=var)
        for p in (ex.gu, ex.dn):
            pl = oracle_plane(p)
            for level in (2, 3, 4) if nested else (2, 4):
                want = O.dense_W(pl, level, nested=nested and level >= 3)
                got = OT.dense_W(pl, level, nested=nested and level >= 3).numpy()
                assert same_f16(got, want) == 0, (seed, level)


def test_golden_dense_fixture(golden_dir):
    """a fixture the reference's own dense_W wrote (residual code 7 with a sign plane): the torch restatement gives its bits"""
    from tests.util import u32
    z = np.load(f"{golden_dir}/proj_rk7_var1.npz")
    N, K, rk = int(z["N"]), int(z["K"]), int(z["rk"])
    nrec = (N // 16) * (K // 128) * 32
    pl = O.Plane(N, K, u32(torch.from_numpy(z["base"])).reshape(-1, 4), rk=rk, res=O.unpack_words(z["p4"], nrec, O.rbits(rk)),
                 d4=u32(torch.from_numpy(z["d4"])), var=z["var"])
    for level, key in ((2, "W2"), (4, "W4")):
        assert same_f16(OT.dense_W(pl, level).numpy(), z[key].view(np.float16)) == 0


def test_layer_equals_the_numpy_oracle():
    H, I, NE = 256, 128, 5
    levels = [2, 4, 3, 0, 4]
    ex = [F.Expert(H, I, seed=30 + i, dev="cpu", nested=i in (2, 4), var=i == 1, rk_gu=(0, 3)[i == 1]) for i in range(NE)]
    planes = [(oracle_plane(e.gu), oracle_plane(e.dn), e.nested) for e in ex]
    signs = [e.signs.numpy() for e in ex]
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(3, H, generator=g) * 0.05).half().float().numpy()
    sel = np.array([[0, 1, 2], [2, 3, 4], [4, 4, 0]]); rw = np.array([[.5, .25, .25], [.3, .3, .4], [.2, 0., .8]], np.float16)

    def dense(e):
        pg, pd, n = planes[e]
        return O.dense_W(pg, levels[e], nested=n).astype(np.float32), O.dense_W(pd, levels[e], nested=n).astype(np.float32)
    want = O.moe_forward(dense, levels, lambda e: signs[e], x, sel, rw, dtype=np.float64)
    got = OT.moe_ref(lambda e: planes[e], levels, lambda e: signs[e], x, sel, rw).numpy()
    assert rel_err(got, want) < 5e-4          # fp32 sums against the float64 arbiter (5 % extreme block words: weights in the thousands)
    wrong = O.moe_forward(dense, [2] * NE, lambda e: signs[e], x, sel, rw, dtype=np.float64)
    assert rel_err(got, wrong) > 1e-2          # and it does tell the levels apart
