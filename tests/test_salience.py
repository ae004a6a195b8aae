"""Decode salience export (sal[e] += (rsf w)^2 |x|^2 per pick): the oracle against exact known answers and an independent
float64 closed form on the CPU; the HIP kernel against the oracle on the GPU -- exactly where every partial sum is exact (rows
of small powers of two), to fp32 rounding of the squared norm (1e-5 relative) otherwise."""
import numpy as np
import pytest
import torch

from oracle import nq_oracle as O


def closed_form(x, w, ids, rsf, E):
    out = np.zeros(E)
    xn = (x.astype(np.float64) ** 2).sum(1)
    for t in range(ids.shape[0]):
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            if float(w[t, k]) != 0.0 and 0 <= e < E:
                out[e] += (rsf * float(w[t, k])) ** 2 * xn[t]
    return out


def test_oracle_known_answers():
    E, H = 16, 6144
    x = np.ones((2, H), np.float16); x[1] *= 2                       # |x|^2 = 6144 and 4 * 6144, every partial sum exact
    w = np.array([[0.5, 0.25, 0.0, 1.0], [0.5, 0.5, 0.5, 0.5]], np.float16)
    ids = np.array([[3, 5, 7, 3], [5, 5, 99, -1]])                   # duplicates in a token and across tokens, ids outside the table
    acc = np.zeros(E); acc[3] = 1.5
    touched = O.salience(x, w, ids, 2.0, acc)
    want = np.zeros(E)
    want[3] = 1.5 + (1.0 + 4.0) * 6144                                 # (2 * 0.5)^2 + (2 * 1)^2
    want[5] = 0.25 * 6144 + 2 * 1.0 * 4 * 6144
    assert np.array_equal(acc, want) and touched == [3, 5]            # expert 7 had weight 0; 99 and -1 are outside the table
    assert np.array_equal(closed_form(x, w, ids, 2.0, E), want - np.eye(E)[3] * 1.5)
    # a second call keeps adding
    O.salience(x[:1], w[:1], ids[:1], 1.0, acc)
    assert acc[3] == want[3] + (0.25 + 1.0) * 6144 and acc[5] == want[5] + 0.0625 * 6144


@pytest.mark.parametrize("H", [6144, 100, 8, 2056])
def test_oracle_matches_float64_closed_form(H):
    rng = np.random.default_rng(H)
    E, T, K = 32, 5, 8
    x = (rng.standard_normal((T, H)) * 0.7).astype(np.float16)
    w = rng.random((T, K)).astype(np.float16); w[2, 3] = 0
    ids = rng.integers(0, E, (T, K))
    acc = np.zeros(E)
    O.salience(x, w, ids, 2.5, acc)
    assert np.allclose(acc, closed_form(x, w, ids, 2.5, E), rtol=3e-7, atol=0)        # rsf * w is an fp32 product in the oracle, as in the kernels


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_hip_salience(dtype):
    from nestquant_amd import salience as SA
    g = torch.Generator().manual_seed(11)
    E, K = 256, 8
    # exact cases: rows of +-1 and +-2 (every partial sum is a small integer), weights that are powers of two
    S = SA.Salience(E, rsf=2.0)
    want = np.zeros(E)
    for T, H, cut in ((2, 6144, 0), (8, 6144, 0), (3, 100, 0), (4, 2048, 1), (1, 8, 0)):
        sign = torch.randint(0, 2, (T, H + 16), generator=g) * 2 - 1
        big = (sign * (1 + torch.arange(T)[:, None] % 2)).to(dtype)
        x = big[:, cut:cut + H]                                       # cut = 1: rows off 16-byte alignment
        w = (0.5 ** torch.randint(0, 4, (T, K), generator=g)).half(); w[0, 1] = 0
        ids = torch.randint(0, E, (T, K), generator=g); ids[-1, 0] = E + 3; ids[0, 2] = ids[0, 5]
        touched = O.salience(x.float().numpy(), w.numpy(), ids.numpy(), 2.0, want)
        S(x.cuda(), w.cuda(), ids.cuda()) if cut == 0 else SA.sal(big.cuda()[:, cut:cut + H], w.cuda(), ids.cuda(), 2.0, S.acc, S.host)
        torch.cuda.synchronize()
        got = S.acc.cpu().numpy()
        assert np.array_equal(got, want), (T, H, cut, np.abs(got - want).max())
        assert np.array_equal(S.host.numpy()[touched], want[touched])
    # general values: fp32 rounding of the squared norm
    S = SA.Salience(E, rsf=2.5)
    want = np.zeros(E)
    for T, H, cut in ((1, 6144, 0), (8, 6144, 0), (3, 100, 0), (4, 2048, 1), (5, 4096, 8), (7, 2056, 0)):
        big = (torch.randn(T, H + 16, generator=g) * 0.7).to(dtype)
        x = big[:, cut:cut + H]
        w = torch.rand(T, K, generator=g).half(); w[0, 1] = 0
        ids = torch.randint(0, E, (T, K), generator=g); ids[-1, 0] = E + 3; ids[0, 2] = ids[0, 5]
        xo = x.float().half().float().numpy() if dtype != torch.bfloat16 else x.float().numpy()
        touched = O.salience(xo, w.numpy(), ids.numpy(), 2.5, want)
        S(x.cuda(), w.cuda(), ids.cuda()) if cut == 0 else SA.sal(big.cuda()[:, cut:cut + H], w.cuda(), ids.cuda(), 2.5, S.acc, S.host)
        torch.cuda.synchronize()
        got = S.acc.cpu().numpy()
        assert np.allclose(got, want, rtol=1e-5, atol=0), (T, H, cut, np.abs(got / np.maximum(want, 1e-30) - 1).max())
        assert np.array_equal(S.host.numpy()[touched], got[touched])
        assert np.array_equal(got == 0, want == 0)                     # skipped picks touch nothing
        want = got.copy()                                              # the running sums continue from the device's values
    # int32 ids and bf16 / fp32 weights read as the casts would leave them
    x = (torch.randn(2, 512, generator=g)).to(dtype).cuda()
    w32 = torch.rand(2, K, generator=g); ids = torch.randint(0, E, (2, K), generator=g)
    a = SA.Salience(E, 1.0); b = SA.Salience(E, 1.0)
    a(x, w32.half().cuda(), ids.cuda()); b(x, w32.cuda(), ids.int().cuda())
    torch.cuda.synchronize()
    assert torch.equal(a.acc, b.acc) and a.acc.sum() > 0


@pytest.mark.gpu
def test_salience_errors_and_forward_hook():
    from nestquant_amd import format as F, moe as M, salience as SA
    S = SA.Salience(8)
    x = torch.zeros(9, 128, dtype=torch.float16, device="cuda")
    w = torch.ones(9, 2, dtype=torch.float16, device="cuda"); ids = torch.zeros(9, 2, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="at most 8"):
        S(x, w, ids)
    with pytest.raises(RuntimeError, match="nqsal"):
        S(x[:2].double(), w[:2], ids[:2])
    with pytest.raises(RuntimeError, match="nqsal"):
        SA.sal(x[:2], w[:2], ids[:2], 1.0, S.acc.float(), S.host)
    S(x[:0], w[:0], ids[:0])                                          # no tokens: nothing to do
    # the serving step feeds it: steps of up to Bmax tokens and the slices of steps of up to 16
    H, I, E = 256, 128, 4
    L = M.MoELayer(E, H, I, Bmax=4, topk=2)
    for e in range(E):
        ex = F.Expert(H, I, seed=e, dev="cpu"); ex.gu.to("cuda"); ex.dn.to("cuda"); ex.signs = ex.signs.cuda()
        L.keep = getattr(L, "keep", []) + [ex]
        L.set(e, ex, 2)
    g = torch.Generator().manual_seed(3)
    S = SA.Salience(E, rsf=1.5)
    want = np.zeros(E)
    for T in (3, 4, 11, 16, 17):
        xt = torch.randn(T, H, generator=g).bfloat16().cuda()
        wt = torch.rand(T, 2, generator=g).cuda(); it = torch.stack([torch.randperm(E, generator=g)[:2] for _ in range(T)]).int().cuda()
        M.forward(L, None, xt, wt, it, sal=S)
        if T <= 16:
            for i in range(0, T, 4):
                O.salience(xt[i:i + 4].float().cpu().numpy(), wt[i:i + 4].half().cpu().numpy(), it[i:i + 4].cpu().numpy(), 1.5, want)
    torch.cuda.synchronize()
    assert np.allclose(S.acc.cpu().numpy(), want, rtol=1e-5, atol=0) and np.array_equal(S.host.numpy(), S.acc.cpu().numpy())
