"""The minimal encoder (nestquant_amd/encode.py), CPU. Parity with the reference's encoder is not claimed (its Viterbi
lives in exllamav3, absent here); what is pinned: optimality by brute force on a small trellis, the distortions the
reference reports for this code on Gaussian data at 2, 3 and 4 bits, tail-biting consistency, the block-word search by its
closed form and by exhaustive search, and decode(encode) through the oracle at every level."""
import itertools

import numpy as np
import torch

from nestquant_amd import encode as EN
from oracle import nq_oracle as O
from tests.util import same_f16, u32


def test_codebook_equals_oracle():
    lut = EN.codebook().numpy()
    assert np.array_equal(lut, O.q2_value(O.hash_sum(np.arange(65536))).astype(np.float32))


def test_viterbi_is_optimal_on_a_small_trellis():
    """4-bit states (2 steps of memory), 2 bits per step, rings of 10 steps: brute force over all 4^10 tail-biting sequences.
    The two-pass tail-biting search (the reference's) is a heuristic; with the ring much longer than the trellis memory,
    as in the real code (256 steps vs 8), it finds the optimum."""
    g = torch.Generator().manual_seed(0)
    L, K, SB = 10, 2, 4
    seqs = torch.tensor(list(itertools.product(range(4), repeat=L)))
    states = torch.zeros_like(seqs)
    for i in range(L):                                           # state at step i: symbols of steps i, i-1 (most recent lowest)
        for back in range(SB // K):
            states[:, i] |= seqs[:, (i - back) % L] << (K * back)
    exact = 0
    for trial in range(3):
        lut = torch.randn(1 << SB, generator=g)
        w = torch.randn(6, L, generator=g)
        st = EN.viterbi_ring(w, lut, K=K, state_bits=SB)
        got = (lut[st] - w).square().sum(1)
        best = torch.stack([(lut[states] - w[t]).square().sum(-1).min() for t in range(6)])
        assert torch.all(got >= best - 1e-5) and torch.all(got <= best * 1.10 + 1e-5)
        exact += int((got <= best + 1e-5).sum())
        for t in range(6):                                       # a valid ring: each state extends its predecessor, also across the wrap
            for i in range(L):
                assert int(st[t, i]) >> K == int(st[t, (i - 1) % L]) & ((1 << (SB - K)) - 1)
    assert exact >= 15                                           # of 18 rings


def test_gaussian_distortion_matches_reference_report():
    g = torch.Generator().manual_seed(1)
    w = torch.randn(24, 256, generator=g)
    st = EN.viterbi_ring(w, EN.codebook())
    mse = float((EN.codebook()[st] - w).square().mean())
    assert abs(mse - 0.0684) < 0.004                              # reference: 0.06843 (CUDA Viterbi), 0.06828 (torch Viterbi)


def test_round_f16_rounds_once():
    """values a hair above and below the midpoint of two fp16 neighbours: through fp32 both land on the midpoint and then
    round to even; one rounding must separate them"""
    h = np.array([1.0, 1.5, 0.3330078125, 3.453125, 100.25], np.float16)
    up = np.nextafter(h, np.float16(np.inf))
    mid = (h.astype(np.float64) + up.astype(np.float64)) / 2
    v = np.concatenate([mid * (1 + 2.0**-40), mid * (1 - 2.0**-40), mid, -mid * (1 + 2.0**-40), -mid * (1 - 2.0**-40)])
    rng = np.random.default_rng(0)
    v = np.concatenate([v, rng.standard_normal(20000) * 4, rng.standard_normal(2000) * 1e-3])
    got = EN.round_f16(torch.from_numpy(v)).numpy()
    assert np.array_equal(got.view(np.uint16), v.astype(np.float16).view(np.uint16))
    assert not np.array_equal(torch.from_numpy(v[:10]).float().half().numpy().view(np.uint16), got[:10].view(np.uint16))


def test_fold_value_equals_oracle_for_every_block_word():
    words = O.all_block_words()                                   # 33149 (Mb, N)
    rng = np.random.default_rng(1)
    Sb = rng.integers(0, 1021, (len(words), 24)); Sr = rng.integers(0, 1021, (len(words), 24))
    Sb[:, 0], Sr[:, 0], Sb[:, 1], Sr[:, 1] = 0, 0, 1020, 1020
    want = O.fold_value(Sb, Sr, words[:, :1], words[:, 1:])
    got = EN.fold_value(torch.from_numpy(Sb), torch.from_numpy(Sr), torch.from_numpy(words[:, 0]), torch.from_numpy(words[:, 1]))
    assert np.array_equal(got.numpy().view(np.uint16), want.view(np.uint16))
    assert np.array_equal(EN.hash_sum(torch.arange(65536)).numpy(), O.hash_sum(np.arange(65536)))


def test_block_word_candidates():
    """first candidate = the reference's closed form (largest Mb with Mb (1 + delta) <= 257, N = round(delta Mb)); all twelve
    are valid block words; and the best of them is as good as the best of all 33149 words for a step size"""
    d = torch.tensor([0.0, 0.25, 1.0, 0.2612, 3.0, 300.0, 0.004])
    Mb, N = EN.block_word_candidates(d)
    assert Mb[:, 1].tolist() == [255, 205, 128, 203, 64, 1, 255]          # candidate 1 is (Mb0, round(delta Mb0))
    assert N[:, 1].tolist() == [0, 51, 128, 53, 192, 255, 1]
    assert bool(((Mb >= 1) & (Mb <= 255) & (N >= 0) & (N <= 255) & (Mb + N <= 257)).all())
    allw = torch.from_numpy(O.all_block_words()).double()
    for i in range(5):
        near = (allw[:, 1] / allw[:, 0] - d[i].double()).abs().min()
        assert float((N[i].double() / Mb[i].double() - d[i].double()).abs().min()) <= float(near) + 2e-3


def test_refinement_distortion_matches_reference_report():
    """base + one-bit plane 0.018747, base + two-bit plane 0.004729 / 0.004709 on N(0,1) with 256-weight rings (reference
    threads/03-nested-trellis-code/exp3_mul1L.log:3-4, REPORT.md:23); those use a real-valued step size per fit, this one
    the integer fold and a block word per 8 rings, which costs < 1 %"""
    g = torch.Generator().manual_seed(1)
    w = torch.randn(8, 8, 256, generator=g)
    st = EN.viterbi_rings(w.reshape(-1, 256), 2).reshape(8, 8, 256)
    want = {1: 0.018747, 2: 0.004729}
    for K in (1, 2):
        e = EN.encode_residual(w, st, K)
        mse = float((e["Q"] - w).square().mean())
        assert abs(mse / want[K] - 1) < 0.04, (K, mse)
        # the chosen block word is within 1 % of the best of ALL words for these states (exhaustive search on two units;
        # words of nearly the same ratio differ by how the fold's integer rounding happens to fall)
        Sb, Sr = EN.hash_sum(st[:2]), EN.hash_sum(e["states"][:2])
        allw = torch.from_numpy(O.all_block_words())
        for u in range(2):
            q = EN.fold_value(Sb[u:u + 1].expand(len(allw), 8, 256), Sr[u:u + 1].expand(len(allw), 8, 256), allw[:, 0], allw[:, 1])
            c = (q.float() - w[u]).double().square().sum((1, 2))
            mine = (e["Q"][u] - w[u]).double().square().sum()
            assert float(mine) <= float(c.min()) * 1.01


def test_second_plane_search_with_the_first_plane_frozen():
    """viterbi_ring_given_p3 on rings of 16 steps against brute force over all 2^16 P4 rings: a valid tail-biting ring (every
    8-bit window extends its predecessor, also across the wrap); exactly the best of all rings that close on the same seven
    bits (the second pass is an exact search under that constraint); never better than the best ring of all. How close it
    comes to that one is the two-pass heuristic's business (the reference's, harness.py:297-364), and a ring of 16 steps is
    only twice this code's memory, where the real rings are 32 times."""
    g = torch.Generator().manual_seed(3)
    L = 16
    lut = EN.codebook()
    seqs = torch.arange(1 << L)
    bits = (seqs[:, None] >> torch.arange(L)) & 1                 # bits[s, i] = the bit that enters at Viterbi step i
    win = torch.zeros(1 << L, L, dtype=torch.int64)
    for i in range(L):
        for back in range(8):
            win[:, i] |= bits[:, (i - back) % L] << back
    for trial in range(4):
        w = torch.randn(3, L, generator=g) * 1.2
        a = torch.randint(0, 256, (3, L), generator=g)
        b = EN.viterbi_ring_given_p3(w, a, lut)
        for t in range(3):
            for i in range(L):
                assert int(b[t, i]) >> 1 == int(b[t, (i - 1) % L]) & 0x7F
            err = (lut[EN.spread8(a[t])[None] | EN.spread8(win) << 1] - w[t][None]).square().sum(1)
            got = float((lut[EN.spread8(a[t]) | EN.spread8(b[t]) << 1] - w[t]).square().sum())
            same_close = (win[:, L - 1] & 0x7F) == (int(b[t, L - 1]) & 0x7F)
            assert abs(got - float(err[same_close].min())) < 1e-4, (trial, t)
            assert got >= float(err.min()) - 1e-5


def test_interleaved_two_plane_level4_fit_and_what_it_costs():
    """encode_nested(interleave=True): level 3 = base + P3 as before; level 4 = base + P3 and P4 interleaved (window code 12),
    decoded bit for bit by the oracle from the packed planes. With P3 frozen everywhere the second plane is a fresh one-bit fit
    with eight steps of memory, no better than level 3 -- the two levels read unrelated hashed windows, so a strictly nested
    hash code cannot be good at both (the reference's three-plane code that reaches 0.00516 / 0.00493 ADDS two refinement
    terms, threads/03-nested-trellis-code/REPORT.md:27-28, which this single-window format cannot express). share4 moves
    units from one end to the other: both planes of a unit from one two-bit fit (level 4 = the wide plane's 0.0047 there, level
    3 ~ the base plane's 0.068); with half the units moved the levels refine in order again."""
    g = torch.Generator().manual_seed(2)
    N, K = 128, 128
    W = torch.randn(N, K, generator=g)
    nrec = (N // 16) * (K // 128) * 32
    got = {}
    for share in (0.0, 0.5):
        r = EN.encode_nested(W, seed=3, interleave=True, share4=share)
        p = O.Plane(N, K, u32(r["base"]).reshape(-1, 4), p3=O.unpack_words(r["p3"].numpy(), nrec, 64), d3=u32(r["d3"]),
                    p4n=O.unpack_words(r["p4n"].numpy(), nrec, 64), d4n=u32(r["d4n"]))
        assert same_f16(O.dense_W(p, 3, nested=True), r["Q3"].half().numpy()) == 0
        assert same_f16(O.dense_W(p, 4, nested="interleave"), r["Q4n"].half().numpy()) == 0
        got[share] = tuple(float((r[k] - r["target"]).square().mean()) for k in ("Q", "Q3", "Q4n", "Q4"))
    d2, d3, d4n, d4w = got[0.0]
    assert abs(d3 / 0.018747 - 1) < 0.08 and abs(d4w / 0.004729 - 1) < 0.08
    assert 0.019 < d4n < 0.023                                    # a one-bit fit with eight steps of memory: not better than level 3
    assert got[0.5][1] > d3 and got[0.5][2] < d4n and got[0.5][2] < got[0.5][1]     # half and half: monotone 2 -> 3 -> 4 again
    print("N(0,1) distortion at levels 2 / 3 / nested 4 / wide 4 by share4:", {k: tuple(round(x, 5) for x in v) for k, v in got.items()})


def test_encode_decode_round_trip_through_the_oracle():
    g = torch.Generator().manual_seed(2)
    N, K = 128, 128
    W = torch.randn(N, K, generator=g) * torch.linspace(0.5, 2.0, K)[None]        # uneven input channels
    r = EN.encode_nested(W, seed=3, var=True)                    # with the sign plane: every ring in its better orientation
    nrec = (N // 16) * (K // 128) * 32
    p = O.Plane(N, K, u32(r["base"]).reshape(-1, 4), rk=0,
                res=O.unpack_words(r["p4"].numpy(), nrec, 128), d4=u32(r["d4"]),
                p3=O.unpack_words(r["p3"].numpy(), nrec, 64), d3=u32(r["d3"]), var=r["var"].numpy())
    negated = int(((r["var"].long()[:, None] >> torch.arange(8)) & 1).sum())
    assert 16 <= negated <= 48                                    # of 64 rings: about half are better negated
    # a negated ring is at least as good as the ring fitted as it is
    tr = EN.to_rings(r["target"])
    plain = EN.viterbi_rings(tr, 2)
    e_plain = (EN.codebook()[plain] - tr).square().sum(1)
    e_var = (EN.to_rings(r["Q"]) - tr).square().sum(1)
    assert bool((e_var <= e_plain + 1e-6).all()) and float(e_var.sum()) < float(e_plain.sum())
    B = lambda X, d: EN.blocked_had(X, d)
    # W ~= D(sv) B Q B D(su): relative error of the code on Gaussian data is sqrt(0.068), sqrt(0.0187), sqrt(0.0047)
    for level, key, lo, hi in ((2, "Q", 0.22, 0.30), (3, "Q3", 0.12, 0.155), (4, "Q4", 0.06, 0.078)):
        Wq = O.dense_W(p, level)
        assert same_f16(Wq, r[key].half().numpy()) == 0          # the decoder reproduces the encoder's matrix bit for bit
        West = r["sv"].double()[:, None] * B(B(torch.from_numpy(Wq.astype(np.float64)), 1), 0) * r["su"].double()[None, :]
        rel = float((West - W.double()).norm() / W.double().norm())
        assert lo < rel < hi, (level, rel)
    # sign vectors are +-scale: all magnitudes positive, both signs present
    assert (r["su"].abs() > 0).all() and (r["su"] > 0).any() and (r["su"] < 0).any()


def test_block_ldl():
    g = torch.Generator().manual_seed(4)
    X = torch.randn(400, 256, generator=g, dtype=torch.float64)
    H = X.T @ X / 400
    L, D = EN.block_ldl(H)
    assert float((L @ torch.block_diag(*D) @ L.T - H).abs().max()) < 1e-10
    assert float(L.triu(1)[:128, 128:].abs().max()) == 0          # block lower triangular ...
    assert float((L[:128, :128] - torch.eye(128)).abs().max()) < 1e-12 and float((L[128:, 128:] - torch.eye(128)).abs().max()) < 1e-12
    assert all(float(torch.linalg.eigvalsh(D[i]).min()) > 0 for i in range(2))


def test_ldlq_fit_feeds_errors_forward_and_lowers_the_output_error():
    """activations with a few strong directions shared by both 128-column chunks. Pinned: (1) the LDLQ identity
    tr(E H' E^T) = sum over chunks of tr(eta D eta^T), eta the chunk's own fitting error against its fed-forward target --
    exact for any quantiser, and broken by a wrong sign, a transposed factor or a wrong chunk order; (2) the last chunk, which
    receives no feedback, is fitted as without a Hessian; (3) the expected output error falls by a third or more against the
    fit that ignores H, at every level, where the plain squared error rises slightly; (4) decode(encode) through the oracle."""
    g = torch.Generator().manual_seed(5)
    N, K = 128, 256
    W = torch.randn(N, K, generator=g)
    V = torch.randn(4, K, generator=g)
    X = torch.randn(4096, 4, generator=g) @ V * 1.5 + torch.randn(4096, K, generator=g)
    H = (X.T @ X / 4096).double()
    r = EN.encode_ldlq(W, H, seed=3)
    T, Hr = r["target"].double(), r["Hr"]
    # the chunk that is fitted first, as the H-agnostic fit would do it (same targets; its block words are costed with D there)
    tr1 = EN.to_rings(r["target"][:, 128:].contiguous()).reshape(-1, 8, 256)
    st1 = EN.viterbi_rings(tr1.reshape(-1, 256), 2).reshape(-1, 8, 256)
    assert torch.equal(st1, r["states"].reshape(8, 2, 8, 256)[:, 1])
    # the other chunk without feedback
    tr0 = EN.to_rings(r["target"][:, :128].contiguous()).reshape(-1, 8, 256)
    st0 = EN.viterbi_rings(tr0.reshape(-1, 256), 2).reshape(-1, 8, 256)
    plain0 = {2: EN.codebook()[st0], 3: EN.encode_residual(tr0, st0, 1)["Q"], 4: EN.encode_residual(tr0, st0, 2)["Q"]}
    for lvl, key in ((2, "Q"), (3, "Q3"), (4, "Q4")):
        E = T - r[key].double()
        lhs = float(((E @ Hr) * E).sum())
        eta = r["eta"][lvl].reshape(N, 2, 128)
        rhs = float(sum(((eta[:, a] @ r["D"][a]) * eta[:, a]).sum() for a in range(2)))
        assert abs(lhs / rhs - 1) < 1e-9, (lvl, lhs, rhs)
        plain = r[key].clone()
        plain[:, :128] = EN.from_rings(plain0[lvl].reshape(-1, 256), N, 128)
        p_plain, p_ldlq = EN.proxy_loss(plain, r["target"], Hr), r["proxy"][lvl]
        assert p_ldlq < 0.70 * p_plain, (lvl, p_ldlq, p_plain)
        assert float((r[key] - r["target"]).square().mean()) > 0.99 * float((plain - r["target"]).square().mean())
    nrec = (N // 16) * (K // 128) * 32
    p = O.Plane(N, K, u32(r["base"]).reshape(-1, 4), rk=0, res=O.unpack_words(r["p4"].numpy(), nrec, 128), d4=u32(r["d4"]),
                p3=O.unpack_words(r["p3"].numpy(), nrec, 64), d3=u32(r["d3"]))
    for level, key in ((2, "Q"), (3, "Q3"), (4, "Q4")):
        assert same_f16(O.dense_W(p, level), r[key].half().numpy()) == 0


def test_g_scale_search_grid_and_vertex():
    """the reference's scale search (threads/05-exl3-harness/harness.py:371-387). With rings of ones the stand-in quantiser sees
    y = s and returns y (1 + (y - s*)), so mean((q / s - x)^2) = (s - s*)^2 exactly: the coarse grid must pick the right
    neighbourhood, the fine grid the nearest point, and the parabola's vertex must land on s* itself; a wrong sign of the
    vertex shift, a swapped neighbour or a wrong step would miss it. Then the real trellis fit on Gaussian rings: the found
    scale is at least as good as every point of the fine grid around it and as no scaling at all."""
    ones = torch.ones(9, 256)
    for target in (0.42, 0.97, 1.33, 1.84):
        q = lambda y, K, t=target: y * (1 + (y - t))
        s, m = EN.g_scale_search(ones, 2, q)
        assert abs(s - target) < 1e-6 and m <= 0.0375 ** 2 + 1e-9, (target, s, m)
    s, _ = EN.g_scale_search(ones, 2, lambda y, K: y * (1 + (y - 0.004)))          # below the grid: its lowest positive point region
    assert 0.01 <= s <= 0.1
    g = torch.Generator().manual_seed(4)
    w = torch.randn(12, 256, generator=g) * 0.8                   # not unit variance: the search must undo it
    lut = EN.codebook()
    mse = lambda v: float((lut[EN.viterbi_ring(w * v, lut, 2)] / v - w).square().mean())
    s, _ = EN.g_scale_search(w, 2)
    here = mse(s)
    assert 1.0 < s < 1.6 and here <= mse(1.0)
    assert all(here <= mse(s + d) * 1.01 for d in (-0.15, 0.15))
    # in units of the data's own rms the found scale is the same whatever the data's size
    s2, _ = EN.g_scale_search(w * 1.25, 2)
    assert abs(s2 * 1.25 / s - 1) < 0.08


def test_two_sided_ldlq_identity_and_gain():
    """encode_ldlq2 on one chunk of 128 columns and eight strips, activations and output weights with a few strong directions.
    Pinned: tr(Go E H' E^T) = sum over the units of tr(Dout eta Din eta^T) with eta each unit's own fitting error against the
    target it was given -- exact for any quantiser, broken by a wrong sign, a transposed factor or a wrong order of the units;
    the unit in the far corner gets no feedback, so it is fitted as the plain encoder fits it. The packed planes decode bit for
    bit through the oracle. (The gain over the one-sided and the plain fit is measured on the GPU, tests/test_gpu_configs12.py.)"""
    g = torch.Generator().manual_seed(5)
    N, K = 128, 128
    W = torch.randn(N, K, generator=g)
    X = torch.randn(4096, 4, generator=g) @ torch.randn(4, K, generator=g) * 1.5 + torch.randn(4096, K, generator=g)
    Y = torch.randn(4096, 3, generator=g) @ torch.randn(3, N, generator=g) * 1.5 + torch.randn(4096, N, generator=g)
    H, G = (X.T @ X / 4096).double(), (Y.T @ Y / 4096).double()
    r = EN.encode_ldlq2(W, H, G, seed=3)
    T = r["target"].double()
    S = N // 16
    for lvl, key in ((2, "Q"), (3, "Q3"), (4, "Q4")):
        E = T - r[key].double()
        lhs = float(((r["Go"] @ E @ r["Hr"]) * E).sum())
        eta = r["eta"][lvl].reshape(S, 16, 128)
        rhs = float(sum(((r["Dout"][c] @ eta[c] @ r["Din"][0]) * eta[c]).sum() for c in range(S)))
        assert abs(lhs / rhs - 1) < 1e-9, (lvl, lhs, rhs)
    last = EN.to_rings(r["target"][N - 16:].contiguous())         # strip 7: nothing was fitted before it
    assert torch.equal(EN.viterbi_rings(last, 2), r["states"][S - 1].reshape(8, 256))
    nrec = (N // 16) * (K // 128) * 32
    p = O.Plane(N, K, u32(r["base"]).reshape(-1, 4), rk=0, res=O.unpack_words(r["p4"].numpy(), nrec, 128), d4=u32(r["d4"]),
                p3=O.unpack_words(r["p3"].numpy(), nrec, 64), d3=u32(r["d3"]))
    for level, key in ((2, "Q"), (3, "Q3"), (4, "Q4")):
        assert same_f16(O.dense_W(p, level), r[key].half().numpy()) == 0


def test_low_rank_plane_detect_metric_fit():
    """lr_detect / lr_metric / lr_fit (reference threads/12-reference-encoder/nq_encode.py:507-556), pinned by what the linear
    algebra fixes: a second moment built from known orthonormal directions gives those directions back, in order, cut at the
    share threshold and at rmax; the metric agrees with H off the span and is m * identity on it; the fitted coefficients
    satisfy the normal equations (the residual has nothing left inside span(V)), any other coefficients fit worse, and the
    expected output error under activations that live mostly in the span falls by the share the span holds."""
    g = torch.Generator().manual_seed(9)
    K, N = 128, 128
    Qo, _ = torch.linalg.qr(torch.randn(K, K, generator=g).double())
    v1, v2, v3 = Qo[:, 0], Qo[:, 1], Qo[:, 2]
    H = torch.eye(K, dtype=torch.float64) + 40 * torch.outer(v1, v1) + 15 * torch.outer(v2, v2) + 0.5 * torch.outer(v3, v3)
    V = EN.lr_detect(H)                                           # shares 41 / 183.5, 16 / 183.5, 1.5 / 183.5 (< 0.05), 1 / 183.5 ...
    assert V.shape == (2, K) and V.dtype == torch.float16
    assert abs(abs(float(V[0].double() @ v1)) - 1) < 1e-3 and abs(abs(float(V[1].double() @ v2)) - 1) < 1e-3
    assert EN.lr_detect(H, rmax=1).shape[0] == 1 and EN.lr_detect(H, tau=0.3).shape[0] == 0
    assert EN.lr_detect(H, tau=0.001, rmax=4).shape[0] == 4       # rmax caps what the threshold would let through
    Vd = torch.stack([v1, v2])
    Mx = EN.lr_metric(H, Vd)
    w = Qo[:, 5] * 0.7 + Qo[:, 9] * 0.3                           # orthogonal to the span
    assert abs(float(w @ Mx @ w) - float(w @ H @ w)) < 1e-9
    P = Vd.T @ Vd
    m = float(((torch.eye(K, dtype=torch.float64) - P) @ H @ (torch.eye(K, dtype=torch.float64) - P)).diagonal().mean())
    assert torch.allclose(Mx @ v1, m * v1, atol=1e-9) and torch.allclose(Mx, Mx.T, atol=1e-12)
    assert float(torch.linalg.eigvalsh(Mx).min()) > 0.5 and EN.lr_metric(H, Vd[:0]) is H
    # fit on a quantised weight
    W = torch.randn(N, K, generator=g)
    r = EN.encode_nested(W, seed=4)
    su, sv = r["su"], r["sv"]
    back = EN.dense_from_rotated(r["target"], su, sv)
    assert float((back - W).norm() / W.norm()) < 1e-5             # D(sv) B target B D(su) is the weight itself
    d2, d4 = EN.dense_from_rotated(r["Q"], su, sv), EN.dense_from_rotated(r["Q4"], su, sv)
    U2, U4, w2, w4 = EN.lr_fit(W, d2, d4, V)
    assert U2.shape == U4.shape == (2, N) and U2.dtype == torch.float16
    Vf = V.double()
    for dense, fitted in ((d2, w2), (d4, w4)):
        left = (W.double() - fitted.double()) @ Vf.T              # what the residual still has inside the span
        was = (W.double() - dense.double()) @ Vf.T
        assert float(left.norm()) < 0.02 * float(was.norm())      # fp16 coefficients: not zero, but two orders down
    for _ in range(3):                                            # any other coefficients are worse
        Uo = (U2.double() + 0.02 * torch.randn(2, N, generator=g).double())
        assert float((W.double() - d2.double() - Uo.T @ Vf).norm()) > float((W.double() - w2.double()).norm())
    cost = lambda D: float((((W.double() - D.double()) @ H) * (W.double() - D.double())).sum())
    assert cost(w2) < 0.75 * cost(d2) and cost(w4) < 0.75 * cost(d4)   # the span holds 57 of H's trace of 183.5
    assert w4.dtype == torch.float32 and float((w4 - d4 - (U2.float() + U4.float()).T @ V.float()).abs().max()) < 1e-3
