"""The minimal level-2 encoder (nestquant_amd/encode.py), CPU. Parity with the reference's encoder is not claimed (its
Viterbi lives in exllamav3, absent here); what is pinned: optimality by brute force on a small trellis, the distortion the
reference reports for this code on Gaussian data, tail-biting consistency, and decode(encode) through the oracle."""
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


def test_encode_decode_round_trip_through_the_oracle():
    g = torch.Generator().manual_seed(2)
    W = torch.randn(128, 256, generator=g) * torch.linspace(0.5, 2.0, 256)[None]      # uneven input channels
    r = EN.encode_level2(W, seed=3)
    p = O.Plane(128, 256, u32(r["base"]).reshape(-1, 4))
    Wq = O.dense_W(p, 2)
    assert same_f16(Wq, r["Q"].half().numpy()) == 0              # the decoder reproduces the encoder's Q bit for bit
    # W ~= D(sv) B Q B D(su): relative error of a 2-bit code on Gaussian data is sqrt(0.068) ~ 26 %
    B = lambda X, d: EN.blocked_had(X, d)
    West = r["sv"].double()[:, None] * B(B(torch.from_numpy(Wq.astype(np.float64)), 1), 0) * r["su"].double()[None, :]
    rel = float((West - W.double()).norm() / W.double().norm())
    assert 0.22 < rel < 0.30
    # sign vectors are +-scale: all magnitudes positive, both signs present
    assert (r["su"].abs() > 0).all() and (r["su"] > 0).any() and (r["su"] < 0).any()
