"""Config 4 at its full size: prefill of 4096 tokens, top-8 over 256 experts with Zipf(1.1) popularity, H 6144, I 2048, every
expert at level 4 (the workload of bench.py's prefill leg). The float64 oracle cannot run 4096 tokens in seconds, so it checks
a sample of tokens (first, last and six inside: within 1e-4, the reference's smoke_prefill.py bar is 3e-3), and the rest is held
by properties that do not depend on the size: the prefill result of whole 8-token slices agrees with the decode path run on
the same slices (reference sm120/smoke_prefill.py: prefill against the 8-token slice loop), a second call gives the same bits,
the exported hits equal the routing's counts, and a token whose weights are all zero comes out zero."""
import numpy as np
import pytest
import torch

from nestquant_amd import moe as M
from oracle import nq_oracle as O
from tests.util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_config4_full_size_prefill():
    import bench as BN
    H, E, T = BN.H, BN.E, 4096
    L, MB, ex, levels = BN.build_layer(DEV, Bmax=8)
    for e in range(E):
        L.set(e, ex[e], 4)
    sel, rw = BN.zipf_routing(T, DEV)
    rw = rw.clone()
    rw[777] = 0                                                   # a token that no expert contributes to
    rw[2048, 3] = 0
    g = torch.Generator().manual_seed(12)
    x = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    hits = torch.zeros(E, dtype=torch.int32, device=DEV)
    L.hits_ptr = hits.data_ptr()
    try:
        y = L.prefill(x, sel, rw).clone()
        torch.cuda.synchronize()
        assert hits.cpu().tolist() == torch.bincount(sel[rw != 0].flatten().cpu(), minlength=E).tolist()
    finally:
        L.hits_ptr = 0
    y2 = L.prefill(x, sel, rw)
    torch.cuda.synchronize()
    assert torch.equal(y, y2), "prefill is not repeatable"
    assert bool(torch.isfinite(y).all()) and not y[777].any()
    # the decode path on whole 8-token slices (other tilings, other summation order, same arithmetic otherwise)
    worst = 0.0
    for s0 in (0, 776, 1336, 2048, 2896, T - 8):
        sl = slice(s0, s0 + 8)
        yd = L(x[sl], sel[sl], rw[sl]).clone()
        torch.cuda.synchronize()
        err = rel_err(y[sl].cpu().numpy(), yd.cpu().numpy())
        worst = max(worst, err)
        assert err < 1e-4, (s0, err)
    # the float64 oracle over the HIP-decoded dense weights of the sampled tokens' experts (the decoder is bit-exact: test_gpu_dequant)
    toks = [0, 5, 1337, 2048, 2901, 3333, 4000, T - 1]
    cache = {}

    def dense(e):
        if e not in cache:
            cache[e] = (M.dense_W(ex[e], 0, 4).float().cpu().numpy(), M.dense_W(ex[e], 1, 4).float().cpu().numpy())
        return cache[e]
    want = O.moe_forward(dense, [4] * E, lambda e: ex[e].signs.cpu().numpy(), x[toks].cpu().numpy(), sel[toks].cpu().numpy(),
                         rw[toks].cpu().numpy(), dtype=np.float64)
    err = rel_err(y[toks].cpu().numpy(), want)
    assert err < 1e-4, err
    pure = O.moe_forward(dense, [4] * E, lambda e: ex[e].signs.cpu().numpy(), x[toks].cpu().numpy(), sel[toks].cpu().numpy(),
                         rw[toks].cpu().numpy(), round_acts=False, dtype=np.float32)
    assert rel_err(y[toks].cpu().numpy(), pure) < 1e-3
    print(f"config 4 full size: {len(toks)} tokens within {err:.1e} of the float64 oracle, 48 tokens within {worst:.1e} of the decode path")
