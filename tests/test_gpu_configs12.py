"""The CPU-plumbing and single-projection configurations on the GPU.
Config 1: one 512 x 256 weight ~ N(0,1), encoded at level 2 (minimal encoder), decoded by the HIP decoder (bit-exact vs
the oracle), then decode+GEMV against one fp16 activation vector, within 1e-3 of an fp32 matmul over the oracle-dequantised
weights. Config 2: single projection 6144 -> 2048 at levels 2/3/4 on the same base, token batch 1/4/8."""
import numpy as np
import pytest
import torch

from nestquant_amd import encode as EN, format as F, moe as M
from oracle import nq_oracle as O, nq_oracle_c as OC
from tests.util import oracle_plane, rel_err, same_f16, u32

pytestmark = pytest.mark.gpu
DEV = "cuda"


class _Ex:
    pass


def test_config1_encode_decode_gemv():
    N, K = 512, 256
    g = torch.Generator().manual_seed(0)
    W = torch.randn(N, K, generator=g)
    r = EN.encode_level2(W.to(DEV), seed=1)                       # the torch encoder runs on the GPU
    base_cpu = r["base"].cpu()
    Wq = OC.decode_proj(u32(base_cpu).reshape(-1, 4), N, K, 2)    # C oracle
    assert same_f16(Wq, O.dense_W(O.Plane(N, K, u32(base_cpu).reshape(-1, 4)), 2)) == 0
    assert same_f16(Wq, r["Q"].half().cpu().numpy()) == 0
    # as the gate|up projection of an expert with H = 256, I = 256 (gate rows = W[:256], up rows = W[256:], same su)
    H, I = K, N // 2
    ex = _Ex()
    ex.H, ex.I, ex.nested, ex.lr = H, I, False, None
    ex.gu = EN.EncodedProj(N, K, r["base"])
    ex.dn = EN.EncodedProj(H, I, torch.zeros(F.proj_sizes(H, I)["base"] // 4, dtype=torch.int32, device=DEV))
    one = torch.ones(I, dtype=torch.float16, device=DEV)
    ex.signs = torch.cat([r["su"], r["sv"][:I], r["sv"][I:], one, torch.ones(H, dtype=torch.float16, device=DEV), r["su"]]).contiguous()
    L = M.MoELayer(1, H, I, Bmax=1, topk=1)
    L.set(0, ex, 2)
    assert same_f16(M.dense_W(ex, 0, 2).cpu().numpy(), Wq) == 0   # HIP decoder: bit-exact
    x = torch.randn(1, K, generator=g).half().to(DEV)
    raw = M.proj_gemv(L, x)[0].cpu().numpy()                      # W_q . fp16(Hadamard(su * x)) from the fused kernel
    su, sv = r["su"].float().cpu().numpy(), r["sv"].float().cpu().numpy()
    xr = O.wht(x.float().cpu().numpy()[0] * su).astype(np.float16).astype(np.float32)
    want_raw = Wq.astype(np.float32) @ xr
    assert rel_err(raw, want_raw) < 1e-3
    y, want = sv * O.wht(raw), sv * O.wht(want_raw)
    assert rel_err(y, want) < 1e-3
    # and the quantised layer approximates the original weight: 2-bit Gaussian distortion ~ 26 % on W x
    exact = W.numpy() @ x.float().cpu().numpy()[0]
    assert 0.15 < rel_err(y, exact) < 0.40
    print("config 1: dequant bit-exact, GEMV rel err %.1e, vs unquantised W x %.3f" % (rel_err(y, want), rel_err(y, exact)))


@pytest.mark.parametrize("level", [2, 3, 4])
def test_config2_single_projection(level):
    """6144 -> 2048 as the gate|up projection of an expert with I = 1024 (2I = 2048 rows), B = 1 / 4 / 8"""
    H, I = 6144, 1024
    ex = F.Expert(H, I, seed=11, dev="cpu", nested=True)
    op = oracle_plane(ex.gu)
    signs = O.split_signs(ex.signs.numpy(), H, I)
    ex.gu.to(DEV); ex.dn.to(DEV); ex.signs = ex.signs.to(DEV)
    ex.gu.slot = ex.gu.nested_plane(); ex.dn.slot = ex.dn.nested_plane()
    Wq = O.dense_W(op, level, nested=True)
    L = M.MoELayer(1, H, I, Bmax=8, topk=1)
    L.set(0, ex, level)
    assert same_f16(M.dense_W(ex, 0, level).cpu().numpy(), Wq) == 0
    g = torch.Generator().manual_seed(level)
    for B in (1, 4, 8):
        x = (torch.randn(B, H, generator=g) * 0.05).half().to(DEV)
        raw = M.proj_gemv(L, x).cpu().numpy()
        xf = x.float().cpu().numpy()
        xg = O.wht(xf * signs["su_g"]).astype(np.float16).astype(np.float64)
        xu = O.wht(xf * signs["su_u"]).astype(np.float16).astype(np.float64)
        want = np.concatenate([xg @ Wq[:I].astype(np.float64).T, xu @ Wq[I:].astype(np.float64).T], 1)
        assert rel_err(raw, want) < 1e-4, (level, B)             # fp32 accumulation over K = 6144 with block-word extremes
