"""Prefill path (pre -> decode-fused grouped GEMM -> mid -> grouped GEMM -> post through the C ABI) against the float64
oracle and against the decode kernels run in 8-token slices (the reference's own cross-check, sm120/smoke_prefill.py)."""
import numpy as np
import pytest
import torch

from nestquant_amd import format as F, moe as M
from oracle import nq_oracle as O
from tests.test_gpu_moe import experts_on_gpu, oracle_layer, to_dev
from tests.util import oracle_plane, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def gumbel_topk(T, E, k, seed, skew=1.1):
    """Zipf(skew) expert popularity, k distinct experts per token (Gumbel top-k, as sm120/smoke_prefill.py:77-78)"""
    g = torch.Generator().manual_seed(seed)
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -skew
    p = (p / p.sum())[torch.randperm(E, generator=g)]
    u = torch.rand(T, E, generator=g, dtype=torch.float64).clamp_min(1e-300)
    ids = torch.topk(p.log()[None] - torch.log(-torch.log(u)), k, dim=-1).indices
    w = torch.rand(T, k, generator=g) + 0.1
    return ids.to(DEV), (w / w.sum(1, keepdim=True)).half().to(DEV)


def sliced_decode(L, x, sel, rw):
    out = torch.empty(x.shape[0], x.shape[1], dtype=torch.float32, device=DEV)
    for i in range(0, x.shape[0], 8):
        L(x[i:i + 8], sel[i:i + 8].contiguous(), rw[i:i + 8].contiguous(), out=out[i:i + 8])
    return out


def test_small_prefill_vs_oracle_and_slices():
    H, I, NE, T, K = 512, 256, 10, 70, 4
    rk = [(0, 0), (3, 7), (6, 9), (8, 3), (0, 0), (1, 2), (4, 5), (0, 0), (7, 6), (0, 0)]
    ex = experts_on_gpu(H, I, NE, 40, nested_ids=(4, 7, 9), rk=rk, var_ids=(1, 4))
    planes = [(oracle_plane(e.gu), oracle_plane(e.dn), e.nested) for e in ex]
    signs = [e.signs.numpy() for e in ex]
    levels = [2, 4, 4, 4, 3, 4, 4, 4, 2, 0]
    to_dev(ex)
    L = M.MoELayer(NE, H, I, Bmax=8, topk=K)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    sel, rw = gumbel_topk(T, NE, K, seed=3)
    rw[5, 1] = 0
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    hits = torch.zeros(NE, dtype=torch.int32, device=DEV)
    L.hits_ptr = hits.data_ptr()
    for R in (None, 64):                                         # one pass, and row chunks that split experts
        hits.zero_()
        y = L.prefill(x, sel, rw, R=R)
        torch.cuda.synchronize()
        want = oracle_layer(planes, levels, signs, x, sel, rw)
        assert rel_err(y.cpu().numpy(), want) < 5e-5, R
        want_hits = torch.bincount(sel[rw != 0].flatten().cpu(), minlength=NE)
        assert hits.cpu().tolist() == want_hits.tolist()
    L.hits_ptr = 0
    ys = sliced_decode(L, x, sel, rw)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), ys.cpu().numpy()) < 2e-5


def test_full_shape_prefill_vs_decode_slices():
    """H 6144, I 2048, 16 experts (levels 2/3/4/0), 300 tokens with Zipf popularity: tiles of every height occur"""
    H, I, NE, T = 6144, 2048, 16, 300
    levels = [4, 2, 4, 3, 2, 4, 4, 2, 3, 4, 2, 4, 0, 4, 2, 3]
    nested = tuple(i for i in range(NE) if levels[i] == 3 or i % 2 == 0)
    ex = to_dev(experts_on_gpu(H, I, NE, 500, nested_ids=nested, rk=[(6, 7) if i == 5 else (0, 0) for i in range(NE)]))
    L = M.MoELayer(NE, H, I, Bmax=8)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    sel, rw = gumbel_topk(T, NE, 8, seed=9)
    g = torch.Generator().manual_seed(10)
    x = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    y = L.prefill(x, sel, rw)
    ys = sliced_decode(L, x, sel, rw)
    torch.cuda.synchronize()
    cnt = torch.bincount(sel.flatten().cpu(), minlength=NE).tolist()
    kinds = M.pf_tiles([(e, 0, c) for e, c in enumerate(cnt) if c])
    assert max(cnt) > 256 and len(kinds) >= 3                    # multi-tile experts and remainder tiles of several heights
    assert rel_err(y.cpu().numpy(), ys.cpu().numpy()) < 5e-5     # two summation orders, each ~1e-5 from exact
    # float64 oracle on a few tokens through HIP-decoded dense weights (the decoder is proved bit-exact elsewhere)
    from tests.test_gpu_moe import _dense_from_gpu
    dense = _dense_from_gpu(ex, levels); signs = [e.signs.cpu().numpy() for e in ex]
    idx = [0, 137, 299]
    want = O.moe_forward(dense, levels, lambda e: signs[e], x[idx].cpu().numpy(), sel[idx].cpu().numpy(), rw[idx].cpu().numpy(), dtype=np.float64)
    assert rel_err(y[idx].cpu().numpy(), want) < 5e-5


def test_hot_expert_scratch_gives_the_same_bits():
    """experts with more than one 256-row tile decoded once into the operand scratch (nq_pf_wdecode, off by default): the
    grouped GEMM multiplies the same operands in the same order, so the result is bitwise the one of the decode-fused tiles"""
    H, I, NE, T = 1024, 512, 6, 700
    levels = [4, 2, 3, 4, 2, 4]
    ex = to_dev(experts_on_gpu(H, I, NE, 900, nested_ids=(0, 2, 4)))
    L = M.MoELayer(NE, H, I, Bmax=8)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    sel, rw = gumbel_topk(T, NE, 2, seed=5)
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    assert M.PF_HOT_SLOTS == 0
    y0 = L.prefill(x, sel, rw)
    torch.cuda.synchronize()
    cnt = torch.bincount(sel.flatten().cpu(), minlength=NE)
    assert int((cnt >= M.PF_HOT_MIN).sum()) >= 2                  # several experts qualify
    try:
        M.PF_HOT_SLOTS = 1                                       # fewer slots than hot experts: the rest keep decoding per tile
        y1 = L.prefill(x, sel, rw)
        M.PF_HOT_SLOTS = 4
        y2 = L.prefill(x, sel, rw)
        torch.cuda.synchronize()
    finally:
        M.PF_HOT_SLOTS = 0
    assert torch.equal(y0, y1) and torch.equal(y0, y2)
    ys = sliced_decode(L, x, sel, rw)
    torch.cuda.synchronize()
    assert rel_err(y0.cpu().numpy(), ys.cpu().numpy()) < 5e-5


def test_prefill_argument_errors_and_empty():
    L = M.MoELayer(4, 256, 256, Bmax=2, topk=2)
    tb = L.table
    with pytest.raises(RuntimeError, match="tile height"):
        t = torch.tensor([[0, 0, 4, 0]], dtype=torch.int32, device=DEV)
        buf = torch.zeros(8, 512, dtype=torch.float16, device=DEV); c = torch.zeros(8, 512, device=DEV)
        from nestquant_amd import _lib
        _lib.check(_lib.lib().nq_pf_gemm(tb.data_ptr(), t.data_ptr(), 1, 48, 0, buf.data_ptr(), buf.data_ptr(), c.data_ptr(), 4, 256, 256, None, None))
    x = torch.zeros(12, 256, dtype=torch.float16, device=DEV)
    sel = torch.zeros(12, 2, dtype=torch.int64, device=DEV); sel[:, 1] = 1
    rw = torch.full((12, 2), 0.5, dtype=torch.float16, device=DEV)
    y = L.prefill(x, sel, rw)                                    # every expert at level 0: output is zero, nothing faults
    torch.cuda.synchronize()
    assert not y.any()


def test_device_tile_planner_matches_host_lists():
    """nq_pf_plan against pf_tiles (the host construction the reference's prefill uses) for random expert counts and chunk
    windows: the same set of tiles per height, everything else marked as skipped"""
    from nestquant_amd import _lib
    g = torch.Generator().manual_seed(21)
    for E, scale in ((7, 40), (256, 300), (300, 5), (64, 2000)):
        cnt = (torch.rand(E, generator=g) ** 3 * scale).int()
        cnt[torch.randint(0, E, (max(1, E // 5),), generator=g)] = 0
        if E == 64:
            cnt[3] = 256; cnt[4] = 512; cnt[5] = 257; cnt[6] = 16; cnt[7] = 17
        P = int(cnt.sum())
        start = torch.cumsum(cnt, 0) - cnt
        for lo, n in ((0, P), (P // 3, P // 2), (0, 0), (P - 1, 1)) if P else ((0, 0),):
            segs = []
            for e in range(E):
                u, v = max(int(start[e]), lo), min(int(start[e] + cnt[e]), lo + n)
                if v > u:
                    segs.append((e, u - lo, v - u))
            want = {bm: sorted(map(tuple, t.tolist())) for bm, t in M.pf_tiles(segs).items()}
            cap = E + n // 256 + 1
            tiles = torch.full((5, cap, 4), 77, dtype=torch.int32, device=DEV)
            _lib.check(_lib.lib().nq_pf_plan(cnt.to(DEV).data_ptr(), E, lo, n, tiles.data_ptr(), cap, None, 0, 0, None))
            torch.cuda.synchronize()
            t = tiles.cpu()
            for i in range(5):
                used = t[i, : (E if i < 4 else cap)]
                live = used[used[:, 0] >= 0]
                assert sorted(map(tuple, live.tolist())) == want.get(16 << i, []), (E, lo, n, i)
                assert bool((used[used[:, 0] < 0][:, 0] == -1).all())
                covered = sum(r for _, _, r, _ in live.tolist())
            total = sum(int(t[i, : (E if i < 4 else cap)][t[i, : (E if i < 4 else cap), 0] >= 0][:, 2].sum()) for i in range(5))
            assert total == n
    with pytest.raises(RuntimeError, match="cap"):
        _lib.check(_lib.lib().nq_pf_plan(cnt.to(DEV).data_ptr(), 64, 0, 1024, tiles.data_ptr(), 64, None, 0, 0, None))


def test_prefill_on_a_side_stream_matches_the_default_stream():
    """prefill() forks its grouped-GEMM launches onto side streams and joins them again: the result must not depend on which
    stream the caller is on, nor on work the caller queued right before and after it"""
    H, I, NE, T = 512, 256, 8, 200
    ex = to_dev(experts_on_gpu(H, I, NE, 640, rk=[(3, 9)] * NE))
    L = M.MoELayer(NE, H, I, Bmax=8, topk=4)
    for e in range(NE):
        L.set(e, ex[e], (4, 2, 4, 4, 2, 4, 0, 4)[e])
    sel, rw = gumbel_topk(T, NE, 4, seed=3)
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(T, H, generator=g) * 0.05).half().to(DEV)
    want = L.prefill(x, sel, rw).clone()
    torch.cuda.synchronize()
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        x2 = x * 1.0                                                # produced on the side stream just before the call
        got = L.prefill(x2, sel, rw)
        got2 = got * 2.0                                            # consumed on it right after
    s2.synchronize()
    assert torch.equal(got, want) and torch.equal(got2, want * 2.0)
    for _ in range(3):                                              # back to back: the scratch is reused, nothing overtakes
        assert torch.equal(L.prefill(x, sel, rw), want)


def test_row_restricted_pre_and_mid_cover_the_rows_of_their_heights_exactly():
    """nq_pf_pre_rows / nq_pf_mid_rows over the five single-height masks write, together, bitwise what nq_pf_pre / nq_pf_mid
    write, each launch only the rows of tiles of its height (everything else keeps the fill value), with the height of a row
    taken from the host construction of the tile lists"""
    from nestquant_amd import _lib
    Lb = _lib.lib()
    H, I, E = 256, 512, 12
    ex = to_dev(experts_on_gpu(H, I, E, 900, rk=[(0, 3)] * E))
    L = M.MoELayer(E, H, I, Bmax=8, topk=2)
    for e in range(E):
        L.set(e, ex[e], 4 if e % 3 else 2)
    g = torch.Generator().manual_seed(77)
    cnt = torch.tensor([0, 5, 16, 17, 40, 64, 100, 129, 256, 300, 513, 31])
    pe = torch.repeat_interleave(torch.arange(E), cnt).int()
    pe[3] = -1; pe[40] = E + 2                                   # rows of no valid expert: height 256 by convention
    n = int(cnt.sum())
    T = 50
    pt = torch.randint(0, T, (n,), generator=g).int()
    x = (torch.randn(T, H, generator=g) * 0.3).half().to(DEV)
    acc = torch.randn(n, 2 * I, generator=g).to(DEV)
    pe_d, pt_d = pe.to(DEV), pt.to(DEV)
    cap = E + n // 256 + 1
    tiles = torch.empty(5, cap, 4, dtype=torch.int32, device=DEV)
    _lib.check(Lb.nq_pf_plan(cnt.int().to(DEV).data_ptr(), E, 0, n, tiles.data_ptr(), cap, None, 0, 0, None))
    # height class of every row from the host lists
    start = torch.cumsum(cnt, 0) - cnt
    cls = torch.full((n,), 4)
    for bm, t in M.pf_tiles([(e, int(start[e]), int(cnt[e])) for e in range(E) if cnt[e]]).items():
        for e, r0, rows, _ in t.tolist():
            cls[r0:r0 + rows] = bm.bit_length() - 5
    cls[3] = cls[40] = 4
    assert sorted(set(cls.tolist())) == [0, 1, 2, 3, 4]

    def pre(rows_mask):
        xg = torch.full((n, H), 7.0, dtype=torch.float16, device=DEV); xu = torch.full_like(xg, 7.0)
        a = (x.data_ptr(), pt_d.data_ptr(), pe_d.data_ptr(), n, L.table.data_ptr(), xg.data_ptr(), xu.data_ptr(), None, E, H, I)
        _lib.check(Lb.nq_pf_pre(*a, None) if rows_mask is None else Lb.nq_pf_pre_rows(*a, tiles.data_ptr(), cap, rows_mask, None))
        return xg.cpu(), xu.cpu()

    def mid(rows_mask):
        h = torch.full((n, I), 7.0, dtype=torch.float16, device=DEV)
        a = (acc.data_ptr(), pe_d.data_ptr(), n, L.table.data_ptr(), h.data_ptr(), None, None, E, H, I)
        _lib.check(Lb.nq_pf_mid(*a, None) if rows_mask is None else Lb.nq_pf_mid_rows(*a, tiles.data_ptr(), cap, rows_mask, None))
        return (h.cpu(),)

    for fn in (pre, mid):
        whole = fn(None)
        for k in range(5):
            part = fn(1 << k)
            for w, q in zip(whole, part):
                mine = cls == k
                assert torch.equal(q[mine], w[mine]) and bool((q[~mine] == 7.0).all()), (fn.__name__, k)
        assert all(torch.equal(a, b) for a, b in zip(fn(31), whole))
