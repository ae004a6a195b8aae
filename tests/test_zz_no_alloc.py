"""nq_moe_forward_static (workspaces in the library's built-in device scratch, nothing allocated) against nq_moe_forward
(workspaces of the caller's), both through the C ABI: same kernels, so every bit of the output must agree. Two calls in a
row share the scratch, the second with a smaller input; then the shapes the scratch cannot hold are refused."""
import ctypes as C

import pytest
import torch

from nestquant_amd import _lib, format as F, moe as M, routing as RT

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _layer(H, I, NE, levels, topk, Bmax, seed0):
    ex = [F.Expert(H, I, seed=seed0 + i, dev="cpu", nested=levels[i] == 3 or i % 2 == 0, var=i == 1) for i in range(NE)]
    for e in ex:
        e.gu.to(DEV); e.dn.to(DEV); e.signs = e.signs.to(DEV)
        if e.nested:
            e.gu.slot = e.gu.nested_plane(); e.dn.slot = e.dn.nested_plane()
    L = M.MoELayer(NE, H, I, Bmax=Bmax, topk=topk)
    for e in range(NE):
        L.set(e, ex[e], levels[e])
    return L, ex


def test_static_scratch_entry_equals_caller_workspace_entry():
    H, I, NE, topk = 1024, 512, 8, 4
    levels = [2, 4, 3, 4, 0, 2, 4, 3]
    L, ex = _layer(H, I, NE, levels, topk, 8, 300)            # ex: the table holds raw addresses of these planes
    g = torch.Generator().manual_seed(5)
    import random
    rng = random.Random(3)
    alloc = []
    for B in (8, 3, 5, 1):                                     # a big call, then smaller ones into the same scratch
        sel, rw = RT.routing_tensors(RT.make_sel(B, range(NE), "recency", p=0.5, rng=rng, topk=topk), seed=B)
        if B == 3:
            rw[1, 2] = 0
        x = (torch.randn(B, H, generator=g) * 0.05).half().to(DEV)
        want = L(x, sel, rw).clone()
        torch.cuda.synchronize()
        out = torch.full((B, H), float("nan"), dtype=torch.float32, device=DEV)
        before = torch.cuda.memory_allocated()
        L(x, sel, rw, out=out, static_ws=True)
        L(x, sel, rw, out=out, static_ws=True)                 # again: the counters of the first call are back at zero
        torch.cuda.synchronize()
        alloc.append(torch.cuda.memory_allocated() - before)
        assert torch.equal(out, want), B
        # other tilings and a bf16 result, still bitwise the caller-workspace result
        for cg, cd in (([1, 2, 2], [1, 1, 2]), ([2, 4, 2], [1, 4, 1])):
            want = L(x, sel, rw, cfg_gu=cg, cfg_dn=cd).clone()
            got = L(x, sel, rw, out=torch.empty_like(out), cfg_gu=cg, cfg_dn=cd, static_ws=True)
            assert torch.equal(got, want), (B, cg, cd)
        wb = L(x, sel, rw, out=torch.empty(B, H, dtype=torch.bfloat16, device=DEV))
        gb = L(x, sel, rw, out=torch.empty(B, H, dtype=torch.bfloat16, device=DEV), static_ws=True)
        assert torch.equal(gb, wb)
    assert alloc == [0, 0, 0, 0]
    # torch's counter sees only torch's allocator; the driver's own count of free device memory (hipMemGetInfo) would show a
    # hipMalloc / hipFree inside the library, and a call recorded into a graph cannot allocate at all (it would fail the capture)
    out = torch.empty(B, H, dtype=torch.float32, device=DEV)
    want = L(x, sel, rw).clone()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(8):
        L(x, sel, rw, out=out, static_ws=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    st = torch.cuda.Stream()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        L(x, sel, rw, out=out, static_ws=True)
    torch.cuda.synchronize()
    with torch.cuda.graph(gr, stream=st):
        L(x, sel, rw, out=out, static_ws=True)
    for _ in range(3):                                         # every replay against the eager result, eager work between them
        out.fill_(float("nan"))
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        assert torch.equal(L(x, sel, rw).clone(), want)
    del ex
    assert int(L.cnt_gu.abs().sum()) == 0 and int(L.cnt_d.abs().sum()) == 0


def test_static_entry_full_shape_and_refusal():
    """the full layer shape at B = 2 fits the scratch; a k-split too fine for it is refused on the host with a message"""
    H, I, NE = 6144, 2048, 4
    L, ex = _layer(H, I, NE, [2, 4, 3, 4], 4, 2, 320)
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(2, H, generator=g) * 0.05).half().to(DEV)
    sel = torch.tensor([[0, 1, 2, 3], [3, 2, 1, 0]], device=DEV)
    rw = torch.tensor([[.4, .3, .2, .1], [.25, .25, .25, .25]], device=DEV).half()
    want = L(x, sel, rw).clone()
    got = L(x, sel, rw, out=torch.empty(2, H, dtype=torch.float32, device=DEV), static_ws=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    Lb, exb = _layer(H, I, NE, [2, 4, 3, 4], 8, 8, 320)
    x8 = (torch.randn(8, H, generator=g) * 0.05).half().to(DEV)
    sel8 = torch.arange(8, device=DEV).repeat(8, 1) % NE
    rw8 = torch.full((8, 8), 0.125, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="built-in scratch holds"):
        Lb(x8, sel8, rw8, cfg_gu=[1, 4, 1], cfg_dn=[1, 4, 1], static_ws=True)       # 48 + 16 k-slices of 64 picks: 72 MiB
    # and the refusal left nothing behind: the next call is right
    got = L(x, sel, rw, out=torch.empty(2, H, dtype=torch.float32, device=DEV), static_ws=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    del ex, exb
