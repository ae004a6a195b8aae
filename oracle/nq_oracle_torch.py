"""torch-CPU restatement of the reference's own CPU path for one layer step.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module; it exists so that bench.py's cpu_baseline leg can time, on the GPU
box's host cores, the computation the reference runs when it has no kernel: dense decode of every routed expert in
vectorised torch, then fp32 matmuls (reference sm120/moe.py: lane_sums / fold_vals / lane_vals :111-153, dense_W :156-166,
H128 :168-172, Expert.ref :196-210, moe_ref :344-351). It takes the oracle's Plane objects (numpy, host memory) and follows
the numpy oracle (oracle/nq_oracle.py) operation for operation, with torch tensors in place of numpy arrays, so that
torch.set_num_threads decides how many cores the decode and the matmuls use.

Pinned by tests/test_oracle_torch.py: dense_W equals the numpy oracle's bit for bit (which the golden fixtures of the
reference's decoder pin) at levels 2 / 3 / 4 for wide and nested planes with sign variants, and the layer output equals
the numpy oracle's fp32 layer math to fp32 rounding. Mask mode, other base codes and G = 2 are not restated here (the
benchmark's planes use none of them); asking for them raises.
"""
import numpy as np
import torch

from . import nq_oracle as O

_I64 = torch.int64


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(np.asarray(a, np.uint32).astype(np.int64)))


def lane_sums(words, code):
    """words [nrec, NW] (int64 holding uint32) -> byte sum S(state) of each of the 64 lane weights, int64 [nrec, 64]
    (reference sm120/moe.py:111-127; rings of four lanes)."""
    ka, mask = O.RKP[code]
    bits = O.rbits(code)
    nrec, nw = words.shape
    lane = torch.arange(nrec)
    nb = (lane // 4) * 4 + (lane % 4 + 1) % 4
    first = words[nb, 0]
    ext = torch.zeros(nrec, nw + 2, dtype=_I64)
    ext[:, :nw] = words
    t = bits % 32
    if t == 0:
        ext[:, nw] = first
    else:
        ext[:, nw - 1] = (ext[:, nw - 1] & ((1 << t) - 1)) | ((first << t) & 0xFFFFFFFF)
        ext[:, nw] = first >> (32 - t)
    offs = O.step_off(np.arange(64), ka, mask)
    out = torch.empty(nrec, 64, dtype=_I64)
    for j in range(64):
        o = int(offs[j]); i, s = o >> 5, o & 31
        st = ((ext[:, i] | (ext[:, i + 1] << 32)) >> s) & 0xFFFF
        x = (st * O.HC) & 0xFFFFFFFF
        out[:, j] = (x & 255) + ((x >> 8) & 255) + ((x >> 16) & 255) + (x >> 24)
    return out


def fold_consts(Mb, N):
    """per-unit fp16 constants of the integer fold, fp32 operations in the spec's order (reference sm120/moe.py:128-132)"""
    rcp = torch.tensor(1.0, dtype=torch.float32) / Mb.float()
    Ah = (torch.tensor(1.732421875, dtype=torch.float32) * rcp).half()
    k0 = torch.tensor(O.K0, dtype=torch.float32)
    tt = (N.float() * rcp) * k0 + k0
    Ch = (tt - torch.tensor(1024.0, dtype=torch.float32) * Ah.float()).half()
    return Ah, Ch


def lane_vals(p, level, nested):
    """decoded weights in lane-weight order, fp16 [S, C, 32, 64] (reference sm120/moe.py:136-153)"""
    if p.flags is not None or p.bk != 0:
        raise NotImplementedError("the torch restatement covers dense planes over the K = 2 base only")
    S, C = p.S, p.C
    Sb = lane_sums(_t(p.base), 0).reshape(S, C, 32, 64)
    sign = 1.0
    if p.var is not None:
        ring = torch.arange(32) >> 2
        bit = (torch.from_numpy(np.asarray(p.var, np.int64)).reshape(S, C, 1) >> ring) & 1
        sign = (1.0 - 2.0 * bit.double())[..., None]
    if level == 2:
        return ((sign * O.A_) * (1024.0 + Sb.double()) + sign * O.B_).half()
    code, words, dw = p.residual(level, nested)
    Sr = lane_sums(_t(words), code).reshape(S, C, 32, 64)
    dw = _t(dw).reshape(S, C, 1, 1)
    Mb, N = dw & 255, (dw >> 8) & 255
    Ah, Ch = fold_consts(Mb, N)
    F = (Mb * Sb + N * Sr + 128) >> 8
    return ((sign * Ah.double()) * (1024.0 + F.double()) + sign * Ch.double()).half()


def dense_W(p, level, nested=False):
    """dense rotated-domain weights [N, K] fp16 (reference sm120/moe.py:156-166)"""
    f = lane_vals(p, level, nested)
    S, C = p.S, p.C
    row, col = O.lane_to_rowcol()
    row, col = torch.from_numpy(row + 0 * col), torch.from_numpy(col + 0 * row)
    W = torch.zeros(p.N, p.K, dtype=torch.float16)
    rows = (torch.arange(S).reshape(S, 1, 1, 1) * 16 + row[None, None]).expand(S, C, 32, 64)
    cols = (torch.arange(C).reshape(1, C, 1, 1) * 128 + col[None, None]).expand(S, C, 32, 64)
    W[rows.reshape(-1), cols.reshape(-1)] = f.reshape(-1)
    return W


def H128(n=128):
    H = torch.ones(1, 1)
    while H.shape[0] < n:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    return H / n ** 0.5


def expert_ref(x, Wgu, Wdn, signs):
    """x [T, H] fp32 -> [T, H] fp32 through dense fp16 weights (reference Expert.ref, sm120/moe.py:196-210)"""
    H, I = Wdn.shape
    had = lambda v: (v.reshape(*v.shape[:-1], -1, 128) @ H128()).reshape(v.shape)
    su_g, sv_g, sv_u, su_d, sv_o, su_u = torch.split(signs.float(), [H, I, I, I, H, H])
    Wg, Wu, Wd = Wgu[:I].float(), Wgu[I:].float(), Wdn.float()
    g = had(had(x * su_g).half().float() @ Wg.T) * sv_g
    u = had(had(x * su_u).half().float() @ Wu.T) * sv_u
    h = had(torch.nn.functional.silu(g) * u * su_d).half().float()
    return had(h @ Wd.T) * sv_o


def moe_ref(planes, levels, signs, x, sel, rw):
    """layer output fp32 [T, H] (reference moe_ref, sm120/moe.py:344-351): every distinct routed expert is decoded once.
    planes: e -> (Plane gate|up, Plane down, nested); signs: e -> fp16 vector (numpy); x [T, H], sel [T, k], rw [T, k] numpy."""
    x = torch.from_numpy(np.asarray(x, np.float32)); T, H = x.shape
    y = torch.zeros(T, H, dtype=torch.float32)
    w = np.asarray(rw, np.float32)
    for e in sorted(set(np.asarray(sel).reshape(-1).tolist())):
        if levels[e] <= 0:
            continue
        hit = (np.asarray(sel) == e) & (w != 0)
        rows = np.nonzero(hit.any(1))[0]
        if rows.size == 0:
            continue
        pg, pd, nested = planes(e)
        Wgu, Wdn = dense_W(pg, levels[e], nested), dense_W(pd, levels[e], nested)
        ye = expert_ref(x[rows], Wgu, Wdn, torch.from_numpy(np.asarray(signs(e)).view(np.float16).copy()))
        y[rows] += torch.from_numpy((w * hit)[rows].sum(1, keepdims=True)) * ye
    return y
