"""NestQuant grouped MoE layer on MI355X: device table, workspaces, launch wrappers.

Host-side mirror of the reference's Python op surface (sm120/moe.py): `entry` :216-229, `MoELayer` :231-260,
`prefill` :282-326, `Mailbox` :329-342, `dense_W` :156-166, `H128` :168-172. The kernels behind it are the HIP kernels of
libnq_moe_hip.so, reached through ctypes with raw device pointers; there is no CPU path in this module.
"""
import ctypes as C

import torch

from . import _lib
from .format import (CODE_L3, CODE_L4N, RK_OF, RKP, TBL_W, Expert, Proj, all_MbN, pack_words, popc, proj_sizes,  # noqa: F401
                     rbits, split_bits, step_off, unpack_words)


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def had_dn(ex):
    """down-projection input Hadamard width (absent = 128)"""
    return int(getattr(ex, "had_dn", 128) or 128)


def base_code(p):
    return int(getattr(p, "bk", 0) or 0)


def H128(dev="cuda", n=128):
    """normalised Sylvester Hadamard matrix of order n"""
    H = torch.ones(1, 1)
    while H.shape[0] < n:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    return (H / n**0.5).to(dev)


def entry(ex, level):
    """table row int64[TBL_W] of expert `ex` at `level` (0, 2, 3, 4). Level 3 and, for experts built with nested=True,
    level 4 point at the nested planes (codes 10 / 11); otherwise level 4 points at the wide residual plane p4 (code rk)."""
    e = torch.zeros(TBL_W, dtype=torch.int64)
    e[0] = level
    nested = bool(getattr(ex, "nested", False))
    if level == 3 and not nested:
        raise ValueError("level 3 needs an expert with nested planes")
    for off, p in ((1, ex.gu), (5, ex.dn)):
        e[off] = p.base.data_ptr()
        if nested:
            slot = p.slot
            e[off + 1] = slot.data_ptr()
            e[off + 2] = (p.d3 if level == 3 else p.d4n).data_ptr()
        else:
            e[off + 1] = p.p4.data_ptr()
            e[off + 2] = p.d4.data_ptr()
        if getattr(p, "flags", None) is not None:
            e[off + 3] = p.flags.data_ptr()
    e[9] = ex.signs.data_ptr()
    if nested:
        e[10] = e[11] = CODE_L3 if level == 3 else CODE_L4N
    else:
        e[10], e[11] = ex.gu.rk, ex.dn.rk
    for i, p in ((12, ex.gu), (13, ex.dn)):
        v = getattr(p, "var", None)
        e[i] = 0 if v is None else v.data_ptr()
    lr = getattr(ex, "lr", None)
    if lr is not None:
        e[14] = lr.data_ptr(); e[15] = ex.lr4.data_ptr(); e[16] = ex.rg; e[17] = ex.rd
    w = had_dn(ex)
    e[18] = 0 if w == 128 else w
    e[19] = base_code(ex.gu) | base_code(ex.dn) << 8
    return e


def validate_row(row, H, I):
    """raise RuntimeError if the row uses a field or code the kernels do not implement"""
    r = row.to("cpu", torch.int64).contiguous()
    _lib.check(_lib.lib().nq_validate_row(C.cast(r.data_ptr(), C.POINTER(C.c_int64)), H, I))


def rk_codes():
    """[gate|up mask, down mask] of compiled residual window codes"""
    out = (C.c_uint32 * 4)()
    _lib.check(_lib.lib().nq_codes(out))
    return [int(out[0]), int(out[1])]


def bk_codes():
    out = (C.c_uint32 * 4)()
    _lib.check(_lib.lib().nq_codes(out))
    return [int(out[2]), int(out[3])]


def dequant(row_dev, proj, H, I, level=0, out=None):
    """HIP dense decode of one projection from a table row on the device -> fp16 [N, K]"""
    N, K = (2 * I, H) if proj == 0 else (H, I)
    if out is None:
        out = torch.empty(N, K, dtype=torch.float16, device=row_dev.device)
    _lib.check(_lib.lib().nq_dequant(_ptr(row_dev), proj, level, H, I, _ptr(out), _lib.stream_ptr()))
    return out


def dense_W(ex, proj, level, dtype=torch.float16):
    """dense rotated-domain weights [N, K] of projection `proj` (0 gate|up, 1 down) of expert `ex`, decoded on the GPU"""
    row = entry(ex, level)
    validate_row(row, ex.H, ex.I)
    row = row.to(ex.signs.device)
    return dequant(row, proj, ex.H, ex.I).to(dtype)
