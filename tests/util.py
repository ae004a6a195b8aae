"""Test helpers: bridges between the package's torch planes and the numpy oracle (tests only)."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import nq_oracle as O  # noqa: E402


def u32(t):
    """torch int32/int64 tensor holding uint32 values -> numpy uint32"""
    a = t.detach().cpu().numpy()
    return (a.astype(np.int64) & 0xFFFFFFFF).astype(np.uint32)


def oracle_plane(p):
    """nestquant_amd.format.Proj -> oracle Plane (host numpy)"""
    nrec = p.z["S"] * p.z["C"] * 32
    res = O.unpack_words(p.p4.cpu().numpy(), p.z["nrec_r"], O.rbits(p.rk))
    kw = {}
    if getattr(p, "nested", False):
        kw = dict(p3=O.unpack_words(p.p3.cpu().numpy(), nrec, 64), d3=u32(p.d3),
                  p4n=O.unpack_words(p.p4n.cpu().numpy(), nrec, 64), d4n=u32(p.d4n))
    bk = int(getattr(p, "bk", 0) or 0)
    base = u32(p.base).reshape(-1, 4) if bk == 0 else O.unpack_words(p.base.cpu().numpy(), nrec, O.rbits(bk))
    return O.Plane(p.N, p.K, base, rk=p.rk, bk=bk, res=res, d4=u32(p.d4),
                   var=None if p.var is None else p.var.cpu().numpy(),
                   flags=None if getattr(p, "flags", None) is None else p.flags.cpu().numpy(), **kw)


def same_f16(a, b):
    """bitwise equality of fp16 arrays with +0 and -0 identified; returns number of differing elements"""
    a = np.asarray(a).view(np.uint16).astype(np.int32)
    b = np.asarray(b).view(np.uint16).astype(np.int32)
    diff = a != b
    zero = ((a & 0x7FFF) == 0) & ((b & 0x7FFF) == 0)
    return int((diff & ~zero).sum())


def rel_err(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
