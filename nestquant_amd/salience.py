"""Decode salience export next to the routing hit counters: sal[e] += (rsf w)^2 |x|^2 per pick of expert e.

Host-side mirror of the module the reference obtains from build.get_sal() (sm120/nqsal.cu:62-78; called by the serving
step at sm120/serve/nq_vllm.py:558,572). `sal` has the reference's signature; besides fp16 / bf16 activations, fp16
weights and int64 ids it also takes what moe.forward takes (fp32 activations, bf16 / fp32 weights, int32 ids), reading
them as the casts x.half(), w.half(), ids.long() would leave them.
"""
import ctypes as C

import torch

from . import _lib
from .moe import _DT_IN, _DT_SEL


def sal(x, w, ids, rsf, acc, host_ptr):
    """x [T, H] (last dimension contiguous), w [T, K], ids [T, K], T <= 8, K <= 8; acc float64 [E] on the device; host_ptr
    the address of a pinned float64 [E] the kernel mirrors every touched entry to (a tensor is accepted too)."""
    if not (x.dim() == 2 and x.stride(1) == 1 and x.dtype in _DT_IN):
        raise RuntimeError("nqsal: x must be [T, H] fp16 / bf16 / fp32 with a contiguous last dimension")
    if not (w.is_contiguous() and ids.is_contiguous() and w.dtype in _DT_IN and ids.dtype in _DT_SEL and ids.dim() == 2
            and w.numel() == ids.numel() == x.shape[0] * ids.shape[1]):
        raise RuntimeError("nqsal: w / ids must be contiguous [T, K] (fp16 / bf16 / fp32 and int64 / int32)")
    if acc.dtype != torch.float64 or not acc.is_contiguous():
        raise RuntimeError("nqsal: acc must be contiguous float64")
    if isinstance(host_ptr, torch.Tensor):
        if host_ptr.dtype != torch.float64 or not host_ptr.is_pinned() or host_ptr.numel() < acc.numel():
            raise RuntimeError("nqsal: the host mirror must be pinned float64 [E]")
        host_ptr = host_ptr.data_ptr()
    if not host_ptr:
        raise RuntimeError("nqsal: the host mirror must be given")
    _lib.check(_lib.lib().nq_sal(C.c_void_p(x.data_ptr()), _DT_IN[x.dtype], x.stride(0), C.c_void_p(w.data_ptr()), _DT_IN[w.dtype],
                                 C.c_void_p(ids.data_ptr()), _DT_SEL[ids.dtype], x.shape[0], x.shape[1], ids.shape[1], acc.numel(),
                                 float(rsf), C.c_void_p(acc.data_ptr()), C.c_void_p(host_ptr), _lib.stream_ptr()))


class Salience:
    """the per-layer state the serving step keeps (reference sm120/serve/nq_vllm.py:192-197): device accumulator, pinned
    host mirror, routed scaling factor"""

    def __init__(s, E, rsf=1.0, dev="cuda"):
        s.acc = torch.zeros(E, dtype=torch.float64, device=dev)
        s.host = torch.zeros(E, dtype=torch.float64).pin_memory()
        s.rsf = float(rsf)

    def __call__(s, x, w, ids):
        sal(x, w, ids, s.rsf, s.acc, s.host.data_ptr())
