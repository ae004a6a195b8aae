"""ctypes binding of the C oracle (oracle/nq_oracle.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "_build", "libnq_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-B", "_build/libnq_oracle.so"], check=True, capture_output=True)
    return LIB


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = C.CDLL(LIB)
        L.nqo_rbits.restype = C.c_int; L.nqo_rbits.argtypes = [C.c_int]
        L.nqo_step_off.restype = C.c_int; L.nqo_step_off.argtypes = [C.c_int, C.c_int]
        L.nqo_hash_sum.restype = C.c_int; L.nqo_hash_sum.argtypes = [C.c_uint32]
        L.nqo_f32_to_f16.restype = C.c_uint16; L.nqo_f32_to_f16.argtypes = [C.c_float]
        L.nqo_f16_to_f32.restype = C.c_float; L.nqo_f16_to_f32.argtypes = [C.c_uint16]
        L.nqo_fold_consts.restype = None
        L.nqo_fold_consts.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_uint16), C.POINTER(C.c_uint16)]
        L.nqo_unpack.restype = None; L.nqo_unpack.argtypes = [C.c_void_p, C.c_long, C.c_int, C.c_int, C.c_void_p]
        L.nqo_decode_proj.restype = None
        L.nqo_decode_proj.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.nqo_matvec_f16.restype = None
        L.nqo_matvec_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def unpack(buf, nrec, code, split=False):
    """split: False / 0 = the sub-array layout of `code`; True / 1 = P3's 64-bit records followed by P4's, concatenated per record
    (code 11); 2 = the same storage, interleaved bit by bit per record (code 12)"""
    buf = np.ascontiguousarray(np.frombuffer(np.ascontiguousarray(buf).tobytes(), np.uint8))
    nw = (lib().nqo_rbits(code) + 31) // 32
    out = np.zeros((nrec, nw), np.uint32)
    lib().nqo_unpack(_p(buf), nrec, code, int(split), _p(out))
    return out


def decode_proj(base, N, K, level, code=0, res=None, dw=None, var=None):
    """dense [N, K] fp16 decode; base [nrec,4] uint32, res [nrec,NW] uint32 unpacked words, dw uint32 [units]"""
    base = np.ascontiguousarray(base, np.uint32)
    res = None if res is None else np.ascontiguousarray(res, np.uint32)
    dw = None if dw is None else np.ascontiguousarray(dw, np.uint32)
    var = None if var is None else np.ascontiguousarray(var, np.uint8)
    out = np.empty((N, K), np.uint16)
    lib().nqo_decode_proj(_p(base), _p(res), code, _p(dw), _p(var), N, K, level, _p(out))
    return out.view(np.float16)


def matvec_f16(W, x):
    W = np.ascontiguousarray(W).view(np.uint16); x = np.ascontiguousarray(x, np.float32)
    y = np.empty(W.shape[0], np.float32)
    lib().nqo_matvec_f16(_p(W), _p(x), W.shape[0], W.shape[1], _p(y))
    return y


def fold_consts(Mb, N):
    a, c = C.c_uint16(), C.c_uint16()
    lib().nqo_fold_consts(int(Mb), int(N), C.byref(a), C.byref(c))
    return a.value, c.value
