"""ctypes binding of libnq_moe_hip.so (the C ABI in include/nq_moe_hip.h).

There is no fallback: if the library is missing, `lib()` raises. Build it with `python -m nestquant_amd.build`.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnq_moe_hip.so")
_lib = None

_vp, _i, _i64p, _i32p = C.c_void_p, C.c_int, C.c_void_p, C.c_void_p

class NqMoeArgs(C.Structure):
    """mirror of struct NqMoeArgs in include/nq_moe_hip.h"""
    _fields_ = [("x", C.c_void_p), ("sel", C.c_void_p), ("rw", C.c_void_p), ("table", C.c_void_p), ("out", C.c_void_p),
                ("acc_gu", C.c_void_p), ("h", C.c_void_p), ("acc_d", C.c_void_p), ("cnt_gu", C.c_void_p), ("cnt_d", C.c_void_p),
                ("hits", C.c_void_p),
                ("acc_gu_elems", C.c_int64), ("acc_d_elems", C.c_int64), ("h_elems", C.c_int64), ("out_elems", C.c_int64),
                ("cnt_gu_elems", C.c_int64), ("cnt_d_elems", C.c_int64),
                ("B", C.c_int32), ("topk", C.c_int32), ("E", C.c_int32), ("H", C.c_int32), ("I", C.c_int32),
                ("cfg_gu", C.c_int32 * 4), ("cfg_dn", C.c_int32 * 4), ("force_level", C.c_int32), ("which", C.c_int32),
                ("x_dtype", C.c_int32), ("sel_dtype", C.c_int32), ("rw_dtype", C.c_int32), ("out_dtype", C.c_int32),
                ("cnt_h", C.c_void_p), ("cnt_h_elems", C.c_int64), ("zd", C.c_void_p), ("zd_elems", C.c_int64),
                ("common_rows", C.c_int32), ("G", C.c_int32),
                ("route_ws", C.c_void_p), ("route_ws_bytes", C.c_int64), ("xrot", C.c_void_p), ("xrot_elems", C.c_int64),
                ("mb_table", C.c_void_p), ("mb_stage", C.c_void_p), ("mb_seq", C.c_void_p), ("mb_applied", C.c_void_p),
                ("mb_applied_host", C.c_void_p), ("hoist_value_map", C.c_int32), ("reserved_", C.c_int32)]


ROUTE_WS_BYTES = 32768          # NQ_ROUTE_WS_BYTES


# name -> (restype, argtypes); every symbol declared in include/nq_moe_hip.h
SIGNATURES = {
    "nq_abi_version": (C.c_int, []),
    "nq_last_error": (C.c_char_p, []),
    "nq_codes": (C.c_int, [C.POINTER(C.c_uint32)]),
    "nq_occ": (C.c_int, [_i, _i, _i, _i, C.POINTER(C.c_int)]),
    "nq_validate_row": (C.c_int, [C.POINTER(C.c_int64), _i, _i]),
    "nq_dequant": (C.c_int, [_i64p, _i, _i, _i, _i, _vp, _vp]),
    "nq_pf_decode": (C.c_int, [_i64p, _i32p, _i, _vp, _vp, _i, _i, _vp]),
    "nq_moe_forward": (C.c_int, [C.POINTER(NqMoeArgs), _vp]),
    "nq_moe_forward_static": (C.c_int, [C.POINTER(NqMoeArgs), _vp]),
    "nq_sal": (C.c_int, [_vp, _i, C.c_int64, _vp, _i, _vp, _i, _i, _i, _i, _i, C.c_double, _vp, _vp, _vp]),
    "nq_mailbox": (C.c_int, [_i64p, _i64p, _i32p, _i32p, _i32p, _i, _vp]),
    "nq_pf_pre": (C.c_int, [_vp, _i32p, _i32p, _i, _i64p, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "nq_pf_pre_rows": (C.c_int, [_vp, _i32p, _i32p, _i, _i64p, _vp, _vp, _vp, _i, _i, _i, _i32p, _i, _i, _vp]),
    "nq_pf_gemm": (C.c_int, [_i64p, _i32p, _i, _i, _i, _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "nq_pf_wdecode": (C.c_int, [_i64p, _i32p, _i, _i, _vp, C.c_int64, _i, _i, _i, _vp]),
    "nq_pf_mid": (C.c_int, [_vp, _i32p, _i, _i64p, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "nq_pf_mid_rows": (C.c_int, [_vp, _i32p, _i, _i64p, _vp, _vp, _vp, _i, _i, _i, _i32p, _i, _i, _vp]),
    "nq_pf_post": (C.c_int, [_vp, _i32p, _i64p, _vp, _i, _i, _i, _i, _i64p, _vp, _vp, _i, _i, _i, _vp]),
    "nq_pf_plan": (C.c_int, [_i32p, _i, _i, _i, _i32p, _i, _i32p, _i, _i, _vp]),
    "nq_pf_hits": (C.c_int, [_i32p, _i32p, _i, _vp]),
    # record upgrade engine (host threads; structures mirrored in stream_engine.py)
    "nq_stream_open": (C.c_void_p, [C.c_char_p, C.c_char_p, C.c_int64, _i, _i, _i, _i]),
    "nq_stream_upgrade": (C.c_int, [_vp, C.c_int64, C.c_int64, _vp, _vp, C.POINTER(C.c_int64), _vp, C.c_int32]),
    "nq_stream_post": (C.c_int, [_vp, C.c_int64, _vp, C.POINTER(C.c_int64), _vp, C.c_int32]),
    "nq_stream_upload": (C.c_int, [_vp, C.c_int64, _i, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_int64), _vp,
                                   C.POINTER(C.c_int64), _vp, C.c_int32]),
    "nq_stream_cancel": (C.c_int, [_vp, C.c_int64]),
    "nq_stream_poll": (C.c_int, [_vp, _vp, _i]),
    "nq_stream_tier_load": (C.c_int64, [_vp, C.POINTER(C.c_int64), C.c_int64]),
    "nq_stream_tier_drop": (C.c_int, [_vp]),
    "nq_stream_set_fault": (C.c_int, [_vp, C.c_double, C.c_int64]),
    "nq_stream_stats": (C.c_int, [_vp, _vp]),
    "nq_stream_close": (None, [_vp]),
}


def lib():
    """the loaded library; raises RuntimeError when it has not been built"""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -m nestquant_amd.build` (there is no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(rc):
    """raise the library's last error as RuntimeError (the reference raises RuntimeError from TORCH_CHECK)"""
    if rc:
        raise RuntimeError(lib().nq_last_error().decode())


def stream_ptr():
    """raw hipStream_t of torch's current stream"""
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
