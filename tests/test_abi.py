"""The C-ABI library loads without a GPU and exports every symbol include/nq_moe_hip.h declares; host-only entry
points (validation, code masks, error text) behave as documented. No compute call is made here."""
import ctypes as C
import os
import re

import pytest
import torch

from nestquant_amd import _lib
from nestquant_amd.format import TBL_W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nq_moe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nq_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m nestquant_amd.build`"


def test_every_declared_symbol_is_exported_and_bound():
    L = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 6
    for n in names:
        assert hasattr(L, n), n
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert L.nq_abi_version() == 3


def _row(**kw):
    r = torch.zeros(TBL_W, dtype=torch.int64)
    r[0] = 2; r[1] = r[5] = r[9] = 0x1000
    for k, v in kw.items():
        r[int(k[1:])] = v
    return r


def _validate(r, H=256, I=256):
    return _lib.lib().nq_validate_row(C.cast(r.data_ptr(), C.POINTER(C.c_int64)), H, I)


def test_validate_row_accepts_supported_rows():
    assert _validate(_row()) == 0
    assert _validate(_row(f0=0, f1=0, f5=0, f9=0)) == 0                                   # level 0: nothing else looked at
    assert _validate(_row(f0=4, f2=8, f3=8, f6=8, f7=8, f10=7, f11=3)) == 0
    assert _validate(_row(f0=3, f2=8, f3=8, f6=8, f7=8, f10=10, f11=10)) == 0
    assert _validate(_row(f0=4, f2=8, f3=8, f6=8, f7=8, f10=11, f11=11, f12=8, f18=128)) == 0
    assert _validate(_row(f0=4, f2=8, f3=8, f6=8, f7=8, f10=12, f11=12)) == 0            # P3 and P4 interleaved
    assert _validate(_row(f19=1)) == 0 and _validate(_row(f19=0x101)) == 0 and _validate(_row(f19=0x100)) == 0   # K = 1.75 base


@pytest.mark.parametrize("bad,word", [
    (dict(f0=1), "level"), (dict(f0=5), "level"), (dict(f0=3, f2=8, f3=8, f6=8, f7=8, f10=10, f11=10, f4=8), "mask mode"), (dict(f0=4, f2=8, f3=8, f6=8, f7=8, f10=11, f11=11, f8=8), "mask mode"),
    (dict(f14=8), "low-rank"), (dict(f16=2), "low-rank"), (dict(f18=512), "in_had_down"), (dict(f19=2), "base code"), (dict(f19=0x10001), "base code"),
    (dict(f0=4), "residual planes"), (dict(f0=4, f2=8, f3=8, f6=8, f7=8, f10=13), "out of range"),
    (dict(f0=3, f2=8, f3=8, f6=8, f7=8, f10=0, f11=10), "level 3"), (dict(f0=4, f2=8, f3=8, f6=8, f7=8, f10=10), "level 4"),
    (dict(f1=0), "null base"),
])
def test_validate_row_rejects_unimplemented_fields(bad, word):
    """a field the kernels do not implement is an error, never silently ignored"""
    assert _validate(_row(**bad)) != 0
    assert word in _lib.lib().nq_last_error().decode()


def test_shape_errors_and_code_masks():
    assert _validate(_row(), H=200) != 0 and "multiples of 128" in _lib.lib().nq_last_error().decode()
    out = (C.c_uint32 * 4)()
    assert _lib.lib().nq_codes(out) == 0
    assert out[0] == out[1] == 0x1FFF and out[2] == out[3] == 3
    with pytest.raises(RuntimeError, match="multiples of 128"):
        _lib.check(_validate(_row(), I=100))


def test_argument_checks_run_before_any_device_work():
    """bad arguments are refused on the host, with a message, before anything is launched (so this runs without a GPU)"""
    L = _lib.lib()
    err = lambda: L.nq_last_error().decode()
    buf = (C.c_char * 4096)()
    base = C.addressof(buf)
    base += (-base) % 64                                           # a 64-byte aligned address inside the buffer
    a = _lib.NqMoeArgs()
    for f in ("x", "sel", "rw", "table", "out", "acc_gu", "h", "acc_d", "cnt_gu", "cnt_d", "cnt_h", "zd"):
        setattr(a, f, base)
    a.B, a.topk, a.E, a.H, a.I = 1, 8, 256, 6144, 2048
    a.cfg_gu = (C.c_int32 * 4)(1, 4, 12, 0); a.cfg_dn = (C.c_int32 * 4)(1, 4, 4, 0)
    a.which = 3
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "workspace too small" in err()
    a.x = base + 2
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "16-byte aligned" in err()
    a.x = base; a.B = 9
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "B=9" in err()
    a.B = 1; a.cfg_gu = (C.c_int32 * 4)(1, 3, 12, 0)
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "bad cfg" in err()
    a.cfg_gu = (C.c_int32 * 4)(1, 4, 12, 0); a.G = 3
    a.route_ws = base
    a.acc_gu_elems = a.acc_d_elems = a.h_elems = a.out_elems = a.cnt_gu_elems = a.cnt_d_elems = a.cnt_h_elems = a.zd_elems = 1 << 40
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "route_ws" in err()
    a.route_ws_bytes = _lib.ROUTE_WS_BYTES
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "xrot" in err()
    a.xrot, a.xrot_elems = base, 1 << 40
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "G=3" in err()
    a.G = 4; a.mb_table = base
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "mailbox needs" in err()
    a.mb_table = None; a.G = 3
    a.G = 0; a.common_rows = 2
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "common_rows" in err()
    a.common_rows = 0; a.hoist_value_map = 2
    assert L.nq_moe_forward(C.byref(a), None) != 0 and "hoist_value_map" in err()
    a.hoist_value_map = 0
    assert L.nq_pf_plan(base, 256, 0, 1024, base, 256, None, 0, 0, None) != 0 and "cap" in err()
    assert L.nq_pf_plan(base, 256, 0, 1024, base + 4, 512, None, 0, 0, None) != 0 and "aligned" in err()
    assert L.nq_pf_gemm(base, base, 1, 48, 0, base, base, base, 4, 256, 256, None, None) != 0 and "tile height" in err()
    assert L.nq_pf_gemm(base, base, 1, 16, 0, base + 8, base, base, 4, 256, 256, None, None) != 0 and "aligned" in err()
    assert L.nq_pf_plan(base, 256, 0, 1024, base, 512, base, 0, 4, None) != 0 and "hot_min" in err()
    assert L.nq_pf_wdecode(base, base, 4, 0, base, 100, 2, 256, 256, None) != 0 and "scratch" in err()
    assert L.nq_pf_pre(base + 2, base, base, 1, base, base, base, None, 4, 256, 256, None) != 0 and "aligned" in err()
    assert L.nq_pf_pre_rows(base, base, base, 1, base, base, base, None, 4, 256, 256, base, 3, 1, None) != 0 and "cap" in err()
    assert L.nq_pf_pre_rows(base, base, base, 1, base, base, base, None, 4, 256, 256, base, 4, 32, None) != 0 and "heights" in err()
    assert L.nq_pf_pre_rows(base, base, base, 1, base, base, base, None, 4, 256, 256, base, 4, 0, None) == 0          # no height: nothing to do
    assert L.nq_pf_mid_rows(base, base, 1, base, base, None, None, 4, 256, 256, None, 4, 1, None) != 0 and "null" in err()
    assert L.nq_pf_mid_rows(base, base, 1, base, base, None, None, 4, 256, 256, base + 8, 4, 1, None) != 0 and "aligned" in err()
    assert L.nq_sal(base, 0, 64, base, 0, base, 0, 9, 64, 8, 16, 1.0, base, base, None) != 0 and "at most 8" in err()
    assert L.nq_dequant(base, 2, 0, 256, 256, base, None) != 0 and "proj" in err()
    assert L.nq_mailbox(None, base, base, base, None, 4, None) != 0 and "null" in err()


def test_stream_engine_refuses_bad_arguments_before_touching_the_gpu(tmp_path):
    """the checks of the reference's Engine constructor (streaming/nqstream.cu:76,77,81): record size a multiple of 4 KiB,
    at least as many host entries as reads in flight, the record file must exist"""
    from nestquant_amd.stream_engine import Engine
    f = tmp_path / "r.bin"
    f.write_bytes(b"\0" * 8192)
    with pytest.raises(RuntimeError, match="4096"):
        Engine(str(f), 4095, 8, 2, 0)
    with pytest.raises(RuntimeError, match="n_host"):
        Engine(str(f), 4096, 3, 4, 0)
    with pytest.raises(RuntimeError, match="n_host"):
        Engine(str(f), 4096, 4, 3, 0, alt_path=str(f), qd_alt=2)
    with pytest.raises(RuntimeError, match="open .*missing.bin"):
        Engine(str(tmp_path / "missing.bin"), 4096, 4, 2, 0)
