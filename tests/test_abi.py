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
    assert L.nq_abi_version() == 1


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
    assert _validate(_row(f19=1)) == 0 and _validate(_row(f19=0x101)) == 0 and _validate(_row(f19=0x100)) == 0   # K = 1.75 base


@pytest.mark.parametrize("bad,word", [
    (dict(f0=1), "level"), (dict(f0=5), "level"), (dict(f0=3, f2=8, f3=8, f6=8, f7=8, f10=10, f11=10, f4=8), "mask mode"), (dict(f0=4, f2=8, f3=8, f6=8, f7=8, f10=11, f11=11, f8=8), "mask mode"),
    (dict(f14=8), "low-rank"), (dict(f16=2), "low-rank"), (dict(f18=512), "in_had_down"), (dict(f19=2), "base code"), (dict(f19=0x10001), "base code"),
    (dict(f0=4), "residual planes"), (dict(f0=4, f2=8, f3=8, f6=8, f7=8, f10=12), "out of range"),
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
    assert out[0] == out[1] == 0xFFF and out[2] == out[3] == 3
    with pytest.raises(RuntimeError, match="multiples of 128"):
        _lib.check(_validate(_row(), I=100))
