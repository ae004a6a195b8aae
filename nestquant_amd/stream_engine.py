"""The record upgrade engine (csrc/nq_stream.hip) behind the reference's Python surface, and one rank's record file.

Mirror of streaming/stream_engine.py (`RankFile`, `mod().Engine`) and of the class the reference's streaming/nqstream.cu
binds (:8-26,280-292): same constructor arguments, method names, tuple / dict results, so the reference's executor and
smoke scripts read the same against either. The engine is native code in libnq_moe_hip.so, reached through its C ABI;
there is no Python fallback.

    e = Engine(path, rec_bytes, n_host, qd, device, alt_path="", qd_alt=0)
    e.upgrade(tag, rec_index, slot_ptr, stage_ptr, row, seq_ptr, seq)     # queued; returns at once
    e.post(tag, stage_ptr, row, seq_ptr, seq)                             # row-only op (a downgrade)
    e.poll() -> [(tag, hit, t_read_s, t_e2e_s)]     ops whose device writes are complete
    e.cancel(tag) / e.tier_load(recs) / e.tier_drop() / e.stats() / e.close()
    e.set_fault(read_ms, fail_ppm)                  # what the reference reads from NQ_FAULT_READ_MS / NQ_FAULT_FAIL_PPM
    e.upload(tag, [(host_ptr, dev_ptr, bytes)], stage_ptr, row, seq_ptr, seq)     # from the caller's pinned memory (no file)
"""
import ctypes as C
import json

import torch

from . import _lib
from .format import TBL_W


class NqStreamDone(C.Structure):
    """mirror of struct NqStreamDone in include/nq_moe_hip.h"""
    _fields_ = [("tag", C.c_int64), ("hit", C.c_int32), ("cancelled", C.c_int32), ("t_read", C.c_double), ("t_e2e", C.c_double)]


class NqStreamStats(C.Structure):
    """mirror of struct NqStreamStats in include/nq_moe_hip.h"""
    _fields_ = ([(k, C.c_int64) for k in ("upgrades", "posts", "host_hits", "bytes_read", "fault_injected", "queued", "reading", "copying",
                                          "drives", "n_host")]
                + [(k, C.c_int64 * 2) for k in ("drive_qd", "drive_inflight", "drive_reads", "drive_bytes", "drive_direct")]
                + [("drive_read_s", C.c_double * 2)]
                + [(k, C.c_int64) for k in ("tier_state", "tier_recs", "tier_hits", "tier_bytes", "cancelled", "waiting", "failed")]
                + [("now", C.c_double), ("uploads", C.c_int64), ("upload_bytes", C.c_int64)])


_POLL_MAX = 256


def _row_array(row):
    """int64[TBL_W] ctypes copy of a table row given as a CPU int64 tensor, a numpy array or a sequence"""
    if isinstance(row, torch.Tensor):
        if row.device.type != "cpu" or row.dtype != torch.int64 or row.numel() != TBL_W:
            raise RuntimeError("row: int64 cpu [20]")
        row = row.contiguous().view(-1).tolist()
    else:
        row = [int(v) for v in row]
        if len(row) != TBL_W:
            raise RuntimeError("row: int64 cpu [20]")
    return (C.c_int64 * TBL_W)(*row)


class Engine:
    def __init__(s, path, rec_bytes, n_host, qd, device, alt_path="", qd_alt=0):
        """path "" (or None): an engine without a record file, for upload() and post() only"""
        s.M = _lib.lib()
        s.h = s.M.nq_stream_open(str(path or "").encode(), (alt_path or "").encode(), int(rec_bytes), int(n_host), int(qd), int(qd_alt), int(device))
        if not s.h:
            raise RuntimeError(s.M.nq_last_error().decode())
        s._buf = (NqStreamDone * _POLL_MAX)()

    def _handle(s):
        if not s.h:
            raise RuntimeError("nqstream: engine is closed")
        return s.h

    def upgrade(s, tag, rec, slot, stage, row, seqp, seq):
        _lib.check(s.M.nq_stream_upgrade(s._handle(), int(tag), int(rec), int(slot), int(stage), _row_array(row), int(seqp), int(seq)))

    def post(s, tag, stage, row, seqp, seq):
        _lib.check(s.M.nq_stream_post(s._handle(), int(tag), int(stage), _row_array(row), int(seqp), int(seq)))

    def upload(s, tag, spans, stage, row, seqp, seq):
        """spans: [(pinned host address, device address, bytes)], copied in order before the row and seq; the host memory
        must stay valid until poll() reports the tag"""
        n = len(spans)
        src = (C.c_void_p * n)(*[int(a) for a, _, _ in spans])
        dst = (C.c_void_p * n)(*[int(b) for _, b, _ in spans])
        nb = (C.c_int64 * n)(*[int(c) for _, _, c in spans])
        _lib.check(s.M.nq_stream_upload(s._handle(), int(tag), n, src, dst, nb, int(stage), _row_array(row), int(seqp), int(seq)))

    def cancel(s, tag):
        _lib.check(s.M.nq_stream_cancel(s._handle(), int(tag)))

    def poll(s):
        out = []
        while True:
            n = s.M.nq_stream_poll(s._handle(), s._buf, _POLL_MAX)
            out += [(d.tag, bool(d.hit), d.t_read, d.t_e2e) for d in s._buf[:n]]
            if n < _POLL_MAX:
                return out

    def tier_load(s, recs):
        recs = [int(r) for r in recs]
        n = s.M.nq_stream_tier_load(s._handle(), (C.c_int64 * max(len(recs), 1))(*recs), len(recs))
        if n < 0:
            raise RuntimeError(s.M.nq_last_error().decode())
        return n

    def tier_drop(s):
        _lib.check(s.M.nq_stream_tier_drop(s._handle()))

    def set_fault(s, read_ms=0.0, fail_ppm=0):
        _lib.check(s.M.nq_stream_set_fault(s._handle(), float(read_ms), int(fail_ppm)))

    def stats(s):
        st = NqStreamStats()
        _lib.check(s.M.nq_stream_stats(s._handle(), C.byref(st)))
        if st.failed:
            raise RuntimeError(s.M.nq_last_error().decode())
        nd = st.drives
        d = {k: getattr(st, k) for k in ("upgrades", "posts", "host_hits", "bytes_read", "fault_injected", "queued", "reading", "copying",
                                         "drives", "n_host", "tier_state", "tier_recs", "tier_hits", "tier_bytes", "cancelled", "waiting", "now",
                                         "uploads", "upload_bytes")}
        for k in ("drive_qd", "drive_inflight", "drive_reads", "drive_bytes", "drive_read_s", "drive_direct"):
            d[k] = list(getattr(st, k))[:nd]
        return d

    def close(s):
        if s.h:
            h, s.h = s.h, None
            s.M.nq_stream_close(h)

    def __del__(s):
        try:
            s.close()
        except Exception:
            pass


class _Mod:
    """what the reference's `stream_engine.mod()` returns: a module object with the class Engine"""
    Engine = Engine


def mod():
    _lib.lib()
    return _Mod


class RankFile:
    """record file of one rank (repack.py). rec(L, E) -> record index; engine(...) -> Engine on it.
    Reference: streaming/stream_engine.py:17-25."""

    def __init__(s, repack_dir, rank):
        s.path = f"{repack_dir}/rank{rank}.bin"
        with open(f"{repack_dir}/rank{rank}.json") as f:
            s.idx = json.load(f)
        s.rb = s.idx["rec_bytes"]
        s.lay = dict(seg=s.idx["seg"], rec_bytes=s.rb)

    def rec(s, L, E):
        return (L - s.idx["L0"]) * s.idx["NE"] + E

    def engine(s, n_host=64, qd=8, device=None, alt_path="", qd_alt=0):
        """alt_path: an identical copy of this record file on a second drive ('' = one drive)"""
        return Engine(s.path, s.rb, n_host, qd, torch.cuda.current_device() if device is None else device, alt_path, qd_alt)
