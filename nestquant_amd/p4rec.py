"""Record of one expert's level-4 planes: the bytes a promoted slot holds (format nq-p4rec-v1).

Host-side mirror of the reference's streaming/p4rec.py (`layout` :13, `pack` :24, `row` :31): same names, argument
meaning and byte layout, so a record file written by the reference's repacker fills the slots of this build unchanged.

A record is five segments in the order SEGS, each starting on a SEG_ALIGN boundary; the last one holds the level-4
factors of the low-rank plane, U4_g | U4_u [r, I] | U4_d [r, H] in fp16, sized for rank RMAX whatever the expert's rank.
Every record of a layer has the same size, a multiple of ALIGN, so record i of a layer sits at layer_off + i * rec_bytes
and one aligned read fills a slot. The level-2 planes (base, variant bits, sign vectors, V and U2 of the low-rank plane)
are not part of the record: they stay resident (resident.py).

Besides the reference's three functions there are `seg_bytes` (segment sizes from the residual codes alone, so a slot
pool can be sized before any expert is loaded) and `pack_into` (writes the record into a caller's uint8 tensor, e.g. a
pinned staging buffer or a slot in device memory, without an intermediate bytes object).
"""
import torch

from .format import proj_sizes

SEG_ALIGN = 256
ALIGN = 4096
RMAX = 4
SEGS = ("gu.p4", "gu.d4", "dn.p4", "dn.d4", "lr4")


def _round_up(n, a):
    return -(-n // a) * a


def seg_bytes(H, I, rk_gu=0, rk_dn=0):
    """bytes of each segment for residual codes rk_gu / rk_dn (dense residual planes)"""
    gu, dn = proj_sizes(2 * I, H, None, rk_gu), proj_sizes(H, I, None, rk_dn)
    return {"gu.p4": gu["p4"], "gu.d4": gu["d4"], "dn.p4": dn["p4"], "dn.d4": dn["d4"], "lr4": RMAX * (2 * I + H) * 2}


def layout_of(nbytes):
    """{segment: bytes} -> dict(seg={segment: (offset, bytes)}, rec_bytes=record size)"""
    seg, end = {}, 0
    for name in SEGS:
        seg[name] = (end, nbytes[name])
        end = _round_up(end + nbytes[name], SEG_ALIGN)
    return dict(seg=seg, rec_bytes=_round_up(end, ALIGN))


def _segments(ex):
    lr4 = getattr(ex, "lr4", None)
    return (("gu.p4", ex.gu.p4), ("gu.d4", ex.gu.d4), ("dn.p4", ex.dn.p4), ("dn.d4", ex.dn.d4),
            ("lr4", lr4 if lr4 is not None else torch.zeros(0, dtype=torch.float16)))


def layout(ex, H, I):
    """layout of a layer from any expert of it (the residual codes fix the plane sizes, the same for the whole layer)"""
    nbytes = {name: t.numel() * t.element_size() for name, t in _segments(ex)}
    nbytes["lr4"] = RMAX * (2 * I + H) * 2
    return layout_of(nbytes)


def pack_into(ex, lay, buf):
    """write the record of `ex` into `buf` (uint8 tensor of at least rec_bytes elements, any device); the gaps between
    segments and the tail are zeroed"""
    if buf.dtype != torch.uint8 or buf.dim() != 1 or buf.numel() < lay["rec_bytes"]:
        raise ValueError("pack_into needs a flat uint8 tensor of at least rec_bytes elements")
    rec = buf[: lay["rec_bytes"]]
    rec.zero_()
    for name, t in _segments(ex):
        off, room = lay["seg"][name]
        raw = t.contiguous().view(torch.uint8).reshape(-1)
        if raw.numel() > room:
            raise ValueError(f"segment {name}: {raw.numel()} bytes do not fit the layout's {room}")
        rec[off:off + raw.numel()].copy_(raw)
    return rec


def pack(ex, lay):
    """record of one expert as a bytes object"""
    return pack_into(ex, lay, torch.empty(lay["rec_bytes"], dtype=torch.uint8)).numpy().tobytes()


def row(ex, lay, slot_ptr, entry):
    """level-4 table row of `ex` with the residual planes, their block words and the U4 factors read from the slot at
    device address `slot_ptr`, which holds the expert's record. `entry` is moe.entry. The resident planes stay where they
    are; an expert that carries per-level sign vectors (`ex.sc`) gets the level-4 one."""
    r = entry(ex, 4)
    at = lambda name: slot_ptr + lay["seg"][name][0]
    r[2], r[3], r[6], r[7] = at("gu.p4"), at("gu.d4"), at("dn.p4"), at("dn.d4")
    if ex.rg + ex.rd:
        r[15] = at("lr4")
    if hasattr(ex, "sc"):
        r[9] = ex.sc[4].data_ptr()
    return r
