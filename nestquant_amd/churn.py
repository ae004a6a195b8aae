"""Refinement-plane promotion / demotion into resident slots on a side stream, racing the MoE layer.

The part of the reference's streaming runtime that touches the hot path (streaming/executor.py:71-119 `apply` / `poll`,
streaming/nqstream.cu:183-191 `issue_copies`, sm120/levelswitch_mbox.py:33-65): for an upgrade, copy the expert's
refinement planes from pinned host memory into a free device slot with asynchronous copies (hipMemcpyAsync under
torch's non_blocking copy_), then the new table row into `stage[e]`, then bump `seq[e]` -- all on ONE side stream, in
that order; for a downgrade, post only the row. The compute stream never waits: the mailbox (`Mailbox.apply()` at the start of
each layer call, or the layer call's own `mailbox=`) flips the rows whose `seq` changed. SSD / io_uring / LRU tiers of the reference engine are out of scope:
the host store here is plain pinned RAM.

Slot image of a nested expert (bytes, every part 256-byte aligned):
    [gu.P3 | gu.P4 | dn.P3 | dn.P4 | gu.d3 | dn.d3 | gu.d4 | dn.d4]
P4's sub-array directly follows P3's in each projection (what residual code 11 reads), so 2 -> 3 uploads the P3 parts and
d3, 3 -> 4 uploads the P4 parts and d4, and 2 -> 4 uploads the whole image in one copy.

Protocol invariants (checked by `check_invariants`, after the reference's sm120/serve/nq_slotcheck.py:11-21):
  (B) slot bytes == the host image for every resident expert that is not in transit (for the parts its level uses)
  (T) table[e] == the row built for (level, slot) of e        (O) a level 3/4 row points into a slot its expert owns
  (K) slot_of is injective and no owned slot is in the free list
One outstanding op per expert; a slot is reused only after the level-2 row that released it was applied.
"""
import torch

from .format import CODE_L3, CODE_L4N
from .moe import entry, validate_row

ALIGN = 256


def _al(n):
    return (n + ALIGN - 1) // ALIGN * ALIGN


class SlotLayout:
    """byte offsets of the slot image for projections gate|up [2I, H] and down [H, I]"""

    def __init__(s, H, I):
        rg, rd = (2 * I // 16) * (H // 128) * 32, (H // 16) * (I // 128) * 32
        ug, ud = rg // 32, rd // 32
        s.parts, o = {}, 0
        for name, n in (("gu.p3", rg * 8), ("gu.p4", rg * 8), ("dn.p3", rd * 8), ("dn.p4", rd * 8),
                        ("gu.d3", ug * 4), ("dn.d3", ud * 4), ("gu.d4", ug * 4), ("dn.d4", ud * 4)):
            s.parts[name] = (o, n)
            o += _al(n) if name.endswith(("p4", "d3", "d4")) else n      # P4 must follow P3 without a gap
        s.bytes = _al(o)
        assert s.parts["gu.p4"][0] == s.parts["gu.p3"][0] + s.parts["gu.p3"][1]
        assert s.parts["dn.p4"][0] == s.parts["dn.p3"][0] + s.parts["dn.p3"][1]

    def image(s, ex):
        """pinned host image of a nested expert's refinement planes"""
        img = torch.zeros(s.bytes, dtype=torch.uint8).pin_memory()
        src = {"gu.p3": ex.gu.slot[: ex.gu.slot.numel() // 2], "gu.p4": ex.gu.slot[ex.gu.slot.numel() // 2:],
               "dn.p3": ex.dn.slot[: ex.dn.slot.numel() // 2], "dn.p4": ex.dn.slot[ex.dn.slot.numel() // 2:],
               "gu.d3": ex.gu.d3, "dn.d3": ex.dn.d3, "gu.d4": ex.gu.d4n, "dn.d4": ex.dn.d4n}
        for name, t in src.items():
            o, n = s.parts[name]
            img[o:o + n] = t.contiguous().view(torch.uint8).cpu()
        return img

    def spans(s, frm, to):
        """byte ranges (offset, length) to upload for a promotion frm -> to; adjacent parts are merged"""
        need = []
        if frm < 3 <= to:
            need += ["gu.p3", "dn.p3", "gu.d3", "dn.d3"]
        if to == 4:
            need += ["gu.p4", "dn.p4", "gu.d4", "dn.d4"]
        if frm == 2 and to == 4:
            return [(0, s.bytes)]
        return [s.parts[n] for n in need]


class ChurnExecutor:
    """Level ops of one layer: `promote(e, level)`, `demote(e, level)`, `poll()`.

    layer / mailbox: nestquant_amd.moe.MoELayer / Mailbox; experts: {e: nested Expert whose base planes and sign vector
    are resident on the device}; nslots device slots are allocated here. Every expert starts at level 2."""

    def __init__(s, layer, mailbox, experts, nslots, side_stream=None, native=False):
        """native=True: copies, rows and sequence numbers are issued by the upgrade engine (stream_engine.Engine without a
        record file: its own thread and side stream, `upload` from the pinned images) instead of torch copies on
        `side_stream`; the books and the protocol are the same"""
        s.L, s.MB, s.ex = layer, mailbox, experts
        dev = layer.table.device
        s.eng, s.tag, s.lat = None, 0, []
        if native:
            from .stream_engine import Engine
            s.eng = Engine("", 0, 0, 8, dev.index if dev.index is not None else torch.cuda.current_device())
        s.lay = SlotLayout(layer.H, layer.I)
        s.slots = torch.zeros(nslots, s.lay.bytes, dtype=torch.uint8, device=dev)
        s.host = {e: s.lay.image(x) for e, x in experts.items()}
        s.base_row = {e: entry(x, 2) for e, x in experts.items()}
        s.free = list(range(nslots))[::-1]
        s.slot_of, s.level, s.pend = {}, {e: 2 for e in experts}, {}       # pend[e] = (target level, slot to release or None)
        s.side = side_stream or torch.cuda.Stream(device=dev)
        s.bytes_copied, s.n_ops, s.n_refused = 0, 0, 0

    def row(s, e, level, slot=None):
        """table row of expert e at `level`; levels 3 / 4 point into `slot`"""
        r = s.base_row[e].clone()
        r[0] = level
        sc = getattr(s.ex[e], "sc", None)                          # served experts carry one sign / scale vector per level
        if sc is not None:
            r[9] = sc[level].data_ptr()
        if level >= 3:
            b = s.slots[slot].data_ptr()
            p = s.lay.parts
            r[2], r[6] = b + p["gu.p3"][0], b + p["dn.p3"][0]
            d = "d3" if level == 3 else "d4"
            r[3], r[7] = b + p["gu." + d][0], b + p["dn." + d][0]
            r[10] = r[11] = CODE_L3 if level == 3 else int(getattr(s.ex[e], "l4code", CODE_L4N))
        return r

    def idle(s, e):
        return e not in s.pend and s.MB.done(e)

    def promote(s, e, level):
        """2 -> 3, 2 -> 4 or 3 -> 4. Returns False (and does nothing) when no slot is free or an op is outstanding."""
        cur = s.level[e]
        assert level in (3, 4) and level > cur
        if not s.idle(e) or (cur == 2 and not s.free):
            s.n_refused += 1
            return False
        slot = s.slot_of[e] if cur >= 3 else s.free.pop()
        s.slot_of[e] = slot
        spans = s.lay.spans(cur, level)
        s.bytes_copied += sum(n for _, n in spans)
        if s.eng is not None:
            s._issue(e, s.row(e, level, slot), [(s.host[e].data_ptr() + o, s.slots[slot].data_ptr() + o, n) for o, n in spans])
        else:
            with torch.cuda.stream(s.side):
                for o, n in spans:
                    s.slots[slot, o:o + n].copy_(s.host[e][o:o + n], non_blocking=True)
            s.MB.post(e, s.row(e, level, slot), s.side)           # row, then seq, after the copies, same stream
        s.pend[e] = (level, None)
        s.n_ops += 1
        return True

    def demote(s, e, level=2):
        """4 -> 3, 4 -> 2 or 3 -> 2: row only. The slot of an expert going to level 2 is released when the row is applied."""
        cur = s.level[e]
        assert level in (2, 3) and level < cur
        if not s.idle(e):
            s.n_refused += 1
            return False
        slot = s.slot_of[e]
        row = s.row(e, level, slot if level == 3 else None)
        if s.eng is not None:
            s._issue(e, row, None)
        else:
            s.MB.post(e, row, s.side)
        s.pend[e] = (level, slot if level == 2 else None)
        s.n_ops += 1
        return True

    def _issue(s, e, row, spans):
        """one op through the engine: what Mailbox.post does on the host (row check, sequence number), then upload / post"""
        assert s.MB.done(e), "one outstanding op per expert"
        validate_row(row, s.L.H, s.L.I)
        s.L.rare_rows |= bool(row[4] or row[8] or row[19])
        s.MB.hseq[e] += 1
        s.tag += 1
        stage, seq = s.MB.stage.data_ptr() + s.MB.stage.stride(0) * 8 * e, s.MB.seq.data_ptr() + 4 * e
        if spans:
            s.eng.upload(s.tag, spans, stage, row, seq, s.MB.hseq[e])
        else:
            s.eng.post(s.tag, stage, row, seq, s.MB.hseq[e])

    def close(s):
        if s.eng is not None:
            s.eng.close()
            s.eng = None

    def poll(s):
        """after a layer call finished: ops the mailbox applied take effect on the host books; returns the experts landed"""
        if s.eng is not None:
            s.lat += [t for _, _, _, t in s.eng.poll()]
        landed = []
        for e in list(s.pend):
            if s.MB.done(e):
                level, release = s.pend.pop(e)
                s.level[e] = level
                if release is not None:
                    del s.slot_of[e]
                    s.free.append(release)
                landed.append(e)
        return landed

    def check_invariants(s):
        """(B)(T)(O)(K) on the current device state; synchronises. Raises AssertionError with the violated invariant."""
        torch.cuda.synchronize()
        owned = list(s.slot_of.values())
        assert len(set(owned)) == len(owned), "K: two experts own one slot"
        assert not set(owned) & set(s.free), "K: an owned slot is in the free list"
        table = s.L.table.cpu()
        lo, hi = s.slots.data_ptr(), s.slots.data_ptr() + s.slots.numel()
        for e in s.ex:
            if e in s.pend:
                continue                                          # in transit: row and bytes may be either state
            lv, slot = s.level[e], s.slot_of.get(e)
            assert torch.equal(table[e], s.row(e, lv, slot)), f"T: table row of expert {e} (level {lv}, slot {slot})"
            if lv >= 3:
                for f in (2, 3, 6, 7):
                    a = int(table[e, f])
                    assert lo <= a < hi and (a - lo) // s.lay.bytes == slot, f"O: row field {f} of expert {e} leaves its slot"
                for o, n in s.lay.spans(2, lv):
                    assert torch.equal(s.slots[slot, o:o + n].cpu(), s.host[e][o:o + n]), f"B: slot bytes of expert {e}"
            else:
                assert slot is None, f"K: level-2 expert {e} still owns slot {slot}"
