"""NestQuant grouped MoE layer on MI355X: device table, workspaces, launch wrappers.

Host-side mirror of the reference's Python op surface (sm120/moe.py): `entry` :216-229, `MoELayer` :231-260,
`prefill` :282-326, `Mailbox` :329-342, `dense_W` :156-166, `H128` :168-172, `Expert.ref` :196-210, `moe_ref` :344-351. The kernels behind it are the HIP kernels of
libnq_moe_hip.so, reached through ctypes with raw device pointers; there is no CPU path in this module.
"""
import ctypes as C

import torch

from . import _lib
from .format import (CODE_L3, CODE_L4B, CODE_L4N, RK_OF, RKP, TBL_W, Expert, Proj, all_MbN, make_flags, pack_words, popc, proj_sizes,  # noqa: F401
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
    """table row int64[TBL_W] of expert `ex` at `level` (0, 2, 3, 4). Level 3 points at the one-bit plane p3 (code 10); level 4
    points, for experts built with nested=True, at the planes P3 and P4 read as one record (code 11: concatenated, or code 12
    for experts built with interleave=True: interleaved bit by bit), otherwise at the wide residual plane p4 (code rk)."""
    e = torch.zeros(TBL_W, dtype=torch.int64)
    e[0] = level
    nested = bool(getattr(ex, "nested", False))
    l3 = level == 3
    if l3 and not nested and any(getattr(p, "p3", None) is None for p in (ex.gu, ex.dn)):
        raise ValueError("level 3 needs an expert with the one-bit planes p3 / d3")
    for off, p in ((1, ex.gu), (5, ex.dn)):
        e[off] = p.base.data_ptr()
        if nested:
            slot = p.slot
            e[off + 1] = slot.data_ptr()
            e[off + 2] = (p.d3 if l3 else p.d4n).data_ptr()
        elif l3:
            e[off + 1] = p.p3.data_ptr()
            e[off + 2] = p.d3.data_ptr()
        else:
            e[off + 1] = 0 if p.p4 is None else p.p4.data_ptr()      # None: resident-only expert, a record slot supplies them
            e[off + 2] = 0 if p.d4 is None else p.d4.data_ptr()
        if getattr(p, "flags", None) is not None:
            e[off + 3] = p.flags.data_ptr()
    e[9] = ex.signs.data_ptr()
    if nested or l3:
        e[10] = e[11] = CODE_L3 if l3 else int(getattr(ex, "l4code", CODE_L4N))
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


def occ(mode, sb, shm, any_rows=False):
    """(resident workgroups per CU, registers per lane, spill bytes per lane) of the decode kernel `mode` (0 gate|up, 1 down)
    launched with sb wavefronts per workgroup and shm bytes of dynamic LDS; the reference's M.occ (sm120/nqmoe.cu:930-937)"""
    out = (C.c_int * 3)()
    _lib.check(_lib.lib().nq_occ(mode, int(any_rows), sb, shm, out))
    return tuple(out)


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


# caller element types the decode kernels read / write directly (codes of include/nq_moe_hip.h)
_DT_IN = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}
_DT_SEL = {torch.int64: 0, torch.int32: 1}
_DT_OUT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


class MoELayer:
    """Device table [E, TBL_W] + workspaces for up to Bmax tokens; table rows are flipped in place (graph-safe).

    Same constructor, attributes and call signature as the reference's MoELayer (sm120/moe.py:231-260). Differences that
    a caller can observe: acc_gu / acc_d hold per-k-slice partial sums ([NY, S, 2I] and [NY, S, H]) instead of
    atomically accumulated [S, 2I] / [S, H], so they are not zero between calls and outputs are bitwise repeatable;
    cnt_gu / cnt_d / cnt_h are arrival counters (zero on entry, zero on exit; cnt_h counts the 128-column groups of a
    512-column block when in_had_down = 512); zd carries the low-rank plane's z_d partial sums from the gate|up launch to
    the down launch and needs no zeroing; wq exists for attribute compatibility only (no work queue here) and stays zero."""

    def __init__(s, E, H, I, nm_gu=0, nm_dn=0, Bmax=4, topk=8, G=4, dev="cuda", mod=None):
        if G not in (4, 2):
            raise NotImplementedError("rings of G = 4 lanes (every artifact) or G = 2 (the reference's test variant) only")
        s.M = mod or _lib.lib()
        s.E, s.H, s.I, s.nm_gu, s.nm_dn, s.G, s.Bmax, s.topk = E, H, I, nm_gu, nm_dn, G, Bmax, topk
        s.table = torch.zeros(E, TBL_W, dtype=torch.int64, device=dev)
        S = Bmax * topk
        f32, i32 = torch.float32, torch.int32
        s.cfg_gu, s.cfg_dn = s.default_cfg(H, I)
        s._tuned = True                               # cfg_for may pick the tuned k-slice lengths; set_cfg switches that off
        s.h = torch.zeros(S, I, dtype=torch.float16, device=dev)
        s.cnt_gu = torch.zeros(S * (I // 128), dtype=i32, device=dev); s.cnt_d = torch.zeros(H // 128, dtype=i32, device=dev)
        s.wq = torch.zeros(4, dtype=i32, device=dev)
        s.zd = torch.zeros(S * (I // 128) * 4, dtype=f32, device=dev); s.cnt_h = torch.zeros(S * (I // 128), dtype=i32, device=dev)
        s.out = torch.zeros(Bmax, H, dtype=f32, device=dev)
        s.route = torch.zeros(_lib.ROUTE_WS_BYTES, dtype=torch.uint8, device=dev)    # the routing launch's result for the projection launches
        s.xrot = torch.zeros(S, 2, H, dtype=torch.float16, device=dev)               # and the rotated activations of every pick
        s.hits_ptr = 0
        s.rare_rows = False                           # set once a row in mask mode or with a base window code other than 0 is
                                                      # installed (set / Mailbox.post): the decode call then runs the kernel that
                                                      # carries their loops and prefill also launches its variant kernel. A caller
                                                      # that writes such rows into the table itself must set it, else the tokens
                                                      # that pick them come out NaN
        s._alloc_partials()

    # k-slice lengths (chunks) per token count 1..8 at the full shape H = 6144, I = 2048, top-8 over 256 experts, measured on
    # an MI355X with the routing of the layer benchmark; the reference keeps such tables for its GPUs
    # (sm120/serve/nq_vllm.py:32-33). Index = tokens of the call; other shapes use default_cfg for every count.
    TUNED_NST = {(6144, 2048): ([12, 12, 24, 24, 24, 24, 24, 24, 24], [4, 4, 4, 4, 4, 4, 4, 4, 4])}

    def cfg_for(s, T):
        """(cfg_gu, cfg_dn) for a decode call of T tokens: the layer's defaults, with the tuned k-slice length for T where this
        shape has a table and set_cfg has not replaced the defaults"""
        t = s.TUNED_NST.get((s.H, s.I)) if s._tuned else None
        if t is None or T >= len(t[0]):
            return s.cfg_gu, s.cfg_dn
        return [s.cfg_gu[0], s.cfg_gu[1], t[0][T]], [s.cfg_dn[0], s.cfg_dn[1], t[1][T]]

    @staticmethod
    def default_cfg(H, I):
        """[cpw, sb, nst]: k-slice of cpw * nst chunks, sb wavefronts per block"""
        def pick(C, N, want):
            nc = max(d for d in range(1, want + 1) if C % d == 0)
            sb = max(d for d in (4, 2, 1) if (N // 32) % d == 0 and (I // 32) % d == 0)
            return [1, sb, nc]
        return pick(H // 128, 2 * I, 12), pick(I // 128, H, 8)

    def _ny(s, cfg, C):
        return C // (cfg[0] * cfg[2])

    def _alloc_partials(s, cfg_gu=None, cfg_dn=None):
        """Partial-sum workspaces for the given (default: the layer's) tilings. At construction they are sized for the finest
        k-split among the layer's default and its tuned tilings, so the calls a serving loop makes never re-size them. A call
        that brings a finer split of its own replaces them -- graphs captured before hold the old addresses and must be
        captured again -- and that is refused while the stream is capturing (an allocation cannot be captured)."""
        S, dev = s.Bmax * s.topk, s.table.device
        ny_gu, ny_dn = s._ny(cfg_gu or s.cfg_gu, s.H // 128), s._ny(cfg_dn or s.cfg_dn, s.I // 128)
        first = getattr(s, "acc_gu", None) is None
        if first:
            t = s.TUNED_NST.get((s.H, s.I))
            if t is not None:
                ny_gu = max([ny_gu] + [(s.H // 128) // (s.cfg_gu[0] * n) for n in t[0]])
                ny_dn = max([ny_dn] + [(s.I // 128) // (s.cfg_dn[0] * n) for n in t[1]])
        grow_gu, grow_dn = first or s.acc_gu.shape[0] < ny_gu, first or s.acc_d.shape[0] < ny_dn
        if (grow_gu or grow_dn) and not first and torch.cuda.is_current_stream_capturing():
            raise RuntimeError("this call's k-split needs larger partial-sum workspaces than the layer holds; make one call with "
                               "these tilings (or set_cfg) before capturing")
        if grow_gu:
            s.acc_gu = torch.zeros(ny_gu, S, 2 * s.I, dtype=torch.float32, device=dev)
        if grow_dn:
            s.acc_d = torch.zeros(ny_dn, S, s.H, dtype=torch.float32, device=dev)

    def set_cfg(s, cfg_gu=None, cfg_dn=None):
        """change the default tilings (may replace the partial-sum workspaces: graphs captured before must be captured again)"""
        s.cfg_gu, s.cfg_dn = list(cfg_gu or s.cfg_gu), list(cfg_dn or s.cfg_dn)
        s._tuned = False
        s._alloc_partials()

    def set(s, e, ex, level):
        row = entry(ex, level)
        if s.G != 4 and (row[12] or row[13]):
            raise ValueError("sign-variant planes are defined for rings of G = 4 lanes only (reference sm120/moe.py:143)")
        validate_row(row, s.H, s.I)
        s.rare_rows |= bool(row[4] or row[8] or row[19])
        s.table[e].copy_(row.to(s.table.device), non_blocking=False)

    def __call__(s, x, sel, rw, out=None, force_level=0, which=3, cfg_gu=None, cfg_dn=None, table=None, static_ws=False, mailbox=None, hoist=False):
        """x [B, H], sel [B, topk], rw [B, topk] -> fp32 [B, H] (s.out[:B] unless `out` is given). As in the reference x
        and rw are fp16 and sel int64; the kernels also take x / rw in bf16 or fp32, sel in int32 and `out` in fp16 or
        bf16, with the roundings of x.half(), rw.half() and out.to(dtype) (the casts the reference's caller launches as
        separate kernels, sm120/serve/nq_vllm.py:522,560).
        table: optional [E, TBL_W] override. Everything is enqueued on torch's current stream; nothing syncs.
        mailbox: a Mailbox of this layer, served by the call without a launch of its own: the call's last projection launch
        applies it (table rows and the device copy of `applied`) after the call's routing has read the table, and the routing
        launch of the next call publishes `applied_host`. Rows that land while this call runs are used, and reported done, from
        the next call on -- when `mailbox.apply()` at the head of the next call would have done both. After the last call of
        a sequence one `mailbox.apply()` publishes what that call applied.
        hoist: experts without a sign plane (rows of the common kind) multiply the integers 1024 + S / 1024 + F and apply the value
        map to the sums, so no weight is rounded to fp16: ~4 % faster, ~5e-4 from the default's result (NqMoeArgs.hoist_value_map;
        off by default).
        static_ws: go through nq_moe_forward_static, which ignores this layer's workspaces and uses the library's built-in
        device scratch instead (for callers that must not allocate; calls on one GPU then share that scratch)."""
        assert x.dtype in _DT_IN and rw.dtype in _DT_IN and sel.dtype in _DT_SEL, (x.dtype, rw.dtype, sel.dtype)
        assert x.is_contiguous() and sel.is_contiguous() and rw.is_contiguous()
        B, topk = sel.shape
        out = s.out[:B] if out is None else out
        assert out.dtype in _DT_OUT and out.is_contiguous(), out.dtype
        tb = s.table if table is None else table
        tg, td = s.cfg_for(B)
        cg, cd = list(cfg_gu or tg), list(cfg_dn or td)
        if not static_ws:
            s._alloc_partials(cg, cd)                # grows only when a call brings a finer k-split than any before
        a = _lib.NqMoeArgs()
        a.x, a.sel, a.rw, a.table, a.out = x.data_ptr(), sel.data_ptr(), rw.data_ptr(), tb.data_ptr(), out.data_ptr()
        a.acc_gu, a.h, a.acc_d, a.hits = s.acc_gu.data_ptr(), s.h.data_ptr(), s.acc_d.data_ptr(), s.hits_ptr or None
        a.cnt_gu, a.cnt_d = s.cnt_gu.data_ptr(), s.cnt_d.data_ptr()
        a.acc_gu_elems, a.acc_d_elems, a.h_elems, a.out_elems = s.acc_gu.numel(), s.acc_d.numel(), s.h.numel(), out.numel()
        a.cnt_gu_elems, a.cnt_d_elems = s.cnt_gu.numel(), s.cnt_d.numel()
        a.B, a.topk, a.E, a.H, a.I = B, topk, tb.shape[0], x.shape[1], s.I
        a.cfg_gu = (C.c_int32 * 4)(*(cg + [0] * (4 - len(cg)))); a.cfg_dn = (C.c_int32 * 4)(*(cd + [0] * (4 - len(cd))))
        a.force_level, a.which = force_level, which
        a.cnt_h, a.cnt_h_elems = s.cnt_h.data_ptr(), s.cnt_h.numel()
        a.zd, a.zd_elems = s.zd.data_ptr(), s.zd.numel()
        a.G = s.G
        a.route_ws, a.route_ws_bytes = s.route.data_ptr(), s.route.numel()
        a.xrot, a.xrot_elems = s.xrot.data_ptr(), s.xrot.numel()
        if mailbox is not None:
            a.mb_table, a.mb_stage, a.mb_seq = tb.data_ptr(), mailbox.stage.data_ptr(), mailbox.seq.data_ptr()
            a.mb_applied, a.mb_applied_host = mailbox.applied.data_ptr(), mailbox.applied_host.data_ptr()
        a.common_rows = int(table is None and not s.rare_rows)     # a caller's own table: unknown
        a.hoist_value_map = int(bool(hoist))
        a.x_dtype, a.sel_dtype, a.rw_dtype, a.out_dtype = _DT_IN[x.dtype], _DT_SEL[sel.dtype], _DT_IN[rw.dtype], _DT_OUT[out.dtype]
        _lib.check((s.M.nq_moe_forward_static if static_ws else s.M.nq_moe_forward)(C.byref(a), _lib.stream_ptr()))
        return out


_PF = {}
PF_TILES = (16, 32, 64, 128, 256)            # token-tile heights the grouped GEMM is compiled for
# An expert with at least PF_HOT_MIN pair rows in a chunk (more than one 256-row tile) can be decoded once per call into a scratch
# of decoded weights (at most PF_HOT_SLOTS experts at 6 H I bytes each) instead of once per tile; see nq_pf_wdecode. Off by
# default (0 slots): a tile then reads 75 MB of fp16 operands from HBM where the decode-fused kernel reads 12.6 MB of codes, and
# on the 4096-token benchmark the call takes 6.59-6.65 ms with 32 slots against 6.58-6.61 ms without (the tiles save 0.4 ms, the
# decode launches cost 0.57 ms) plus 2.4 GB of scratch. Same bits either way.
PF_HOT_MIN, PF_HOT_SLOTS = 257, 0


def pf_bytes(H, I, R, G=0):
    """bytes of prefill scratch for R pair rows (G is accepted for signature compatibility: the decoded-weight scratch is sized
    by the rows, not by a group of experts)"""
    return R * (2 * H * 2 + 2 * I * 4 + I * 2 + H * 4 + 32) + max(0, min(PF_HOT_SLOTS, R // PF_HOT_MIN)) * 6 * H * I


def pf_scratch(dev, H, I, R, G=0):
    """Prefill scratch shared by every layer on `dev`, allocated on first use: xg | xu fp16 [R, H], acc_gu fp32 [R, 2I],
    h fp16 [R, I], y fp32 [R, H], and wop: decoded weights of up to PF_HOT_SLOTS hot experts. Unlike the reference
    (sm120/moe.py:263-274), which decodes every expert of a group into dense scratch, only experts with more than one tile go
    through scratch; the others are decoded in registers inside the grouped GEMM."""
    k = (str(dev), H, I, R, PF_HOT_SLOTS)
    if k not in _PF:
        f16, f32 = torch.float16, torch.float32
        slots = max(0, min(PF_HOT_SLOTS, R // PF_HOT_MIN))
        _PF[k] = dict(wop=torch.empty(slots, 3 * H * I, dtype=f16, device=dev) if slots else None,
                      xg=torch.empty(R, H, dtype=f16, device=dev), xu=torch.empty(R, H, dtype=f16, device=dev),
                      acc=torch.empty(R, 2 * I, dtype=f32, device=dev), h=torch.empty(R, I, dtype=f16, device=dev),
                      y=torch.empty(R, H, dtype=f32, device=dev),
                      zg=torch.zeros(R, 4, dtype=f32, device=dev), zd=torch.zeros(R, 4, dtype=f32, device=dev))
    return _PF[k]


def pf_tiles(segs):
    """segs [(expert, first row, rows)] -> {tile height: int32 [n, 4] rows (expert, row0, rows, 0)}. Rows of an expert are
    cut into 256-row tiles; the remainder takes the smallest compiled height that holds it."""
    out = {bm: [] for bm in PF_TILES}
    for e, r0, n in segs:
        while n > 0:
            take = min(n, PF_TILES[-1])
            bm = next(b for b in PF_TILES if b >= take)
            out[bm].append((e, r0, take, 0))
            r0 += take; n -= take
    return {bm: torch.tensor(v, dtype=torch.int32) for bm, v in out.items() if v}


_PF_SIDE = {}
_PF_STREAM_OF = {256: 0, 128: 1, 64: 2, 32: 3, 16: 3}          # stream 0 = the caller's


def _pf_chains(Lb, tb, lists, variants, S, x, pts, pes, n, tiles, cap, E, H, I, wop=None):
    """Everything between the tile plan and the post kernel of one row chunk: rotation of the activations, gate|up GEMM, SwiGLU
    kernel and down GEMM of every tile height. The heights work on disjoint pair rows, so each is a chain of its own. A GEMM
    launch ends with the GPU partly idle while its last workgroups drain (a workgroup runs the whole K loop, ~75 us, so a
    launch of a few dozen tiles is a handful of such rounds); the tallest height stays on the caller's stream and the others
    go to side streams (default priority) between two events, so that the chains overlap, fill each other's tails and the
    memory-bound kernels of one height run under the GEMMs of another."""
    main = torch.cuda.current_stream()
    side = _PF_SIDE.setdefault(str(tb.device), [])
    while len(side) < 3:
        side.append(torch.cuda.Stream(device=tb.device))
    streams = [main] + side
    ready = torch.cuda.Event(); ready.record(main)
    for st in side:
        st.wait_event(ready)
    xg, xu, acc, h, y, zg, zd = (S[k].data_ptr() for k in ("xg", "xu", "acc", "h", "y", "zg", "zd"))

    def gemms(mode, A0, A1, Cm):
        for bm, t, nt in lists:
            stp = C.c_void_p(streams[_PF_STREAM_OF[bm]].cuda_stream)
            for v in variants:
                _lib.check(Lb.nq_pf_gemm(tb.data_ptr(), t.data_ptr(), nt, bm, mode | v, A0, A1, Cm, E, H, I, wop, stp))

    masks = [sum(bm // 16 for bm, _, _ in lists if _PF_STREAM_OF[bm] == i) for i in range(len(streams))]    # bit k = height 16 << k
    for st, heights in zip(streams, masks):
        _lib.check(Lb.nq_pf_pre_rows(x.data_ptr(), pts.data_ptr(), pes.data_ptr(), n, tb.data_ptr(), xg, xu, zg, E, H, I,
                                     tiles.data_ptr(), cap, heights, C.c_void_p(st.cuda_stream)))
    gemms(0, xg, xu, acc)
    for st, heights in zip(streams, masks):
        _lib.check(Lb.nq_pf_mid_rows(acc, pes.data_ptr(), n, tb.data_ptr(), h, zg, zd, E, H, I, tiles.data_ptr(), cap, heights,
                                     C.c_void_p(st.cuda_stream)))
    gemms(1, h, None, y)
    for st in side:
        done = torch.cuda.Event(); done.record(st); main.wait_event(done)


def prefill(s, x, sel, rw, out=None, R=None, G=None, table=None):
    """T > Bmax tokens (reference sm120/moe.py:282-326): pairs sorted by expert, each routed expert decoded inside the
    grouped GEMMs at the level of its live table row, same math as the decode path (fp32 accumulation order differs).
    No host synchronisation (the reference's prefill reads the expert counts back; here the tile lists are built on the
    device by nq_pf_plan). Exports routing hits like the decode kernel. Calls on one device share the scratch of pf_scratch()
    (as the reference's do, sm120/moe.py:262-274) and the side streams of _pf_chains, so they must be ordered on one stream."""
    if s.G != 4:
        raise NotImplementedError("prefill decodes rings of G = 4 lanes only (as the reference's pf_decode)")
    assert x.dtype == torch.float16 and rw.dtype == torch.float16 and sel.dtype == torch.int64, (x.dtype, rw.dtype, sel.dtype)
    assert x.is_contiguous()
    T, k = sel.shape
    H, I, E, dev, Lb = s.H, s.I, s.E, x.device, s.M
    tb = s.table if table is None else table
    st = _lib.stream_ptr()
    out = torch.zeros(T, H, dtype=torch.float32, device=dev) if out is None else out.zero_()
    flat = sel.reshape(-1); rwf = rw.reshape(-1)
    order = torch.argsort(flat, stable=True)
    pe = flat[order].int(); pt = (order // k).int()
    pos = torch.empty_like(order, dtype=torch.int32)
    pos[order] = torch.arange(order.numel(), dtype=torch.int32, device=dev)       # row of pair (t, k) in sorted order
    selc, rwc = sel.contiguous(), rw.contiguous()
    one = torch.ones_like(flat, dtype=torch.int32)
    cnt = torch.zeros(E, dtype=torch.int32, device=dev).scatter_add_(0, flat, one)
    if s.hits_ptr:
        hc = torch.zeros(E + 1, dtype=torch.int32, device=dev).scatter_add_(0, torch.where(rwf != 0, flat, E), one)[:E].contiguous()
        _lib.check(Lb.nq_pf_hits(hc.data_ptr(), s.hits_ptr, E, st))
    P = T * k
    if P == 0:
        return out
    R = min(P, R or int(__import__("os").environ.get("NQ_PF_ROWS", "32768")))
    S = pf_scratch(dev, H, I, R)
    cap = E + R // 256 + 1
    # mask mode / other base codes run in their own kernel variant; a caller's own table may hold such rows, so it gets both,
    # and a lone variant is told so (| 4): should it meet a row of the other kind after all, the result is NaN, not stale scratch
    variants = (0, 2) if (s.rare_rows or table is not None) else (4,)
    for c in range(0, P, R):
        d = min(P, c + R); n = d - c
        # tile lists of the chunk, built on the device from the expert counts: list i = tiles of height 16 << i, entries
        # without a tile are skipped by the GEMM (no host synchronisation anywhere in the call)
        tiles = torch.empty(5, cap, 4, dtype=torch.int32, device=dev)
        # experts with several tiles are decoded once into scratch (rows of the common kind only: the variant kernel of the
        # others decodes in the GEMM); the side streams of _pf_chains start after these launches
        wop = S["wop"] if (S["wop"] is not None and n >= PF_HOT_MIN and not s.rare_rows and table is None) else None
        hot = torch.empty(E, dtype=torch.int32, device=dev) if wop is not None else None
        _lib.check(Lb.nq_pf_plan(cnt.data_ptr(), E, c, n, tiles.data_ptr(), cap, None if hot is None else hot.data_ptr(), PF_HOT_MIN,
                                 0 if wop is None else wop.shape[0], st))
        if wop is not None:
            for mode in (0, 1):
                _lib.check(Lb.nq_pf_wdecode(tb.data_ptr(), hot.data_ptr(), E, mode, wop.data_ptr(), wop.numel() * 2, wop.shape[0], H, I, st))
        lists = [(16 << i, tiles[i], E if i < 4 else cap) for i in (4, 3, 2, 1, 0)]          # tallest first
        pts, pes = pt[c:d], pe[c:d]
        _pf_chains(Lb, tb, lists, variants, S, x, pts, pes, n, tiles, cap, E, H, I, None if wop is None else wop.data_ptr())
        _lib.check(Lb.nq_pf_post(S["y"].data_ptr(), pos.data_ptr(), selc.data_ptr(), rwc.data_ptr(), T, k, c, n, tb.data_ptr(),
                                 out.data_ptr(), S["zd"].data_ptr(), E, H, I, st))
    return out


class Mailbox:
    """Graph-safe table updates (reference sm120/moe.py:329-342): call apply() on the compute stream before the layer;
    stage rows from a side stream with post(). One outstanding op per expert."""

    def __init__(s, layer):
        E, dev = layer.E, layer.table.device
        s.L = layer
        s.stage = torch.zeros(E, TBL_W, dtype=torch.int64, device=dev)
        s.seq = torch.zeros(E, dtype=torch.int32, device=dev)
        s.applied = torch.zeros(E, dtype=torch.int32, device=dev)
        s.applied_host = torch.zeros(E, dtype=torch.int32).pin_memory()
        s.hseq = [0] * E
        s.pins = []

    def apply(s):
        _lib.check(s.L.M.nq_mailbox(s.L.table.data_ptr(), s.stage.data_ptr(), s.seq.data_ptr(), s.applied.data_ptr(),
                                    s.applied_host.data_ptr(), s.L.E, _lib.stream_ptr()))

    def post(s, e, row, stream):
        """enqueue on `stream`, after any plane copy already enqueued there: stage[e] = row; seq[e] += 1"""
        assert s.done(e), "one outstanding op per expert"
        validate_row(row, s.L.H, s.L.I)
        s.L.rare_rows |= bool(row[4] or row[8] or row[19])
        s.hseq[e] += 1
        r = row.pin_memory(); q = torch.tensor([s.hseq[e]], dtype=torch.int32).pin_memory()
        s.pins += [r, q]
        if len(s.pins) > 4096:                       # rows whose copies completed long ago
            del s.pins[:2048]
        with torch.cuda.stream(stream):
            s.stage[e].copy_(r, non_blocking=True)
            s.seq[e:e + 1].copy_(q, non_blocking=True)

    def done(s, e):
        return int(s.applied_host[e]) == s.hseq[e]


MoELayer.prefill = prefill


PF_MIN = 384         # tokens from which a step goes through prefill() (reference NQ_PF_MIN, sm120/serve/nq_vllm.py:187)


def forward(layer, mailbox, x, topk_weights, topk_ids, pf_min=PF_MIN, sal=None):
    """One MoE layer step as the reference's serving caller runs it (sm120/serve/nq_vllm.py:520-574): apply the mailbox,
    then up to Bmax tokens in one decode call, pf_min tokens or more through prefill() (never under graph capture), anything
    between in slices of Bmax tokens. x [T, H] in fp16 / bf16 / fp32, weights [T, topk] likewise, ids int64 / int32;
    returns [T, H] in x's dtype. The decode calls read the caller's dtypes and write the result dtype themselves. `sal`: an
    optional salience.Salience, fed by the decode steps as the reference does (every step of up to Bmax tokens, the slices of
    a step of up to 16 tokens; longer steps count as prefill and are left out)."""
    T = x.shape[0]
    x, w, ids = x.contiguous(), topk_weights.contiguous(), topk_ids.contiguous()
    odt = x.dtype if x.dtype in _DT_OUT else torch.float32
    if 0 < T <= layer.Bmax:
        if sal is not None:
            sal(x, w, ids)
        return layer(x, ids, w, out=torch.empty(T, layer.H, dtype=odt, device=x.device), mailbox=mailbox)   # applied by the call's last launch, for the next step
    if mailbox is not None:
        mailbox.apply()
    if T == 0:
        return torch.empty(0, layer.H, dtype=odt, device=x.device)
    if T >= pf_min and not torch.cuda.is_current_stream_capturing():
        return layer.prefill(x.half(), ids.long(), w.half()).to(x.dtype)
    out = torch.empty(T, layer.H, dtype=odt, device=x.device)
    for i in range(0, T, layer.Bmax):
        j = min(T, i + layer.Bmax)
        layer(x[i:j], ids[i:j], w[i:j], out=out[i:j])
        if sal is not None and T <= 16:
            sal(x[i:j], w[i:j], ids[i:j])
    return out


def _lr_parts(ex, level):
    """the low-rank factors of `ex` as fp32 matrices, read back from the two table buffers (lr = V_g | U2_g | U2_u | V_d | U2_d,
    lr4 = U4_g | U4_u | U4_d): (V_g [rg, H], U_g [rg, I], U_u [rg, I], V_d [rd, I], U_d [rd, H]) with U = U2 (+ U4 at level 4)"""
    H, I, rg, rd = ex.H, ex.I, ex.rg, ex.rd
    cut = lambda t, sizes: [c.float() for c in torch.split(t[: sum(sizes)], sizes)]
    Vg, U2g, U2u, Vd, U2d = cut(ex.lr, [rg * H, rg * I, rg * I, rd * I, rd * H])
    Ug, Uu, Ud = U2g, U2u, U2d
    if level == 4:
        U4g, U4u, U4d = cut(ex.lr4, [rg * I, rg * I, rd * H])
        Ug, Uu, Ud = Ug + U4g, Uu + U4u, Ud + U4d
    return Vg.view(rg, H), Ug.view(rg, I), Uu.view(rg, I), Vd.view(rd, I), Ud.view(rd, H)


def expert_ref(ex, x, level, G=4):
    """One expert's MLP through dense weights (reference Expert.ref, sm120/moe.py:196-210): x [T, H] fp32 -> [T, H] fp32 on the
    expert's device. The weights are decoded by the HIP decoder (bit-exact values); rotations, products and sums are plain
    torch fp32 with the two fp16 roundings of the activations, so this is the slow, transparent twin of the fused kernels that
    check scripts compare them with. Rings of G = 4 lanes."""
    if G != 4:
        raise NotImplementedError("the dense decoder reads rings of G = 4 lanes")
    H, I, dev = ex.H, ex.I, ex.signs.device
    x = x.to(dev, torch.float32)
    had = lambda v, n=128: (v.reshape(*v.shape[:-1], -1, n) @ H128(dev, n)).reshape(v.shape)
    su_g, sv_g, sv_u, su_d, sv_o, su_u = torch.split(ex.signs.float(), [H, I, I, I, H, H])
    Wgu, Wdn = dense_W(ex, 0, level, torch.float32), dense_W(ex, 1, level, torch.float32)
    g = had(had(x * su_g).half().float() @ Wgu[:I].T) * sv_g
    u = had(had(x * su_u).half().float() @ Wgu[I:].T) * sv_u
    lowrank = getattr(ex, "lr", None) is not None
    if lowrank:
        Vg, Ug, Uu, Vd, Ud = _lr_parts(ex, level)
        z = x @ Vg.T
        g, u = g + z @ Ug, u + z @ Uu
    sw = torch.nn.functional.silu(g) * u
    y = had(had(sw * su_d, had_dn(ex)).half().float() @ Wdn.T) * sv_o
    if lowrank:
        y = y + (sw @ Vd.T) @ Ud
    return y


def moe_ref(experts, levels, x, sel, rw, G=4):
    """The layer through expert_ref (reference moe_ref, sm120/moe.py:344-351): out[t] = sum over the picks of rw * expert(x[t]),
    picks of level <= 0 or weight 0 skipped. Every distinct routed expert is decoded once and applied to all its tokens."""
    T, H = x.shape
    y = torch.zeros(T, H, dtype=torch.float32, device=x.device)
    xf, w = x.float(), rw.float()
    for e in sorted(set(sel.flatten().tolist())):
        if not 0 <= e < len(experts) or levels[e] <= 0:
            continue
        hit = (sel == e) & (w != 0)
        rows = hit.any(1).nonzero().flatten()
        if rows.numel():
            y[rows] += (w * hit)[rows].sum(1, keepdim=True) * expert_ref(experts[e], xf[rows], levels[e], G).to(x.device)
    return y


Expert.ref = expert_ref


def proj_gemv(layer, x, e=0, cfg=None):
    """Raw fused decode+GEMV of the gate|up projection of expert e for every token of x [B, H] (B <= 8), without the
    SwiGLU finisher: returns fp32 [B, 2I] = W_gu . fp16(Hadamard(x * su)) (rows < I rotated with su_g, the rest with su_u),
    read back from the layer's k-slice partial sums after a gate|up-only launch whose finisher output is ignored."""
    B = x.shape[0]
    sel = torch.full((B, 1), e, dtype=torch.int64, device=x.device)
    rw = torch.ones(B, 1, dtype=torch.float16, device=x.device)
    cfg = list(cfg or layer.cfg_gu)
    layer(x, sel, rw, which=1, cfg_gu=cfg)
    ny = (layer.H // 128) // (cfg[0] * cfg[2])
    n = 2 * layer.I                                               # partial sums are laid out [k-slice][B * topk of the call][2I]
    return layer.acc_gu.view(-1)[: ny * B * n].view(ny, B, n).sum(0)
