"""Plane format of NestQuant expert weights: window-pattern codes, record sizes, sub-array packing, synthetic planes.

Host-side mirror of the format half of the reference's sm120/moe.py (RKP/RK_OF :10-12, rbits :17, step_off :18-20,
proj_sizes :23-26, pack_words/unpack_words :36-66, Proj :76-107, Expert :177-195). Same names and argument meaning, so
loaders and tests written against the reference read the same here. Base codes 0 (K = 2, one uint4 per record) and 1
(K = 1.75, the residual plane's sub-array layout at 112 bits per record) are implemented; others raise.

Nested levels of this build (the reference serves levels 0/2/4 only): an expert built with nested=True also carries
P3 (64 bits / record, K=1 windows, code 10) with block words d3, and P4 (64 bits / record) with block words d4n. Level 3
decodes base + P3; nested level 4 decodes base + a 128-bit record made of P3's and P4's records and read with K=2 windows:
either the two concatenated, P3 || P4 (code 11), or the two interleaved bit by bit, stream bit 2 i = P3 bit i and bit 2 i + 1 =
P4 bit i (code 12, for experts built with interleave=True), so that every 16-bit window holds eight bits of each plane. In
device memory P4's uint2 sub-array follows P3's either way, so promotion 3 -> 4 uploads only P4 and d4n.
"""
import torch

TBL_W = 20
# window-pattern code -> (KA, MASK): step p carries KA + ((MASK >> (p % 16)) & 1) bits
RKP = {0: (2, 0), 1: (1, 0xEEEE), 2: (2, 0xAAAA), 3: (2, 0x8888), 4: (3, 0), 5: (1, 0xAAAA), 6: (1, 0xFFFE),
       7: (2, 0x9248), 8: (1, 0xFEFE), 9: (2, 0xD5AA), 10: (1, 0), 11: (2, 0), 12: (2, 0)}
RK_OF = {2: 0, 1.75: 1, 2.5: 2, 2.25: 3, 3: 4, 1.5: 5, 1.9375: 6, 2.3125: 7, 1.875: 8, 2.5625: 9}
CODE_L3, CODE_L4N, CODE_L4B = 10, 11, 12


def popc(m):
    return bin(m).count("1")


def _step_bits(KA, MASK):
    """bits carried by each of the 16 steps of a pattern period"""
    return [KA + (MASK >> r & 1) for r in range(16)]


def rbits(rk):
    """bits of one lane record: 64 steps = four periods of the code's window pattern"""
    return 4 * sum(_step_bits(*RKP[rk]))


def step_off(p, KA, MASK):
    """bit offset of step p in a stream with window pattern (KA, MASK): whole periods before it plus the steps of its own"""
    p = torch.as_tensor(p)
    bits = torch.tensor([0] + _step_bits(KA, MASK), device=p.device).cumsum(0)
    return (p >> 4) * bits[16] + bits[p & 15]


def sub_arrays(bits):
    """The sub-array layout of a plane whose records hold `bits` bits (reference sm120/moe.py:36-49, sm120/nqmoe.cu:17-20):
    [(width, pos)] for the whole elements, in storage order -- as many 128-bit ones as fit, then at most one of 64, 32 and 16
    bits, each sub-array contiguous over all records -- and the tail (bits % 16 bits per record, bit-packed over the records
    and followed by 4 bytes of padding) as (tail width, its position in the record). pos = first bit of the record the piece
    holds. The kernels walk the same table (SubArrays in csrc/nq_decode.hpp)."""
    pieces, pos = [], 0
    for width in (128, 64, 32, 16):
        while bits - pos >= width:
            pieces.append((width, pos)); pos += width
    return pieces, (bits - pos, pos)


def split_bits(bits):
    """(#uint4, uint2?, uint?, ushort?, tail bits) of a record of `bits` bits"""
    pieces, (tail, _) = sub_arrays(bits)
    count = lambda w: sum(1 for width, _ in pieces if width == w)
    return count(128), count(64), count(32), count(16), tail


def proj_sizes(N, K, nm=None, rk=0, bk=0):
    """bytes per plane of a projection [N, K] (reference sm120/moe.py:23-26). nm = None: dense residual plane; else mask
    mode: nm flagged chunks per strip, the residual plane and its block words compact over them, flags = int64 per strip"""
    S, C = N // 16, K // 128
    R = C if nm is None else nm
    pad = lambda code: 4 if rbits(code) % 16 else 0
    return dict(S=S, C=C, nm=nm, rk=rk, bk=bk, base=S * C * 32 * rbits(bk) // 8 + pad(bk),
                p4=S * R * 32 * rbits(rk) // 8 + pad(rk), d4=S * R * 4, flags=0 if nm is None else S * 8, nrec_r=S * R * 32,
                p3=S * C * 32 * 8, d3=S * C * 4)


def make_flags(S, C, nm, gen, grp=8):
    """nm flagged chunks per strip, identical across each group of `grp` strips (reference sm120/moe.py:28-34; the draw is the
    reference's, one uniform per (group, chunk), so equal seeds flag equal chunks): the nm chunks of a group whose draws rank
    lowest. -> (int64 [S], bit c = chunk c is refined; bool [S, C])"""
    dev = gen.device
    draws = torch.rand((S + grp - 1) // grp, C, generator=gen, device=dev)
    rank = draws.argsort(1).argsort(1)                            # rank of every chunk's draw within its group
    fl = (rank < nm)[torch.arange(S, device=dev) // grp]
    return (fl.long() << torch.arange(C, device=dev)).sum(1), fl


def _record_bits(w, bits):
    """w [nrec, NW] (uint32 values) -> uint8 [nrec, bits], bit i of a record = bit i % 32 of its word i // 32"""
    sh = torch.arange(32, device=w.device)
    return ((w[:, :, None] >> sh) & 1).to(torch.uint8).reshape(w.shape[0], -1)[:, :bits]


def pack_words(w, bits):
    """w [nrec, NW] int64 (uint32 values) -> int32 tensor in the sub-array layout of sub_arrays(bits). The plane is one long
    bit string: for every piece of the layout the matching columns of the record-by-bit matrix, record after record, then the
    tail columns, then zero bits up to a whole 32-bit word (a whole extra word after a tail)."""
    nrec = w.shape[0]
    B = _record_bits(w, bits)
    pieces, (tail, tpos) = sub_arrays(bits)
    runs = [B[:, pos:pos + width].reshape(-1) for width, pos in pieces]
    if tail:
        runs.append(B[:, tpos:].reshape(-1))
        fill = (-nrec * tail) % 8 + 32                            # to the byte boundary, then the 4-byte pad
        runs.append(torch.zeros(fill, dtype=torch.uint8, device=w.device))
    flat = torch.cat(runs).view(-1, 8)
    by = (flat << torch.arange(8, dtype=torch.uint8, device=w.device)).sum(1, dtype=torch.uint8)
    return by.view(torch.int32)


def unpack_words(t, nrec, bits):
    """inverse of pack_words -> [nrec, NW] int64 (uint32 values): the plane's bit string cut back into the columns of the
    record-by-bit matrix, piece by piece"""
    dev = t.device
    by = t.contiguous().view(torch.uint8)
    flat = ((by[:, None] >> torch.arange(8, dtype=torch.uint8, device=dev)) & 1).reshape(-1)
    nw = (bits + 31) // 32
    B = torch.zeros(nrec, nw * 32, dtype=torch.uint8, device=dev)
    pieces, (tail, tpos) = sub_arrays(bits)
    at = 0
    for width, pos in pieces + ([(tail, tpos)] if tail else []):
        B[:, pos:pos + width] = flat[at:at + nrec * width].view(nrec, width)
        at += nrec * width
    return (B.view(nrec, nw, 32).long() << torch.arange(32, device=dev)).sum(-1)


def lane_words_from_rings(raw, bits, G=4):
    """Ring streams -> lane records (the repack step of the reference's shard loader, sm120/nqload.py:51-55, and the inverse
    of sm120/ref15_spec.py:132-137). raw: uint8, per unit 32 / G rings of G * bits bits each, LSB-first within every byte;
    lane l of a ring holds the stream's bits [l * bits, (l + 1) * bits). -> int64 [records, ceil(bits / 32)] (uint32 values),
    records in (unit, ring, lane) order, the layout pack_words() takes."""
    raw = torch.as_tensor(raw, dtype=torch.uint8).reshape(-1)
    per_unit = 32 * bits // 8
    assert (G * bits) % 8 == 0 and raw.numel() % per_unit == 0, (bits, G, raw.numel())
    dev = raw.device
    b = ((raw.long()[:, None] >> torch.arange(8, device=dev)) & 1).reshape(-1, bits)           # one row per record
    nw = (bits + 31) // 32
    b = torch.nn.functional.pad(b, (0, nw * 32 - bits)).reshape(-1, nw, 32)
    return (b << torch.arange(32, device=dev)).sum(-1)


def rings_from_lane_words(w, bits, G=4):
    """inverse of lane_words_from_rings: int64 [records, NW] -> uint8 ring streams [records / G, G * bits / 8]"""
    dev = w.device
    b = ((w[:, :, None] >> torch.arange(32, device=dev)) & 1).reshape(w.shape[0], -1)[:, :bits]
    b = b.reshape(-1, G * bits // 8, 8)
    return (b << torch.arange(8, device=dev)).sum(-1).to(torch.uint8)


_MBN = None


def interleave_words(p3w, p4w):
    """record words of planes P3 and P4 (int64 [nrec, 2] holding uint32 values) -> the words [nrec, 4] of the 128-bit records of
    window code 12: stream bit 2 i = bit i of P3's record, bit 2 i + 1 = bit i of P4's"""
    sh = torch.arange(32, device=p3w.device)
    bits = lambda w: ((w[..., None] >> sh) & 1).reshape(w.shape[0], 64)
    both = torch.stack([bits(p3w), bits(p4w)], -1).reshape(p3w.shape[0], 4, 32)
    return (both << sh).sum(-1)


def all_MbN():
    """every valid block word (Mb, N): 1 <= Mb <= 255, 0 <= N <= 255, Mb + N <= 257"""
    global _MBN
    if _MBN is None:
        _MBN = torch.tensor([(m, n) for m in range(1, 256) for n in range(0, min(255, 257 - m) + 1)])
    return _MBN


def _block_words(nb, gen, mbn, dev):
    """'rand': realistic delta = N / Mb ~ 0.1-0.8 plus 5% random extremes; ('exh', offset): cycle through all_MbN()"""
    if mbn != "rand":
        table = all_MbN().to(dev)
        pick = table[(torch.arange(nb, device=dev) + mbn[1]) % len(table)]
        return pick[:, 0], pick[:, 1]
    # five draws in the reference's order (sm120/moe.py:93-97), so that the same seed gives the same block words
    uniform = lambda: torch.rand(nb, generator=gen, device=dev)
    integer = lambda lo: torch.randint(lo, 256, (nb,), generator=gen, device=dev)
    m_usual = integer(120)
    n_usual = (uniform() * 0.8 * m_usual).round().long()
    extreme = uniform() < 0.05
    m_any = integer(1)
    n_any = (uniform() * (torch.clamp(257 - m_any, max=255) + 1)).floor().long()
    Mb = torch.where(extreme, m_any, m_usual)
    return Mb, torch.minimum(torch.where(extreme, n_any, n_usual), 257 - Mb)


class Proj:
    """Random packed planes of one projection of one expert, each plane its own tensor so it can live in a pool.
    base int32 [nrec*4]; p4 int32 (packed sub-arrays of residual code rk), d4 int32 (Mb | N << 8 per unit);
    nested=True adds p3 / d3 and p4n / d4n (int32, uint2 per record) drawn after everything else, so the other planes
    do not depend on it. The draws before that follow the reference's order (sm120/moe.py:80-103), so a CPU generator
    with the same seed yields the same planes as the reference's Proj."""

    def __init__(s, N, K, gen, nm=None, rk=0, mbn="rand", var=False, bk=0, nested=False):
        if bk not in (0, 1):
            raise NotImplementedError("base codes other than 0 (K = 2) and 1 (K = 1.75) are not implemented")
        if nm is not None and nested:
            raise NotImplementedError("mask mode applies to the wide residual plane, not to the nested planes")
        dev = gen.device
        z = proj_sizes(N, K, nm, rk, bk)
        s.z, s.N, s.K, s.rk, s.bk, s.nested = z, N, K, rk, bk, nested
        S, C = z["S"], z["C"]
        R = C if nm is None else nm                      # residual records and block words exist for R chunks per strip
        nr, nb = S * C * 32, S * R
        bits = rbits(rk); nw = (bits + 31) // 32
        def record_words(nrec, nbits):
            """random records of nbits bits as 32-bit words in int64 [nrec, ceil(nbits / 32)], the unused top bits cleared"""
            words = torch.randint(0, 2**32, (nrec, (nbits + 31) // 32), generator=gen, dtype=torch.int64, device=dev)
            if nbits % 32:
                words[:, -1] &= (1 << (nbits % 32)) - 1
            return words
        block = lambda Mb, N: (Mb | (N << 8)).to(torch.int32)
        s.bw = None
        if bk:                                          # record words of the base code, stored in the sub-array layout
            s.bw = record_words(nr, rbits(bk))
            s.base = pack_words(s.bw, rbits(bk))
        else:
            s.base = torch.randint(-2**31, 2**31 - 1, (nr * 4,), generator=gen, dtype=torch.int32, device=dev)
        s.p4w = record_words(nb * 32, bits)
        s.p4 = pack_words(s.p4w, bits)
        s.Mb, s.Nn = _block_words(nb, gen, mbn, dev)
        s.d4 = block(s.Mb, s.Nn)
        s.var = torch.randint(0, 256, (S * C,), generator=gen, dtype=torch.int64, device=dev).to(torch.uint8) if var else None
        s.flags, s.fl = (None, None) if nm is None else make_flags(S, C, nm, gen)
        s.p3 = s.d3 = s.p4n = s.d4n = s.p3w = s.p4nw = None
        if nested:
            s.p3w, s.p4nw = record_words(nr, 64), record_words(nr, 64)
            s.p3, s.p4n = pack_words(s.p3w, 64), pack_words(s.p4nw, 64)
            s.Mb3, s.N3 = _block_words(S * C, gen, "rand", dev)
            s.Mb4n, s.N4n = _block_words(S * C, gen, "rand", dev)
            s.d3, s.d4n = block(s.Mb3, s.N3), block(s.Mb4n, s.N4n)

    _TENSORS = ["base", "bw", "p4", "d4", "flags", "fl", "p4w", "Mb", "Nn", "var", "p3", "d3", "p4n", "d4n", "p3w", "p4nw"]

    def to(s, dev):
        for k in s._TENSORS:
            if getattr(s, k, None) is not None:
                setattr(s, k, getattr(s, k).to(dev))
        return s

    def drop_host_words(s):
        """free the unpacked word tensors (only tests need them)"""
        s.p4w = s.p3w = s.p4nw = s.bw = None
        return s

    def nested_plane(s):
        """device layout of the nested two-plane record: P3's uint2 sub-array followed by P4's"""
        return torch.cat([s.p3, s.p4n])


class Expert:
    """Synthetic expert: gate|up [2I, H] and down [H, I] planes + fp16 sign vector
    [H su_g | I sv_g | I sv_u | I su_d | H sv_o | H su_u] (reference sm120/moe.py:177-183)."""

    def __init__(s, H, I, seed, nm_gu=None, nm_dn=None, dev="cuda", rk_gu=0, rk_dn=0, mbn="rand", var=False,
                 bk_gu=0, bk_dn=0, nested=False, gen_dev="cpu", interleave=False):
        gen = torch.Generator(device=gen_dev).manual_seed(seed)
        mbn_dn = mbn if mbn == "rand" else ("exh", mbn[1] + (2 * I // 16) * (H // 128))
        s.gu = Proj(2 * I, H, gen, nm_gu, rk_gu, mbn, var, bk_gu, nested).to(dev)
        s.dn = Proj(H, I, gen, nm_dn, rk_dn, mbn_dn, var, bk_dn, nested).to(dev)
        signs = lambda n: torch.randint(0, 2, (n,), generator=gen, device=gen_dev) * 2 - 1
        s.signs = torch.cat([signs(2 * H + 3 * I), signs(H)]).half().to(dev)     # five vectors in one draw, then su_u
        s.H, s.I, s.nested = H, I, nested
        s.l4code = CODE_L4B if interleave else CODE_L4N           # how nested level 4 reads P3 and P4: interleaved or concatenated
        s.lr, s.lr4, s.rg, s.rd = None, None, 0, 0
        if nested:                                       # slot image: [P3 | P4] per projection, contiguous
            s.gu.slot = s.gu.nested_plane(); s.dn.slot = s.dn.nested_plane()

    def set_lr(s, Vg, U2g, U2u, U4g, U4u, Vd, U2d, U4d):
        """low-rank plane (fp16; reference sm120/moe.py:184-189): Vg [rg, H], U2g / U2u / U4g / U4u [rg, I], Vd [rd, I],
        U2d / U4d [rd, H] -> the two buffers of table words 14 / 15: lr = Vg | U2g | U2u | Vd | U2d, lr4 = U4g | U4u | U4d"""
        s.lrT = (Vg, U2g, U2u, U4g, U4u, Vd, U2d, U4d)
        s.rg, s.rd = Vg.shape[0], Vd.shape[0]
        s.lr = s.lr4 = None
        if s.rg or s.rd:
            flat = lambda parts: torch.cat([t.reshape(-1) for t in parts]).half().contiguous().to(s.signs.device)
            s.lr, s.lr4 = flat((Vg, U2g, U2u, Vd, U2d)), flat((U4g, U4u, U4d))
        return s

    def compact(s):
        """drop everything a layer call does not read (unpacked words; for nested experts the wide plane and the separate
        P3 / P4 tensors, whose bytes live on in `slot`)"""
        for p in (s.gu, s.dn):
            p.drop_host_words()
            p.Mb = p.Nn = None
            if s.nested:
                p._nbytes = dict(p3=p.p3.numel() * 4, p4n=p.p4n.numel() * 4, p4=p.p4.numel() * 4)
                p.p4 = p.d4 = p.p3 = p.p4n = None
                for k in ("Mb3", "N3", "Mb4n", "N4n"):
                    setattr(p, k, None)
        return s

    def bytes(s, level):
        """plane bytes a layer call reads for this expert at `level` (the reference's GB/s numerator, sm120/moe.py:190-195)"""
        b = 0
        for p in (s.gu, s.dn):
            b += p.base.numel() * 4 + (0 if p.var is None else p.var.numel())
            nb = getattr(p, "_nbytes", None) or dict(p3=0 if p.p3 is None else p.p3.numel() * 4,
                                                      p4n=0 if p.p4n is None else p.p4n.numel() * 4)
            if level == 3:
                b += nb["p3"] + p.d3.numel() * 4
            elif level >= 4 and s.nested:
                b += nb["p3"] + nb["p4n"] + p.d4n.numel() * 4
            elif level >= 4:
                b += (p.p4.numel() + p.d4.numel()) * 4
        return b
