"""CPU oracle for the NestQuant routed-expert MoE hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module; only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may. It restates, in plain numpy, the algorithm of the reference's bit-level spec and torch reference:

  window patterns / step offsets      reference sm120/ref15_spec.py:43-46, sm120/moe.py:10-20
  ring streams and 16-bit states      reference sm120/ref15_spec.py:49-61, sm120/moe.py:111-127
  mul1 hash and byte sum S            reference sm120/ref15_spec.py:64-70, sm120/moe.py:114-116
  level-2 value Q2                    reference sm120/ref15_spec.py:17,76, sm120/moe.py:145
  RM_P integer fold (levels 3/4)      reference sm120/ref15_spec.py:79-90, sm120/moe.py:128-134
  unit geometry / dense scatter       reference sm120/ref15_spec.py:118-129, sm120/moe.py:156-166
  residual sub-array packing          reference sm120/moe.py:21-66
  Hadamard-128, expert and layer math reference sm120/moe.py:168-172,196-210,344-351
  routing dedup into runs             reference sm120/nqmoe.cu:375-449
  mailbox state machine               reference sm120/nqmoe.cu:908-923, tests/test_prefill_borrow_cpu.py:36-42
  decode salience export              reference sm120/nqsal.cu:20-60 (the value, in float64)

Two independent decoders live here on purpose: `lane_sums` (lane-local view: a lane's own record plus the first word
of its ring neighbour) and `ring_states` (ring bit-stream view). Tests require them to agree; either alone could hide
a transcription slip in the lane/ring bookkeeping.

Pinned by (see tests/test_oracle_*.py): closed forms and known answers from the reference text (K0 = -3.453125,
zero-mean unit-variance codebook with A ~ 1/147.7 and B ~ -10.39, RBITS table, published plane byte sizes, 33149 valid
block words, exact rational arithmetic for the single-rounded FMAs, unit geometry bijection, Hadamard orthonormality,
the effective-weight identity of the layer) and by golden fixtures holding outputs of the reference's own CPU decoder
(tests/golden/make_fixtures.py): every function here is pinned by at least one of the two.

Nested levels of this build (no production counterpart in the reference; definition in the format notes of the
package): code 10 = K=1 window pattern (1, 0x0000) over a 64-bit record (level 3, plane P3); code 11 = K=2 windows over
the 128-bit record formed by P3's record followed by P4's record (two-plane level 4). Both decode through the same
generic (KA, MASK) machinery as the reference's codes 0..9.
"""
import numpy as np

HC = 0x83DCD12D
TBL_W = 20
A16 = np.array([0x1EEE], np.uint16).view(np.float16)[0]
B16 = np.array([0xC931], np.uint16).view(np.float16)[0]
A_ = float(A16)
B_ = float(B16)
K0 = 1024.0 * A_ + B_                       # -3.453125 exactly
# residual / base window patterns: code -> (KA, MASK); step p carries KA + ((MASK >> (p % 16)) & 1) bits
RKP = {0: (2, 0x0000), 1: (1, 0xEEEE), 2: (2, 0xAAAA), 3: (2, 0x8888), 4: (3, 0x0000), 5: (1, 0xAAAA),
       6: (1, 0xFFFE), 7: (2, 0x9248), 8: (1, 0xFEFE), 9: (2, 0xD5AA),
       10: (1, 0x0000),                       # nested level 3: one refinement plane, 1 bit per step
       11: (2, 0x0000),                       # nested level 4: P3 record || P4 record, 2 bits per step
       12: (2, 0x0000)}                       # nested level 4: P3 and P4 records interleaved bit by bit, 2 bits per step
NESTED_L3, NESTED_L4, NESTED_L4B = 10, 11, 12


def interleave_words(p3, p4):
    """lane records of planes P3 and P4 (uint32 [nrec, 2] each: 64 bits per record) -> the 128-bit records [nrec, 4] whose
    stream bit 2 i is bit i of P3's record and bit 2 i + 1 is bit i of P4's, so that every 16-bit window of the 2-bits-per-step
    stream holds eight bits of each plane (the state of the reference's research decoder T2R2, threads/04-decode-kernel/
    nqk.cu:109, in LSB-first stream order). Lane and ring boundaries stay where they are: the ring stream of the result is
    the bitwise interleave of the two planes' ring streams."""
    bits = lambda w: ((np.asarray(w, np.uint64)[..., None] >> np.arange(32, dtype=np.uint64)) & np.uint64(1)).reshape(len(w), -1)
    b = np.stack([bits(p3), bits(p4)], -1).reshape(len(p3), 128)
    return (b.reshape(len(p3), 4, 32) << np.arange(32, dtype=np.uint64)).sum(-1).astype(np.uint32)


def popc(m):
    return bin(int(m)).count("1")


def rbits(code):
    """bits of one lane record (64 weights) of a plane coded with window pattern `code`"""
    ka, mask = RKP[code]
    return 4 * (16 * ka + popc(mask))


def step_off(p, ka, mask):
    """bit offset of trellis step p in a stream with window pattern (ka, mask); works on ints or arrays"""
    p = np.asarray(p, np.int64)
    within = np.zeros(16, np.int64)
    for r in range(1, 16):
        within[r] = within[r - 1] + ka + ((mask >> (r - 1)) & 1)
    return (p >> 4) * (16 * ka + popc(mask)) + within[p & 15]


# ----------------------------------------------------------------------------------------------------------------------
# plane packing (residual records as sub-arrays)
def split_bits(bits):
    """record of `bits` bits -> (#uint4, has uint2, has uint, has ushort, tail bits)"""
    rem = bits % 128
    return bits // 128, rem // 64, (rem % 64) // 32, (rem % 32) // 16, bits % 16


def plane_bytes(nrec, code):
    b = rbits(code)
    return nrec * b // 8 + (4 if b % 16 else 0)


def _le_bytes(vals, nb):
    v = np.asarray(vals, np.uint64)
    out = np.empty(v.shape + (nb,), np.uint8)
    for i in range(nb):
        out[..., i] = (v >> np.uint64(8 * i)) & np.uint64(255)
    return out.reshape(-1)


def pack_words(w, bits, split_halves=False):
    """w [nrec, NW] (uint32 values, bit i of the record = bit i%32 of word i//32) -> uint8 bytes of the sub-array layout:
    uint4 x n4 | uint2 | uint | ushort, each sub-array contiguous over all records, then the tail (bits % 16 bits per
    record, bit-packed over records, plus a 4-byte pad). split_halves: 128-bit records stored as uint2 | uint2 (the
    nested two-plane layout, code 11)."""
    w = np.asarray(w, np.uint64)
    nrec = w.shape[0]
    if split_halves:
        assert bits == 128
        return np.concatenate([_le_bytes(w[:, 0:2], 4), _le_bytes(w[:, 2:4], 4)])
    n4, n2, n1, nh, tail = split_bits(bits)
    parts, k = [], 0
    if n4:
        parts.append(_le_bytes(w[:, :4 * n4], 4)); k = 4 * n4
    if n2:
        parts.append(_le_bytes(w[:, k:k + 2], 4)); k += 2
    if n1:
        parts.append(_le_bytes(w[:, k], 4)); k += 1
    if nh:
        parts.append(_le_bytes(w[:, k] & np.uint64(0xFFFF), 2))
    if tail:
        a = bits - tail
        t = (w[:, a // 32] >> np.uint64(a % 32)) & np.uint64((1 << tail) - 1)
        b = ((t[:, None] >> np.arange(tail, dtype=np.uint64)) & np.uint64(1)).astype(np.uint8).reshape(-1)
        b = np.concatenate([b, np.zeros(32, np.uint8)])
        b = b[: b.size // 8 * 8].reshape(-1, 8)
        parts.append((b << np.arange(8, dtype=np.uint8)).sum(1).astype(np.uint8))
    return np.concatenate(parts)


def unpack_words(buf, nrec, bits, split_halves=False):
    """inverse of pack_words -> [nrec, NW] uint32"""
    b = np.frombuffer(np.ascontiguousarray(buf).tobytes(), np.uint8).astype(np.uint64)
    nw = (bits + 31) // 32
    w = np.zeros((nrec, nw), np.uint64)
    pos = 0

    def take(nwords, nb):
        nonlocal pos
        x = b[pos:pos + nrec * nwords * nb].reshape(nrec, nwords, nb)
        pos += nrec * nwords * nb
        return (x << (np.uint64(8) * np.arange(nb, dtype=np.uint64))).sum(-1)

    if split_halves:
        assert bits == 128
        w[:, 0:2] = take(2, 4); w[:, 2:4] = take(2, 4)
        return w.astype(np.uint32)
    n4, n2, n1, nh, tail = split_bits(bits)
    k = 0
    if n4:
        w[:, :4 * n4] = take(4 * n4, 4); k = 4 * n4
    if n2:
        w[:, k:k + 2] = take(2, 4); k += 2
    if n1:
        w[:, k] = take(1, 4)[:, 0]; k += 1
    if nh:
        w[:, k] = take(1, 2)[:, 0]
    if tail:
        a = bits - tail
        bb = b[pos:pos + (nrec * tail + 7) // 8]
        bit = ((bb[:, None] >> np.arange(8, dtype=np.uint64)) & np.uint64(1)).reshape(-1)[: nrec * tail]
        bit = bit.reshape(nrec, tail)
        w[:, a // 32] |= (bit << np.arange(tail, dtype=np.uint64)).sum(-1) << np.uint64(a % 32)
    return w.astype(np.uint32)


def proj_sizes(N, K, rk=0, bk=0):
    """plane byte sizes of a dense projection [N, K] (strip = 16 rows, chunk = 128 columns)"""
    S, C = N // 16, K // 128
    nrec = S * C * 32
    return dict(S=S, C=C, nrec=nrec, base=plane_bytes(nrec, bk), p4=plane_bytes(nrec, rk), d4=S * C * 4)


# ----------------------------------------------------------------------------------------------------------------------
# code -> value
def hash_sum(st):
    """S(state): byte sum of state * HC mod 2^32, 0..1020"""
    x = (np.asarray(st, np.uint64) * np.uint64(HC)) & np.uint64(0xFFFFFFFF)
    return ((x & np.uint64(255)) + ((x >> np.uint64(8)) & np.uint64(255)) + ((x >> np.uint64(16)) & np.uint64(255))
            + (x >> np.uint64(24))).astype(np.int64)


def f16(v):
    """single rounding of a float64 array to fp16"""
    return np.asarray(v, np.float64).astype(np.float16)


def q2_value(sb, sign=1.0):
    """level-2 value from the byte sum Sb: fp16(A (1024 + Sb) + B), one rounding"""
    return f16((sign * A_) * (1024.0 + np.asarray(sb, np.float64)) + sign * B_)


def fold_consts(Mb, N):
    """per-unit fp16 constants (A', C) of the integer fold, fp32 operations in the spec's order, no contraction"""
    Mb = np.asarray(Mb); N = np.asarray(N)
    rcp = np.float32(1.0) / Mb.astype(np.float32)
    Ah = (np.float32(1.732421875) * rcp).astype(np.float16)
    t = (N.astype(np.float32) * rcp) * np.float32(K0)
    t = t + np.float32(K0)
    Ch = (t - np.float32(1024.0) * Ah.astype(np.float32)).astype(np.float16)
    return Ah, Ch


def fold_value(Sb, Sr, Mb, N, sign=1.0):
    """levels 3/4: F = (Mb Sb + N Sr + 128) >> 8 ; value = fp16(A' (1024 + F) + C), one rounding"""
    Ah, Ch = fold_consts(Mb, N)
    F = (np.asarray(Mb, np.int64) * Sb + np.asarray(N, np.int64) * Sr + 128) >> 8
    return f16((sign * Ah.astype(np.float64)) * (1024.0 + F) + sign * Ch.astype(np.float64))


def all_block_words():
    """every valid (Mb, N): 1 <= Mb <= 255, 0 <= N <= 255, Mb + N <= 257"""
    return np.array([(m, n) for m in range(1, 256) for n in range(0, min(255, 257 - m) + 1)], np.int64)


# ----------------------------------------------------------------------------------------------------------------------
# decoders
def lane_sums(words, code, G=4):
    """Lane-local view. words [nrec, NW] uint32, records lane-minor (record index = unit*32 + lane); a ring is G
    consecutive lanes. Returns S(state) at each of the 64 lane weights -> int64 [nrec, 64]."""
    ka, mask = RKP[code]
    bits = rbits(code)
    w = np.asarray(words, np.uint64)
    nrec, nw = w.shape
    assert nw == (bits + 31) // 32 and nrec % G == 0
    lane = np.arange(nrec)
    nb = (lane // G) * G + (lane % G + 1) % G                 # ring neighbour holding the next bits of the stream
    first = w[nb, 0]
    ext = np.zeros((nrec, nw + 2), np.uint64)                 # own record, then the neighbour's first 32 bits
    ext[:, :nw] = w
    t = bits % 32
    if t == 0:
        ext[:, nw] = first
    else:
        ext[:, nw - 1] = (ext[:, nw - 1] & np.uint64((1 << t) - 1)) | ((first << np.uint64(t)) & np.uint64(0xFFFFFFFF))
        ext[:, nw] = first >> np.uint64(32 - t)
    out = np.empty((nrec, 64), np.int64)
    offs = step_off(np.arange(64), ka, mask)
    for j in range(64):
        o = int(offs[j]); i, s = o >> 5, o & 31
        both = ext[:, i] | (ext[:, i + 1] << np.uint64(32))
        out[:, j] = hash_sum((both >> np.uint64(s)) & np.uint64(0xFFFF))
    return out


def ring_states(words, code, G=4):
    """Ring-stream view (independent of lane_sums): concatenate the G lane records of each ring LSB-first, read the
    16-bit tail-biting window at step_off(p) for p = 0..64G-1. Returns states int64 [nrec/G, 64 G]."""
    ka, mask = RKP[code]
    bits = rbits(code)
    w = np.asarray(words, np.uint64)
    nrec = w.shape[0]
    b = ((w[:, :, None] >> np.arange(32, dtype=np.uint64)) & np.uint64(1)).reshape(nrec, -1)[:, :bits]
    ring = b.reshape(nrec // G, G * bits).astype(np.int64)
    L = G * bits
    off = step_off(np.arange(64 * G), ka, mask)
    assert int(step_off(64 * G, ka, mask)) == L
    idx = (off[:, None] + np.arange(16)) % L
    return (ring[:, idx] << np.arange(16)).sum(-1)


class Plane:
    """planes of one projection as the oracle sees them (all numpy, host memory):
    N, K; base [nrec,4] uint32; level-4 residual: rk code + res [nrec,NW] uint32 + d4 [units] uint32 (Mb | N << 8);
    nested planes: p3 [nrec,2] + d3 [units], p4n [nrec,2] + d4n [units]; var: uint8 per unit (bit g = ring g negated);
    flags (mask mode, reference sm120/moe.py:134-155): int64 per strip, bit c = chunk c is refined; res and d4 then hold only
    the popcount(flags) refined chunks of each strip, in chunk order, and the other chunks decode at level 2.
    bk: window code of the base plane (reference sm120/moe.py:138-140, sm120/NQ_RES_V2.md:36-49): 0 = two bits per step,
    128-bit records; otherwise base holds the record words [nrec, ceil(rbits(bk) / 32)] of that code's pattern."""

    def __init__(self, N, K, base, rk=0, res=None, d4=None, p3=None, d3=None, p4n=None, d4n=None, var=None, flags=None, bk=0):
        self.N, self.K = N, K
        self.S, self.C = N // 16, K // 128
        self.bk = bk
        self.base = np.asarray(base, np.uint32).reshape(-1, (rbits(bk) + 31) // 32)
        self.rk, self.res, self.d4 = rk, res, d4
        self.p3, self.d3, self.p4n, self.d4n, self.var = p3, d3, p4n, d4n, var
        self.flags = None if flags is None else np.asarray(flags, np.int64)
        assert self.base.shape[0] == self.S * self.C * 32

    def residual(self, level, nested):
        """-> (code, words, block words) used at `level`"""
        if level == 3:
            return NESTED_L3, self.p3, self.d3
        if nested == "interleave":
            return NESTED_L4B, interleave_words(self.p3, self.p4n), self.d4n
        if nested:
            return NESTED_L4, np.concatenate([self.p3, self.p4n], 1), self.d4n
        return self.rk, self.res, self.d4


def lane_vals(p, level, nested=False, G=4):
    """decoded weights in lane-weight order -> fp16 [S, C, 32, 64]"""
    S, C = p.S, p.C
    Sb = lane_sums(p.base, p.bk, G).reshape(S, C, 32, 64)
    sign = 1.0
    if p.var is not None:
        ring = np.arange(32) >> 2
        bit = (np.asarray(p.var, np.int64).reshape(S, C, 1) >> ring) & 1
        sign = (1.0 - 2.0 * bit)[..., None]
    if level == 2:
        return q2_value(Sb, sign)
    code, words, dw = p.residual(level, nested)
    if p.flags is None or level == 3 or nested:
        Sr = lane_sums(words, code, G).reshape(S, C, 32, 64)
        dw = np.asarray(dw, np.int64).reshape(S, C, 1, 1)
        return fold_value(Sb, Sr, dw & 255, (dw >> 8) & 255, sign)
    on = ((p.flags[:, None] >> np.arange(C)[None]) & 1).astype(bool)            # [S, C]
    R = int(on[0].sum())
    assert (on.sum(1) == R).all(), "every strip flags the same number of chunks"
    rank = np.minimum(np.cumsum(on, 1) - on, R - 1)
    si = np.arange(S)[:, None] + 0 * rank
    Sr = lane_sums(words, code, G).reshape(S, R, 32, 64)[si, rank]
    dw = np.asarray(dw, np.int64).reshape(S, R)[si, rank][..., None, None]
    q4 = fold_value(Sb, Sr, dw & 255, (dw >> 8) & 255, sign)
    return np.where(on[..., None, None], q4, q2_value(Sb, sign))


def lane_to_rowcol():
    """lane (0..31), lane weight j (0..63) -> (row in strip, column in chunk)"""
    lane = np.arange(32)[:, None]; j = np.arange(64)[None, :]
    g, t4 = lane >> 2, lane & 3
    pp, e = j >> 1, j & 1
    t, r = pp >> 2, pp & 3
    row = g + 8 * (r & 1) + 0 * j
    col = 16 * t + 2 * t4 + 8 * (r >> 1) + e
    return row, col


def dense_W(p, level, nested=False, G=4):
    """dense rotated-domain weight matrix [N, K] fp16 (bit-exact values)"""
    f = lane_vals(p, level, nested, G)
    S, C = p.S, p.C
    row, col = lane_to_rowcol()
    W = np.zeros((p.N, p.K), np.float16)
    rows = (np.arange(S)[:, None, None, None] * 16 + row[None, None]) + np.zeros((1, C, 1, 1), np.int64)
    cols = (np.arange(C)[None, :, None, None] * 128 + col[None, None]) + np.zeros((S, 1, 1, 1), np.int64)
    W[rows.reshape(-1), cols.reshape(-1)] = f.reshape(-1)
    return W


# ----------------------------------------------------------------------------------------------------------------------
# layer math
def hadamard(n=128):
    """normalised Sylvester Hadamard matrix of order n"""
    H = np.ones((1, 1))
    while H.shape[0] < n:
        H = np.block([[H, H], [H, -H]])
    return (H / np.sqrt(n)).astype(np.float32)


def wht(v, n=128, dtype=np.float32):
    """Hadamard-n on each n-block of the last axis (fp32 unless dtype says otherwise)"""
    v = np.asarray(v, dtype)
    return (v.reshape(*v.shape[:-1], -1, n) @ hadamard(n).astype(dtype)).reshape(v.shape)


def split_signs(signs, H, I):
    """[H su_g | I sv_g | I sv_u | I su_d | H sv_o | H su_u] -> dict of fp32 vectors"""
    s = np.asarray(signs, np.float16).astype(np.float32)
    o = [0, H, H + I, H + 2 * I, H + 3 * I, 2 * H + 3 * I, 3 * H + 3 * I]
    names = ["su_g", "sv_g", "sv_u", "su_d", "sv_o", "su_u"]
    return {n: s[o[i]:o[i + 1]] for i, n in enumerate(names)}


def expert_forward(x, Wgu, Wdn, signs, round_acts=True, dtype=np.float32, had_dn=128, lr=None, level=4):
    """x [T,H] through dense weights Wgu [2I,H], Wdn [H,I] (arrays holding fp16 values) -> [T,H]
    (reference sm120/moe.py:196-210).
    round_acts: round the two rotated activations to fp16 as the kernels do (False = no activation rounding).
    dtype: arithmetic type; float64 gives the exact-arithmetic arbiter used to separate rounding noise from errors.
    had_dn: width of the Hadamard on the down projection's input (128, or 512 = in_had_down).
    lr: low-rank plane, dict of fp16-valued arrays Vg [rg,H], U2g/U2u/U4g/U4u [rg,I], Vd [rd,I], U2d/U4d [rd,H]; the U4
    terms count at level 4 only."""
    H, I = Wdn.shape
    sg = {k: v.astype(dtype) for k, v in split_signs(signs, H, I).items()}
    rnd = (lambda a: a.astype(np.float16).astype(dtype)) if round_acts else (lambda a: a)
    x = np.asarray(x, dtype)
    Wgu = np.asarray(Wgu, dtype); Wdn = np.asarray(Wdn, dtype)
    wht_ = lambda v, n=128: wht(v, n, dtype)
    xg = rnd(wht_(x * sg["su_g"])); xu = rnd(wht_(x * sg["su_u"]))
    g = wht_(xg @ Wgu[:I].T) * sg["sv_g"]
    u = wht_(xu @ Wgu[I:].T) * sg["sv_u"]
    if lr is not None:
        L = {k: np.asarray(v, dtype) for k, v in lr.items()}
        z = x @ L["Vg"].T
        g = g + z @ L["U2g"] + (z @ L["U4g"] if level == 4 else 0)
        u = u + z @ L["U2u"] + (z @ L["U4u"] if level == 4 else 0)
    with np.errstate(over="ignore"):                       # exp overflow gives the correct limit silu(-inf) = -0
        sw = g / (1.0 + np.exp(-g)) * u
    h = rnd(wht_(sw * sg["su_d"], had_dn))
    y = wht_(h @ Wdn.T) * sg["sv_o"]
    if lr is not None:
        z = sw @ L["Vd"].T
        y = y + z @ L["U2d"] + (z @ L["U4d"] if level == 4 else 0)
    return y


def moe_forward(dense, levels, signs, x, sel, rw, round_acts=True, dtype=np.float32, had_dn=128, lr=None):
    """dense: callable e -> (Wgu fp32 [2I,H], Wdn fp32 [H,I]) at the expert's level; levels [E]; signs: e -> vector.
    x [B,H] fp16/fp32, sel [B,topk] int, rw [B,topk] fp16 -> [B,H] fp32. Picks with rw == 0 or level <= 0 add 0.
    had_dn: down-input Hadamard width of every expert; lr: optional callable e -> low-rank dict (or None)."""
    x = np.asarray(x, dtype)
    out = np.zeros_like(x)
    cache = {}
    for b in range(x.shape[0]):
        for k in range(sel.shape[1]):
            e = int(sel[b, k]); w = float(rw[b, k])
            if levels[e] <= 0 or w == 0.0:
                continue
            if e not in cache:
                cache[e] = dense(e)
            Wgu, Wdn = cache[e]
            out[b] += dtype(w) * expert_forward(x[b:b + 1], Wgu, Wdn, signs(e), round_acts, dtype, had_dn,
                                                None if lr is None else lr(e), levels[e])[0]
    return out


def route_runs(sel, rw, levels):
    """dedup the B*topk picks into runs: one run per distinct active expert, numbered by first occurrence; slots
    (= flat pick index) within a run in pick order. Inactive picks (rw == 0 or level <= 0) are dropped."""
    flat = np.asarray(sel).reshape(-1); w = np.asarray(rw, np.float32).reshape(-1)
    runs, index = [], {}
    for s, e in enumerate(flat.tolist()):
        if w[s] == 0 or levels[e] <= 0:
            continue
        if e not in index:
            index[e] = len(runs); runs.append(dict(e=e, slots=[], w=[]))
        runs[index[e]]["slots"].append(s); runs[index[e]]["w"].append(float(w[s]))
    return runs


def mailbox_apply(table, stage, seq, applied):
    """table[e] <- stage[e] wherever seq[e] != applied[e]; then applied <- seq (in place, numpy arrays)"""
    m = seq != applied
    table[m] = stage[m]
    applied[m] = seq[m]
    return int(m.sum())


def salience(x, w, ids, rsf, acc, E=None):
    """acc[e] += sum over picks (t, k) of expert e of (rsf * w[t, k])^2 * |x[t]|^2 (reference sm120/nqsal.cu:20-60), in place on
    the float64 array `acc`; returns the indices written, in first-pick order. x [T, H] float16 (or float32 holding bf16 /
    fp16 values), w [T, K] float16, ids [T, K] integers; picks with w == 0 or an id outside [0, E) are skipped.
    This is the value the export stands for, in float64 throughout except that rsf * w is formed in fp32 as the kernels form
    it; a kernel's fp32 norm agrees with it to fp32 rounding (tests allow 1e-5 relative) and exactly where every partial sum
    is exact (rows of small powers of two). Pinned by exact known answers; the reference holds no stored output of its kernel."""
    x = np.asarray(x); w = np.asarray(w, np.float16); ids = np.asarray(ids)
    T, H = x.shape
    K = ids.shape[1]
    E = len(acc) if E is None else E
    assert T <= 8 and K <= 8
    xn = (x.astype(np.float64) ** 2).sum(1)
    wf = w.astype(np.float32).reshape(-1)
    idf = ids.reshape(-1).astype(np.int64)
    ww = (wf * np.float32(rsf)).astype(np.float32).astype(np.float64)
    term = ww * ww * np.repeat(xn, K)
    live = (wf != 0) & (idf >= 0) & (idf < E)
    touched = []
    for e in dict.fromkeys(idf[live].tolist()):                  # first-pick order; each expert's picks added in pick order
        tot = 0.0
        for j in np.nonzero(live & (idf == e))[0]:
            tot += term[j]
        acc[e] = acc[e] + tot
        touched.append(e)
    return touched
