"""Minimal encoder: dense weight [N, K] -> 2-bit trellis base plane + fp16 sign/scale vectors (encode_level2), and on top
of it the refinement planes of levels 3 and 4 fitted to the base plane's residual (encode_nested), optionally with the
errors of later column chunks fed forward through the block LDL factor of the input Hessian (encode_ldlq).

It exists to produce honest planes for the CPU-plumbing configuration (one 512 x 256 weight, encode -> decode -> GEMV);
it is not the reference's production encoder. What it restates, in plain torch that runs on CPU or GPU:
  * the quick-fit preprocessing with identity Hessian, where LDLQ feedback vanishes (reference sm120/quickfit/fit_quick.py:1-4,
    threads/12-reference-encoder/nq_encode.py:135-172): seeded +-1 signs, per-channel scales, Hadamard-128 on both sides,
    so that  W ~= D(sv) B_N Q B_K D(su)  with B the 128-blocked orthonormal Hadamard;
  * the tail-biting Viterbi over the 16-bit shift-register trellis with the mul1 codebook (reference
    threads/05-exl3-harness/harness.py:297-364: pass 1 rolled by half a ring finds the state entering step 0, pass 2 is
    constrained to start from and end in it), Viterbi step i <-> ring position p = (-i) mod 256
    (threads/12-reference-encoder/nq_encode.py:54-58);
  * the LSB-first packing of ring states into lane records (threads/12-reference-encoder/nq_decode.py:101-109);
  * the greedy refinement stage with identity Hessian (threads/12-reference-encoder/nq_encode.py:286-316 without the LDLQ
    feedback terms; threads/03-nested-trellis-code/exp3.py:20-26,55-60): the residual of the frozen base plane, divided by
    its rms per unit and by the input scale the reference found best on Gaussian data (1.1 at one bit per weight, 1.0 at
    two), goes through the same Viterbi with K = 1 or 2 bits per step; the least-squares step size delta = N / Mb is then
    searched over the reference's twelve block-word candidates (nq_encode.py:186-198, nq_decode.py:158-163) with the
    integer fold itself (sm120/ref15_spec.py:79-90) as the cost, so the chosen word is the best of them for the values
    the decoder really produces.
  * the input scale of a fit found by the reference's grid search (g_scale_search: coarse grid, fine grid, parabola vertex;
    threads/05-exl3-harness/harness.py:371-387), for the base plane (folded into su) and the refinement stages;
  * the two-sided schedule (encode_ldlq2, nq_encode.py:206-339): an output metric beside the input Hessian, both block LDL
    factored, units fitted along anti-diagonals from the far corner with the errors of the fitted units carried over by both
    factors, and the reference's inner iterations (accept-if-better tries with the errors fed back inside a chunk);
  * the second plane of the interleaved two-plane level 4 (window code 12) with the first plane frozen (viterbi_ring_given_p3).
  * the low-rank plane (lr_detect, lr_metric, lr_fit; nq_encode.py:507-556): the strongest eigen-directions of the input second
    moment, the metric that leaves them to the plane, and the least-squares coefficients per level.
The reference's encoder depends on exllamav3 1.5.1, which is not available here, so bit parity with it is not claimed;
the tests pin this encoder by brute force on a small trellis, by decode(encode) self-consistency and by the Gaussian
distortion the reference reports for this code (MSE 0.068 at 2 bits, threads/03-nested-trellis-code/REPORT.md:21; base +
one-bit refinement 0.018747, base + two-bit refinement 0.004729, threads/03-nested-trellis-code/exp3_mul1L.log:3-4).
"""
import torch

from .format import Proj, pack_words, proj_sizes

HC = 0x83DCD12D


def codebook(dev="cpu", state_bits=16):
    """value of every trellis state: fp16(A (1024 + bytesum(state * HC)) + B) as fp32 (reference harness.py:272-278)"""
    s = torch.arange(1 << state_bits, dtype=torch.int64, device=dev)
    x = (s * HC) & 0xFFFFFFFF
    bsum = (x & 255) + ((x >> 8) & 255) + ((x >> 16) & 255) + (x >> 24)
    A = torch.tensor([0x1EEE], dtype=torch.int16).view(torch.float16).double().to(dev)
    B = torch.tensor([0xC931 - 65536], dtype=torch.int16).view(torch.float16).double().to(dev)
    return ((1024 + bsum).double() * A + B).half().float()


def viterbi_ring(w, lut, K=2, state_bits=16):
    """w [T, L] targets in Viterbi order -> states int64 [T, L]: the tail-biting path of least squared error through the
    shift-register trellis state_t = ((state_{t-1} << K) | b_t) mod 2^state_bits with values lut[state]."""
    T, L = w.shape
    dev = w.device
    Kr = state_bits - K
    E, Q = 1 << Kr, 1 << K
    e = torch.arange(E, device=dev)
    q = torch.arange(Q, device=dev)
    states = (q[:, None] << Kr) | e[None, :]                     # state with top K bits q and low bits e ("edge")
    prev = states >> K                                           # edge of the predecessor state
    vals = lut[states]
    back = torch.empty((L, T, E), dtype=torch.uint8, device=dev)

    def forward(roll, pre):
        cost = None
        for i in range(L):
            ri = (i + roll) % L
            d = (vals[None] - w[:, ri, None, None]).square()    # [T, Q, E]
            if cost is None:
                c = d if pre is None else torch.where(prev[None] == pre[:, None, None], d, torch.full_like(d, float("inf")))
            else:
                c = d + cost[:, prev]
            cost, arg = c.min(1)
            back[ri] = arg.to(torch.uint8)
        return cost

    def trace(roll, edge, stop_at_zero):
        out = torch.empty((T, L), dtype=torch.int64, device=dev)
        tt = torch.arange(T, device=dev)
        for i in range(L - 1, -1, -1):
            ri = (i + roll) % L
            st = (back[ri][tt, edge].long() << Kr) | edge
            out[:, ri] = st
            edge = st >> K
            if stop_at_zero and ri == 0:
                break
        return out, edge

    c = forward(L // 2, None)
    _, start = trace(L // 2, c.argmin(1), True)                  # edge entering step 0
    forward(0, start)
    idx, _ = trace(0, start, False)                              # the ring closes on `start`
    return idx


def spread8(a):
    """8-bit values -> their bits at the even positions of a 16-bit value (bit i -> bit 2 i)"""
    a = (a | (a << 4)) & 0x0F0F
    a = (a | (a << 2)) & 0x3333
    return (a | (a << 1)) & 0x5555


def viterbi_ring_given_p3(w, a, lut):
    """The second refinement plane of the interleaved two-plane code, with the first one frozen. Stream bit 2 p is P3's bit p
    (given), bit 2 p + 1 is P4's bit p (sought); the state at position p interleaves the 8-bit windows a(p) = P3 bits [p, p + 8)
    and b(p) = P4 bits [p, p + 8): state = spread(a) | spread(b) << 1. What is left to choose is one bit per step with eight steps
    of memory, over a codebook that changes from step to step with a: value(b) = lut[spread(a) | spread(b) << 1].
    w [T, L] targets and a [T, L] P3 windows, both in Viterbi order (b_t = ((b_{t-1} << 1) | new bit) mod 256) -> b int64 [T, L],
    the tail-biting path of least squared error, found as viterbi_ring finds its own (two passes)."""
    T, L = w.shape
    dev = w.device
    E = 128                                                      # low seven bits of b ("edge"); its top bit is the choice
    e = torch.arange(E, device=dev)
    q = torch.arange(2, device=dev)
    states = (q[:, None] << 7) | e[None, :]
    prev = states >> 1
    sb = spread8(states) << 1                                    # P4's share of the 16-bit state
    sa = spread8(a)
    back = torch.empty((L, T, E), dtype=torch.uint8, device=dev)

    def forward(roll, pre):
        cost = None
        for i in range(L):
            ri = (i + roll) % L
            d = (lut[sa[:, ri, None, None] | sb[None]] - w[:, ri, None, None]).square()     # [T, 2, E]
            if cost is None:
                c = d if pre is None else torch.where(prev[None] == pre[:, None, None], d, torch.full_like(d, float("inf")))
            else:
                c = d + cost[:, prev]
            cost, arg = c.min(1)
            back[ri] = arg.to(torch.uint8)
        return cost

    def trace(roll, edge, stop_at_zero):
        out = torch.empty((T, L), dtype=torch.int64, device=dev)
        tt = torch.arange(T, device=dev)
        for i in range(L - 1, -1, -1):
            ri = (i + roll) % L
            st = (back[ri][tt, edge].long() << 7) | edge
            out[:, ri] = st
            edge = st >> 1
            if stop_at_zero and ri == 0:
                break
        return out, edge

    c = forward(L // 2, None)
    _, start = trace(L // 2, c.argmin(1), True)
    forward(0, start)
    return trace(0, start, False)[0]


def ring_index(dev="cpu"):
    """[8, 256]: ring g, position p -> index (column * 16 + row) inside a 16 x 128 unit (reference ref15_spec.py:118-125)"""
    g = torch.arange(8, device=dev)[:, None, None]; t4 = torch.arange(4, device=dev)[None, :, None]
    j = torch.arange(64, device=dev)[None, None, :]
    pp, e = j >> 1, j & 1
    t, r = pp >> 2, pp & 3
    return ((16 * t + 2 * t4 + 8 * (r >> 1) + e) * 16 + g + 8 * (r & 1)).reshape(8, 256)


def hadamard128(dev="cpu"):
    H = torch.ones(1, 1, device=dev)
    while H.shape[0] < 128:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    return H / 128 ** 0.5


def blocked_had(X, dim):
    """orthonormal Hadamard-128 on every 128-block of dimension `dim`"""
    Hm = hadamard128(X.device).to(X.dtype)
    X = X.movedim(dim, -1)
    Y = (X.reshape(*X.shape[:-1], -1, 128) @ Hm).reshape(X.shape)
    return Y.movedim(-1, dim)


def to_rings(M):
    """[N, K] -> [units * 8, 256] in ring position order (unit = strip * C + chunk)"""
    N, K = M.shape
    S, C = N // 16, K // 128
    units = M.reshape(S, 16, C, 128).permute(0, 2, 3, 1).reshape(S * C, 2048)        # [unit, column * 16 + row]
    return units[:, ring_index(M.device).reshape(-1)].reshape(S * C * 8, 256)


def from_rings(R, N, K):
    """inverse of to_rings"""
    S, C = N // 16, K // 128
    U = torch.empty(S * C, 2048, dtype=R.dtype, device=R.device)
    U[:, ring_index(R.device).reshape(-1)] = R.reshape(S * C, 2048)
    return U.reshape(S, C, 128, 16).permute(0, 3, 1, 2).reshape(N, K)


def viterbi_rings(rings, K=2, chunk=64):
    """rings [T, 256] in ring position order -> states int64 [T, 256] in the same order.
    Viterbi step i <-> position p = (-i) mod 256, a permutation that is its own inverse."""
    dev = rings.device
    ip = (-torch.arange(256, device=dev)) % 256
    lut = codebook(dev)
    st = torch.empty(rings.shape, dtype=torch.int64, device=dev)
    for a in range(0, rings.shape[0], chunk):
        st[a:a + chunk] = viterbi_ring(rings[a:a + chunk][:, ip].contiguous(), lut, K)[:, ip]
    return st


def viterbi_rings_given_p3(rings, st3, chunk=256):
    """rings [T, 256] targets and st3 [T, 256] the 16-bit states of the one-bit plane P3, both in ring position order ->
    (b [T, 256]: 8-bit windows of plane P4, st4 [T, 256]: the 16-bit states of the interleaved stream), position order"""
    dev = rings.device
    ip = (-torch.arange(256, device=dev)) % 256
    lut = codebook(dev)
    a = st3 & 0xFF                                               # P3 bits [p, p + 8)
    b = torch.empty(rings.shape, dtype=torch.int64, device=dev)
    for i in range(0, rings.shape[0], chunk):
        b[i:i + chunk] = viterbi_ring_given_p3(rings[i:i + chunk][:, ip].contiguous(), a[i:i + chunk][:, ip].contiguous(), lut)[:, ip]
    return b, spread8(a) | (spread8(b) << 1)


def one_bit_states(bits):
    """ring bits [T, 256] (bit p of a one-bit-per-step stream) -> the 16-bit states [T, 256]: state(p) = bits [p, p + 16), wrapping"""
    idx = (torch.arange(256, device=bits.device)[:, None] + torch.arange(16, device=bits.device)[None]) % 256
    return (bits[:, idx] << torch.arange(16, device=bits.device)).sum(-1)


def lane_records(st, K):
    """ring states [T, 256] (position order) of a K-bits-per-step stream -> record words int64 [T * 4, 2 K] (uint32 values).
    Stream bit K p + b = bit b of state(p): the low K bits of each state are the new bits of its step; lane t4 of a ring
    holds the stream's bits [64 K t4, 64 K (t4 + 1)), so records come out in (unit, ring, lane) order."""
    dev = st.device
    bits = torch.stack([(st >> b) & 1 for b in range(K)], -1).reshape(-1, 256 * K)
    sym = (bits.reshape(-1, 256, K) << torch.arange(K, device=dev)).sum(-1)
    n = 16 // K
    idx = (torch.arange(256, device=dev)[:, None] + torch.arange(n, device=dev)[None]) % 256
    assert torch.equal((sym[:, idx] << (K * torch.arange(n, device=dev))).sum(-1), st), "ring states are not tail-biting"
    return (bits.reshape(-1, 8 * K, 32) << torch.arange(32, device=dev)).sum(-1).reshape(-1, 2 * K)


def prepare(W, seed=0):
    """signs, scales and rotations: W [N, K] -> (su fp16 [K], sv fp16 [N], target fp32 [N, K]) with
    W = D(sv) B_N target B_K D(su) up to the fp16 rounding of the scales, B the 128-blocked orthonormal Hadamard"""
    N, K = W.shape
    assert N % 128 == 0 and K % 128 == 0
    dev = W.device
    g = torch.Generator().manual_seed(seed)
    sgn_u = (torch.randint(0, 2, (K,), generator=g) * 2 - 1).to(dev).double()
    sgn_v = (torch.randint(0, 2, (N,), generator=g) * 2 - 1).to(dev).double()
    Wd = W.double()
    c_in = Wd.square().mean(0).sqrt().clamp_min(1e-12)           # per input channel
    W1 = Wd / c_in
    r_out = W1.square().mean(1).sqrt().clamp_min(1e-12)          # per output channel
    su = (sgn_u * c_in).half(); sv = (sgn_v * r_out).half()
    # the decoder applies the fp16-rounded scales, so the target is built from them
    Wn = Wd / su.double()[None, :] / sv.double()[:, None]
    return su, sv, blocked_had(blocked_had(Wn, 1), 0).float()    # B_N Wn B_K


def signed32(w):
    """uint32 values held in int64 -> int32 with the same bits"""
    return torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)


def encode_level2(W, seed=0, chunk=64, g_scale=False):
    """W [N, K] float (N % 16 == 0, K % 128 == 0; N % 128 == 0 for the output rotation) ->
    dict(base int32 [nrec*4], su fp16 [K], sv fp16 [N], states int64 [units, 8, 256] (ring position order), Q fp32 [N, K])
    with  W ~= D(sv) B_N Q B_K D(su)  and Q the matrix the decoder reproduces bit for bit from `base`."""
    N, K = W.shape
    su, sv, target = prepare(W, seed)
    if g_scale:                                                  # the fit's input scale from the grid search instead of 1
        su, target, _ = apply_g_scale(su, target)
    st = viterbi_rings(to_rings(target), 2, chunk)
    base = signed32(lane_records(st, 2).reshape(-1))             # record = (unit, lane 4 g + t4): 4 words
    Q = from_rings(codebook(W.device)[st], N, K)                 # decoded values
    return dict(base=base, su=su, sv=sv, states=st.reshape(-1, 8, 256), Q=Q, target=target)


# ----------------------------------------------------------------------------------------------------------------------
# refinement planes (levels 3 and 4)
A_ = float(torch.tensor([0x1EEE], dtype=torch.int16).view(torch.float16))
K0 = 1024.0 * A_ + float(torch.tensor([0xC931 - 65536], dtype=torch.int16).view(torch.float16))
RES_SCALE = {1: 1.1, 2: 1.0}     # best input scale of the refinement stage on Gaussian data (reference exp3_mul1L.log:3-4)
RES_SCALE_GIVEN_P3 = 1.2         # the same for the interleaved second plane (one free bit per step, eight steps of memory); found here


def hash_sum(st):
    """byte sum S of state * HC mod 2^32 (reference sm120/ref15_spec.py:64-70)"""
    x = (st * HC) & 0xFFFFFFFF
    return (x & 255) + ((x >> 8) & 255) + ((x >> 16) & 255) + (x >> 24)


def round_f16(v):
    """float64 -> fp16 with one rounding. Going through fp32 rounds twice; rounding to odd at 24 bits first (truncate, then
    set the last bit if anything was cut off) makes the second rounding see on which side of a tie the value lies."""
    f = v.float()
    cut = f.double() != v
    bits = f.view(torch.int32) - (f.double().abs() > v.abs()).to(torch.int32)      # one step towards zero where fp32 rounded away
    return (bits | cut.to(torch.int32)).view(torch.float32).half()


_FOLD = None


def fold_table():
    """fp16 constants (A', C) of the integer fold for every block word, as fp32 [256, 258, 2] indexed by (Mb, N): fp32
    operations in the spec's order, none contracted (reference sm120/ref15_spec.py:79-86). Built once on the CPU, whose
    fp32 division and products are correctly rounded."""
    global _FOLD
    if _FOLD is None:
        Mb = torch.arange(256, dtype=torch.float32).clamp_min(1)[:, None]
        N = torch.arange(258, dtype=torch.float32)[None, :]
        rcp = torch.ones(1) / Mb
        Ah = (torch.tensor(1.732421875) * rcp).half()
        t = (N * rcp) * torch.tensor(K0, dtype=torch.float32)
        t = t + torch.tensor(K0, dtype=torch.float32)
        Ch = (t - torch.tensor(1024.0) * Ah.float()).half()
        _FOLD = torch.stack([Ah.float().expand(256, 258), Ch.float()], -1).contiguous()
    return _FOLD


def fold_value(Sb, Sr, Mb, N):
    """levels 3 / 4: F = (Mb Sb + N Sr + 128) >> 8, value = fp16(A' (1024 + F) + C) with one rounding
    (reference sm120/ref15_spec.py:87-90, sm120/moe.py:128-134). Sb, Sr int64 [U, ...]; Mb, N int64 [U]. -> fp16"""
    shape = (-1,) + (1,) * (Sb.dim() - 1)
    Mb_, N_ = Mb.view(shape), N.view(shape)
    c = fold_table().to(Sb.device)[Mb, N].double()
    F = (Mb_ * Sb + N_ * Sr + 128) >> 8
    return round_f16(c[:, 0].view(shape) * (1024 + F).double() + c[:, 1].view(shape))


def block_word_candidates(delta):
    """[U] step sizes -> (Mb, N) int64 [U, 12]: the largest-Mb rational N / Mb nearest to delta with Mb + N <= 257,
    Mb <= 255, and its neighbours Mb - 0..3, N - 1..N + 1; a candidate outside the valid range is replaced by the first
    (reference nq_decode.py:158-163, nq_encode.py:186-198)."""
    d = delta.double().clamp_min(0)
    Mb0 = torch.floor(257 / (1 + d)).clamp(1, 255).long()
    N0 = torch.minimum(torch.round(d * Mb0).long(), 257 - Mb0)
    Ms, Ns = [], []
    for dm in range(4):
        Mb = (Mb0 - dm).clamp(1, 255)
        Nr = torch.round(d * Mb).long()
        for dn in (-1, 0, 1):
            Ms.append(Mb); Ns.append(Nr + dn)
    Mb, N = torch.stack(Ms, 1), torch.stack(Ns, 1)
    ok = (N >= 0) & (N <= 255) & (Mb + N <= 257)
    return torch.where(ok, Mb, Mb0[:, None]), torch.where(ok, N, N0[:, None].clamp_max(255))


def base_rings(rings, chunk=64, var=False):
    """base plane of rings [T, 256] (ring position order) -> (states int64 [T, 256], sign fp32 [T, 1]): with var, each ring is
    fitted as it is and negated, and keeps the better of the two by its squared error (the reference's 'sign' base variant,
    nq_encode.py:87-113; the decoder negates the ring's values, table words 12 / 13)"""
    T = rings.shape[0]
    st = viterbi_rings(torch.cat([rings, -rings]) if var else rings, 2, chunk)
    sign = torch.ones(T, 1, device=rings.device)
    if var:
        lut = codebook(rings.device)
        e_pos = (lut[st[:T]] - rings).square().sum(1)
        e_neg = (lut[st[T:]] + rings).square().sum(1)
        neg = e_neg < e_pos
        st = torch.where(neg[:, None], st[T:], st[:T])
        sign[neg] = -1.0
    return st, sign


def encode_residual(target, st_base, K, chunk=64, scale=None, cost=None, sign=None, p3_states=None, states=None):
    """One refinement stage on the frozen base plane. target fp32 [U, 8, 256] and st_base int64 [U, 8, 256] in ring position
    order, K = 1 or 2 bits per weight -> dict(states [U, 8, 256], Mb [U], N [U], Q fp32 [U, 8, 256], delta [U]).
    cost: error fp64 [U, 8, 256] -> [U], what the block-word search minimises (default: the squared error).
    sign [U, 8, 1] (+-1): rings whose decoded values are negated, base and refinement alike.
    p3_states [U, 8, 256] (with K = 2): the 16-bit states of an already fitted one-bit plane P3, which stays as it is; the stage
    then fits plane P4 of the interleaved two-plane code (window code 12) and also returns its ring bits as `p4_bits`.
    states [U, 8, 256]: the refinement plane's states are these (no search); only the block word is fitted."""
    U = target.shape[0]
    dev = target.device
    lut = codebook(dev)
    cost = cost or (lambda E: E.square().sum((1, 2)))
    sign = torch.ones(U, 8, 1, device=dev) if sign is None else sign
    Sb = hash_sum(st_base)
    r = (target * sign).double() - lut[st_base].double()         # in the ring's own orientation
    rms = r.square().mean((1, 2)).sqrt().clamp_min(1e-12)
    p4_bits = None
    if states is not None:
        st = states
    elif p3_states is None:
        s0 = rms / (RES_SCALE[K] if scale is None else scale)
        st = viterbi_rings((r / s0[:, None, None]).float().reshape(U * 8, 256), K, chunk).reshape(U, 8, 256)
    else:
        assert K == 2
        s0 = rms / (RES_SCALE_GIVEN_P3 if scale is None else scale)
        b, st = viterbi_rings_given_p3((r / s0[:, None, None]).float().reshape(U * 8, 256), p3_states.reshape(U * 8, 256))
        st, p4_bits = st.reshape(U, 8, 256), (b & 1).reshape(U, 8, 256)
    Sr = hash_sum(st)
    a = A_ * Sr.double() + K0                                    # unrounded value of the refinement code
    delta = ((a * r).sum((1, 2)) / a.square().sum((1, 2)).clamp_min(1e-30)).clamp_min(0)
    Mbs, Ns = block_word_candidates(delta)
    best = None
    for ci in range(Mbs.shape[1]):
        q = fold_value(Sb, Sr, Mbs[:, ci], Ns[:, ci]).float() * sign
        c = cost((target - q).double())
        if best is None:
            best = dict(c=c, Q=q, Mb=Mbs[:, ci].clone(), N=Ns[:, ci].clone())
        else:
            w = c < best["c"]
            best["c"] = torch.where(w, c, best["c"]); best["Q"][w] = q[w]
            best["Mb"][w] = Mbs[w, ci]; best["N"][w] = Ns[w, ci]
    return dict(states=st, Mb=best["Mb"], N=best["N"], Q=best["Q"], delta=delta, p4_bits=p4_bits)


def pack_planes(r, N, K, st2, fits, sign=None):
    """ring states of the base plane [units, 8, 256], the refinement fits {3: e3, 4: e4} (encode_residual's dicts over all
    units) and the ring signs [units, 8, 1] (None: all +1) -> r gains base, states, Q and p3 / d3 / Q3 / states3,
    p4 / d4 / Q4 / states4, and with signs var (uint8 per unit, bit g = ring g negated)"""
    dev = st2.device
    r["states"] = st2
    r["base"] = signed32(lane_records(st2.reshape(-1, 256), 2).reshape(-1))
    q2 = codebook(dev)[st2]
    r["var"] = None
    if sign is not None:
        q2 = q2 * sign
        r["var"] = ((sign.reshape(-1, 8) < 0).long() << torch.arange(8, device=dev)).sum(1).to(torch.uint8)
    r["Q"] = from_rings(q2.reshape(-1, 256), N, K)
    for lvl, e in fits.items():
        if lvl == "4n":                                          # plane P4 of the interleaved two-plane level 4: 64-bit records of its own
            r["p4n"] = pack_words(lane_records(one_bit_states(e["p4_bits"].reshape(-1, 256)), 1), 64)
            r["d4n"] = signed32(e["Mb"] | (e["N"] << 8))
            r["Q4n"] = from_rings(e["Q"].reshape(-1, 256), N, K)
            r["states4n"] = e["states"]
            continue
        bpw = lvl - 2
        r["p%d" % lvl] = pack_words(lane_records(e["states"].reshape(-1, 256), bpw), 64 * bpw)
        r["d%d" % lvl] = signed32(e["Mb"] | (e["N"] << 8))
        r["Q%d" % lvl] = from_rings(e["Q"].reshape(-1, 256), N, K)
        r["states%d" % lvl] = e["states"]
    return r


def encode_nested(W, seed=0, chunk=64, var=False, interleave=False, share4=0.0):
    """encode_level2 plus the two refinement planes, each fitted to the residual of the same frozen base plane:
    p3 / d3 (one bit per weight, 64-bit records; level 3 = base + P3) and p4 / d4 (two bits per weight, 128-bit records of
    window code 0; level 4 = base + the wide plane). Adds p3, d3, Q3, p4, d4, Q4 (Q3 / Q4 fp32 [N, K]: the matrices the
    decoder reproduces bit for bit at levels 3 / 4) to encode_level2's dict. var: also fit every ring negated and keep the
    better orientation (adds the sign plane `var`).
    interleave: also the strictly nested two-plane level 4 of window code 12 -- P3 stays as level 3 fitted it and a second
    one-bit plane P4 is fitted so that base + the bitwise interleave of P3 and P4 is as close as one more bit per weight gets
    it: adds p4n, d4n, Q4n (a promotion 2 -> 3 -> 4 then uploads P3 + d3, then P4 + d4n). Both levels read one hashed window
    per weight, so the bits that level 3 chose carry nothing for level 4's code: with P3 frozen everywhere, level 4 is a fresh
    one-bit fit with half the memory, no better than level 3 (N(0,1): 0.0209 against 0.0186). share4 in [0, 1] trades the levels
    against each other unit by unit: that share of the units (largest base residual first) gets both planes from one two-bit fit
    -- P3 = the low bit, P4 = the high bit of every step, so level 4 is the wide plane's fit there -- while level 3 in those
    units falls back to about the base plane (its block word is fitted to bits not chosen for it and comes out near N = 0)."""
    N, K = W.shape
    su, sv, target = prepare(W, seed)
    tr = to_rings(target).reshape(-1, 8, 256)
    st2, sign = base_rings(tr.reshape(-1, 256), chunk, var)
    st2, sign = st2.reshape(-1, 8, 256), sign.reshape(-1, 8, 1)
    fits = {lvl: encode_residual(tr, st2, lvl - 2, chunk, sign=sign) for lvl in (3, 4)}
    if interleave:
        fits["4n"] = encode_residual(tr, st2, 2, chunk, sign=sign, p3_states=fits[3]["states"])
        nj = int(round(share4 * tr.shape[0]))
        if nj:
            resid = (tr * sign - codebook(tr.device)[st2]).square().sum((1, 2))
            ju = torch.argsort(resid, descending=True)[:nj]
            wide = fits[4]["states"][ju]                         # two bits per step: bit 0 of each state is P3's, bit 1 is P4's
            st3 = one_bit_states((wide & 1).reshape(-1, 256)).reshape(nj, 8, 256)
            e3 = encode_residual(tr[ju], st2[ju], 1, chunk, sign=sign[ju], states=st3)
            for k in ("states", "Mb", "N", "Q"):
                fits[3][k][ju] = e3[k]
                fits["4n"][k][ju] = fits[4][k][ju]
            fits["4n"]["p4_bits"][ju] = (wide >> 1) & 1
    return pack_planes(dict(su=su, sv=sv, target=target), N, K, st2, fits, sign if var else None)


# ----------------------------------------------------------------------------------------------------------------------
# Hessian-aware fit: block LDL feedback (LDLQ) with one error state per level
def block_ldl(H, b=128):
    """H = L D L^T with L unit block lower triangular (identity diagonal blocks of size b) and D block diagonal:
    from the Cholesky factor C, L = C diag(C_ii)^-1 and D_i = C_ii C_ii^T (reference nq_encode.py:115-132).
    -> (L [n, n], D [n / b, b, b]), float64"""
    n = H.shape[0]
    m = n // b
    C = torch.linalg.cholesky(H.double().cpu())                  # factorised on the host: seconds at n = 6144, and no device solver needed
    Cd = torch.stack([C[i * b:(i + 1) * b, i * b:(i + 1) * b] for i in range(m)])
    L = torch.cat([C[:, i * b:(i + 1) * b] @ torch.linalg.inv(Cd[i]) for i in range(m)], 1)
    return L.to(H.device), (Cd @ Cd.transpose(1, 2)).to(H.device)


def rotated_hessian(H, su, sigma=0.01):
    """second moment of the activations the quantised matrix multiplies: y = D(sv) B Q (B D(su) x), so
    H' = B D(su) H D(su) B; then sigma * mean(diag) on the diagonal (reference nq_encode.py:141-147, which rotates with the
    signs only and folds the scale into the weights instead)"""
    Hs = H.double() * su.double()[:, None] * su.double()[None, :]
    Hr = blocked_had(blocked_had(Hs, 0), 1)
    return Hr + sigma * Hr.diagonal().mean() * torch.eye(H.shape[0], dtype=torch.float64, device=H.device)


def proxy_loss(Q, target, Hr):
    """tr((Q - T) H' (Q - T)^T) / tr(T H' T^T): the expected squared output error relative to the output's energy"""
    E = Q.double() - target.double()
    return float(((E @ Hr) * E).sum() / ((target.double() @ Hr) * target.double()).sum())


def encode_ldlq(W, H, seed=0, chunk=64, lam=0.3, sigma=0.01, var=False):
    """encode_nested for a layer whose input second moment H [K, K] is known: the 128-column chunks are fitted from the last
    to the first, and each chunk's target is the weight plus the errors of the chunks already fitted, carried over by the
    block LDL factor of H', T_a = W_a + sum_{b > a} E_b L[b, a] (reference nq_encode.py:206-339, its one-sided schedule).
    Then tr(E H' E^T) = sum_a tr(eta_a D_a eta_a^T) with eta_a = T_a - Q_a the chunk's own fitting error. One error state
    per level (the reference keeps two, for levels 2 and 4): the base plane is fitted to (1 - lam) T_2 + lam T_4, the refinement
    planes to T_3 - Q_2 and T_4 - Q_2, their block words costed with D_a.
    Adds Hr, D (the block diagonal factor), eta = {2, 3, 4: fp64 [N, K]} and proxy = {2, 3, 4: proxy_loss} to encode_nested's dict."""
    N, K = W.shape
    S, C = N // 16, K // 128
    dev = W.device
    su, sv, target = prepare(W, seed)
    Hr = rotated_hessian(H.to(dev), su, sigma)
    L, D = block_ldl(Hr)
    Tg = target.double()
    err = {lvl: torch.zeros(N, K, dtype=torch.float64, device=dev) for lvl in (2, 3, 4)}
    eta = {lvl: torch.zeros(N, K, dtype=torch.float64, device=dev) for lvl in (2, 3, 4)}
    st2 = torch.empty(S, C, 8, 256, dtype=torch.int64, device=dev)
    sign = torch.ones(S, C, 8, 1, device=dev)
    fit = {lvl: dict(states=torch.empty(S, C, 8, 256, dtype=torch.int64, device=dev), Q=torch.empty(S, C, 8, 256, device=dev),
                     Mb=torch.empty(S, C, dtype=torch.int64, device=dev), N=torch.empty(S, C, dtype=torch.int64, device=dev))
           for lvl in (3, 4)}
    rings = lambda M: to_rings(M.float()).reshape(S, 8, 256)     # a chunk [N, 128] is one unit per strip
    for a in range(C - 1, -1, -1):
        cols = slice(a * 128, (a + 1) * 128)
        T = {lvl: Tg[:, cols] + err[lvl] @ L[:, cols] for lvl in (2, 3, 4)}      # later chunks only: the others' errors are still zero
        tb = (1 - lam) * T[2] + lam * T[4]
        sa, sg = base_rings(rings(tb).reshape(-1, 256), chunk, var)
        sa, sg = sa.reshape(S, 8, 256), sg.reshape(S, 8, 1)
        st2[:, a] = sa; sign[:, a] = sg
        q2 = from_rings((codebook(dev)[sa] * sg).reshape(-1, 256), N, 128).double()
        err[2][:, cols], eta[2][:, cols] = Tg[:, cols] - q2, T[2] - q2
        Da = D[a]

        def cost(E):                                             # ring order -> [strip, 16 rows, 128 columns]
            Eu = from_rings(E.reshape(-1, 256), N, 128).reshape(S, 16, 128)
            return ((Eu @ Da) * Eu).sum((1, 2))
        for lvl in (3, 4):
            e = encode_residual(rings(T[lvl]), sa, lvl - 2, chunk, cost=cost, sign=sg)
            for k in ("states", "Q", "Mb", "N"):
                fit[lvl][k][:, a] = e[k]
            q = from_rings(e["Q"].reshape(-1, 256), N, 128).double()
            err[lvl][:, cols], eta[lvl][:, cols] = Tg[:, cols] - q, T[lvl] - q
    flat = {lvl: dict(states=f["states"].reshape(-1, 8, 256), Q=f["Q"].reshape(-1, 8, 256), Mb=f["Mb"].reshape(-1), N=f["N"].reshape(-1))
            for lvl, f in fit.items()}
    r = pack_planes(dict(su=su, sv=sv, target=target, Hr=Hr, D=D, eta=eta), N, K, st2.reshape(-1, 8, 256), flat,
                    sign.reshape(-1, 8, 1) if var else None)
    r["proxy"] = {2: proxy_loss(r["Q"], target, Hr), 3: proxy_loss(r["Q3"], target, Hr), 4: proxy_loss(r["Q4"], target, Hr)}
    return r


# ----------------------------------------------------------------------------------------------------------------------
# input scale of a trellis fit: grid search
CB_RMS = 1.24371088              # rms of the codebook's 65536 values (reference nq_encode.py:32)


def g_scale_search(rings, K, quantize=None):
    """The scale s by which rings [T, 256] (Viterbi order does not matter here) are multiplied before the fit so that
    mean((q(s x) / s - x)^2) is least: a coarse grid 0.1, 0.3 .. 1.9 on every third ring, five points 0.075 apart around the best
    of them on all rings, then the vertex of the parabola through the best point and its neighbours, at most half a step away
    (reference threads/05-exl3-harness/harness.py:371-387, after exllamav3's g_scale_search_batch). quantize(x, K) -> values of
    the fitted code (default: the tail-biting Viterbi over the mul1 codebook). -> (scale >= 0.01, mse at the best grid point)"""
    if quantize is None:
        lut = codebook(rings.device)
        quantize = lambda x, k: lut[viterbi_ring(x, lut, k)]

    def mse(x, s):
        return float((quantize(x * s, K) / s - x).square().mean())
    coarse = [0.1 + 0.2 * i for i in range(10)]
    third = rings[::3]
    c = min(coarse, key=lambda v: mse(third, v))
    step = 0.075
    fine = [c + step * (i - 2) for i in range(5)]
    m = [mse(rings, v) if v > 0 else float("inf") for v in fine]
    best = min(range(5), key=lambda i: m[i])
    shift = 0.0
    if 0 < best < 4 and m[best - 1] < float("inf"):
        bend = m[best - 1] - 2 * m[best] + m[best + 1]
        if bend > 0:
            shift = max(-0.5, min(0.5, 0.5 * (m[best - 1] - m[best + 1]) / bend))
    return max(fine[best] + shift * step, 0.01), m[best]


def sample_rings(rings, limit=384):
    """an evenly spaced sample of at most `limit` rings (the reference samples tiles with exllamav3's sample_scale_tiles, which is
    not available here)"""
    T = rings.shape[0]
    return rings if T <= limit else rings[torch.linspace(0, T - 1, limit, device=rings.device).round().long()]


def apply_g_scale(su, target, K=2):
    """the searched scale folded into the fit: the code is fitted to gs * target and the input scale vector carries 1 / gs, so
    that W ~= D(sv) B Q B D(su) still holds (reference nq_encode.py:175-177: weight *= gs; su /= gs). The target is rebuilt from
    the fp16-rounded su so that it is exactly what the decoder's scales imply. -> (su fp16, target fp32, gs)"""
    gs, _ = g_scale_search(sample_rings(to_rings(target)), K)
    su2 = (su.double() / gs).half()
    ratio = (su.double() / su2.double()).float()                  # = gs up to the fp16 rounding of every channel's scale
    return su2, blocked_had(blocked_had(target, 1) * ratio[None, :], 1), gs


# ----------------------------------------------------------------------------------------------------------------------
# two-sided LDLQ: an output metric beside the input Hessian, units fitted along anti-diagonals, inner iterations
def rotated_out_metric(G, sv, sigma=0.03):
    """second moment of what the layer's output error is weighed with, in the rotated output basis: the output is
    y = D(sv) B (Q xr), so an error E of Q costs e^T G e with e = D(sv) B E xr, i.e. the metric on the rotated rows is
    B D(sv) G D(sv) B; then sigma * mean(diag) on the diagonal (the reference builds this with exllamav3's prepare_H_out from
    G and sv, nq_encode.py:178-183; that function is not available here and this is the form the layer math gives)"""
    Gs = G.double() * sv.double()[:, None] * sv.double()[None, :]
    Gr = blocked_had(blocked_had(Gs, 0), 1)
    return Gr + sigma * Gr.diagonal().mean() * torch.eye(G.shape[0], dtype=torch.float64, device=G.device)


def encode_ldlq2(W, H, G, seed=0, chunk=64, lam=0.3, sigma=0.01, sigma_out=0.03, var=False, inner=0, beta=1.0, g_scale=False):
    """encode_ldlq with a metric on both sides (reference nq_encode.py:206-339, its two-sided schedule): the expected cost of an
    error E = T - Q of the rotated weight is tr(Go E H' E^T), Go [N, N] the rotated output metric (rotated_out_metric) and H'
    [K, K] the rotated input Hessian. With H' = Lk Din Lk^T (unit block lower, blocks of 128 columns = a chunk) and
    Go = Ln Dout Ln^T (blocks of 16 rows = a strip) the cost is the sum over the units (strip c, chunk a) of
    tr(Dout_c eta Din_a eta^T), eta_ca = block (c, a) of Ln^T E Lk = E_ca + the errors of the units with c' >= c and a' >= a
    carried over by both factors. So the units are fitted along anti-diagonals from the far corner (largest c + a first), each
    to its weight plus what the already fitted units pass on, T_ca = W_ca + (Ln^T E Lk)_ca over the fitted units only, and its
    own fitting error is eta_ca. One error state per level, as in encode_ldlq.
    inner > 0 (reference :249-258,:271-302): that many further tries per stage inside a unit's chunk. Din_a itself factors
    with blocks of 16 columns, Din_a = L16 D16 L16^T; a try refits the stage to its target plus beta * (target - the previous
    try's values) (L16 - I), the errors of the later 16-column groups fed to the earlier ones, and is kept for the units whose
    local cost tr(Dout eta Din eta^T) it lowers, so the cost never rises.
    g_scale: search the input scale of the base fit (apply_g_scale) and of the refinement stages (on the first anti-diagonal's
    residuals) instead of the constants 1 and RES_SCALE.
    Adds Hr, Go, Din, Dout, eta = {2, 3, 4: fp64 [N, K]}, proxy = {2, 3, 4} and, with inner, n_inner_kept to encode_nested's dict."""
    N, K = W.shape
    S, C = N // 16, K // 128
    dev = W.device
    su, sv, target = prepare(W, seed)
    gs = 1.0
    if g_scale:
        su, target, gs = apply_g_scale(su, target)
    Hr = rotated_hessian(H.to(dev), su, sigma)
    Go = rotated_out_metric(G.to(dev), sv, sigma_out)
    Lk, Din = block_ldl(Hr, 128)
    Ln, Dout = block_ldl(Go, 16)
    U16 = None
    if inner:
        U16 = torch.stack([block_ldl(Din[a], 16)[0] for a in range(C)]) - torch.eye(128, dtype=torch.float64, device=dev)
    Tg = target.double()
    levels = (2, 3, 4)
    err = {l: torch.zeros(N, K, dtype=torch.float64, device=dev) for l in levels}     # W - Q of the fitted units
    eta = {l: torch.zeros(N, K, dtype=torch.float64, device=dev) for l in levels}
    st2 = torch.empty(S, C, 8, 256, dtype=torch.int64, device=dev)
    sign = torch.ones(S, C, 8, 1, device=dev)
    fit = {l: dict(states=torch.empty(S, C, 8, 256, dtype=torch.int64, device=dev), Q=torch.empty(S, C, 8, 256, device=dev),
                   Mb=torch.empty(S, C, dtype=torch.int64, device=dev), N=torch.empty(S, C, dtype=torch.int64, device=dev)) for l in (3, 4)}
    Q2u = torch.empty(S, C, 16, 128, device=dev)
    lut = codebook(dev)
    kept = 0
    res_scale = dict(RES_SCALE)

    def units_of(M, cs, as_):                                   # [N, K] -> [T, 16, 128]
        return M.reshape(S, 16, C, 128).permute(0, 2, 1, 3)[cs, as_]

    def rings_of(U):                                            # [T, 16, 128] -> [T, 8, 256] ring position order
        flat = U.permute(0, 2, 1).reshape(U.shape[0], 2048)     # [unit, column * 16 + row]
        return flat[:, ring_index(dev).reshape(-1)].reshape(-1, 8, 256)

    def unit_of_rings(R):                                       # inverse of rings_of
        flat = torch.empty(R.shape[0], 2048, dtype=R.dtype, device=dev)
        flat[:, ring_index(dev).reshape(-1)] = R.reshape(R.shape[0], 2048)
        return flat.reshape(-1, 128, 16).permute(0, 2, 1)

    for s in range(S + C - 2, -1, -1):
        as_ = torch.arange(max(0, s - (S - 1)), min(C - 1, s) + 1, device=dev)
        cs = s - as_
        Tn = len(as_)
        Da, Do = Din[as_], Dout[cs]
        lcost = lambda E: ((Do @ E.double() @ Da) * E.double()).sum((1, 2))            # tr(Dout eta Din eta^T) per unit
        Tl = {l: units_of(Tg + Ln.T @ err[l] @ Lk, cs, as_) for l in levels}           # unfitted units contribute nothing: their err is 0

        def fit_base(tb):
            sa, sg = base_rings(rings_of(tb.float()).reshape(-1, 256), chunk, var)
            sa, sg = sa.reshape(Tn, 8, 256), sg.reshape(Tn, 8, 1)
            return sa, sg, unit_of_rings(lut[sa] * sg)
        tb = (1 - lam) * Tl[2] + lam * Tl[4]
        sa, sg, q2 = fit_base(tb)
        if inner:
            c_best, cur = lcost(tb - q2), q2
            for _ in range(inner):
                na, ng, nq = fit_base(tb + beta * (tb - cur.double()) @ U16[as_])
                c = lcost(tb - nq); w = c < c_best
                sa[w], sg[w], q2[w] = na[w], ng[w], nq[w]
                c_best = torch.where(w, c, c_best); cur = nq; kept += int(w.sum())
        st2[cs, as_], sign[cs, as_], Q2u[cs, as_] = sa, sg, q2
        Wu = units_of(Tg, cs, as_)

        def put(M, U):                                          # write units back into [N, K]
            M.reshape(S, 16, C, 128).permute(0, 2, 1, 3)[cs, as_] = U
        put(err[2], Wu - q2.double()); put(eta[2], Tl[2] - q2.double())
        cost = lambda E: lcost(unit_of_rings(E))                  # encode_residual hands over errors in ring order
        for l in (3, 4):
            Kb = l - 2
            if g_scale and s == S + C - 2:                        # first units: search the refinement stage's input scale once
                rr = (rings_of(Tl[l].float()) * sg - lut[sa]).reshape(-1, 256)
                rr = rr / rr.square().mean(1, keepdim=True).sqrt().clamp_min(1e-12)
                res_scale[Kb] = g_scale_search(sample_rings(rr), Kb)[0]
            tr_l = rings_of(Tl[l].float())
            e = encode_residual(tr_l, sa, Kb, chunk, cost=cost, sign=sg, scale=res_scale[Kb])
            if inner:
                c_best = cost((tr_l - e["Q"]).double()); cur = unit_of_rings(e["Q"])
                for _ in range(inner):
                    t_try = Tl[l] + beta * (Tl[l] - cur.double()) @ U16[as_]
                    n = encode_residual(rings_of(t_try.float()), sa, Kb, chunk, cost=cost, sign=sg, scale=res_scale[Kb])
                    # the try's block word was fitted to the shifted target: cost it, and refit the word, against the real one
                    n = encode_residual(tr_l, sa, Kb, chunk, cost=cost, sign=sg, states=n["states"])
                    c = cost((tr_l - n["Q"]).double()); w = c < c_best
                    for k in ("states", "Q", "Mb", "N"):
                        e[k][w] = n[k][w]
                    c_best = torch.where(w, c, c_best); cur = unit_of_rings(n["Q"]); kept += int(w.sum())
            for k in ("states", "Q", "Mb", "N"):
                fit[l][k][cs, as_] = e[k]
            q = unit_of_rings(e["Q"]).double()
            put(err[l], Wu - q); put(eta[l], Tl[l] - q)
    flat = {l: dict(states=f["states"].reshape(-1, 8, 256), Q=f["Q"].reshape(-1, 8, 256), Mb=f["Mb"].reshape(-1), N=f["N"].reshape(-1))
            for l, f in fit.items()}
    r = pack_planes(dict(su=su, sv=sv, target=target, Hr=Hr, Go=Go, Din=Din, Dout=Dout, eta=eta, gs=gs, res_scale=res_scale, n_inner_kept=kept),
                    N, K, st2.reshape(-1, 8, 256), flat, sign.reshape(-1, 8, 1) if var else None)
    r["proxy"] = {2: proxy_loss2(r["Q"], target, Hr, Go), 3: proxy_loss2(r["Q3"], target, Hr, Go), 4: proxy_loss2(r["Q4"], target, Hr, Go)}
    return r


def proxy_loss2(Q, target, Hr, Go):
    """tr(Go E H' E^T) / tr(Go T H' T^T) with E = Q - T: the expected weighted output error relative to the output's"""
    E, T = Q.double() - target.double(), target.double()
    return float(((Go @ E @ Hr) * E).sum() / ((Go @ T @ Hr) * T).sum())


# ----------------------------------------------------------------------------------------------------------------------
# Low-rank plane: fp16 corrections U^T V on the un-rotated input side, for the few input directions that carry most of the
# activations' energy (table words 14 .. 17; the layer adds (x V^T) U2 at every level and (x V^T) U4 at level 4)

LR_TAU, LR_RMAX = 0.05, 4        # the reference's production setting (nq_encode.py:500-501); its sparsified variant is off there


def dense_from_rotated(Q, su, sv):
    """the dense weight a rotated-domain matrix Q [N, K] stands for: D(sv) B_N Q B_K D(su), fp32"""
    return (blocked_had(blocked_had(Q.double(), 1), 0) * su.double()[None, :] * sv.double()[:, None]).float()


def lr_detect(H, tau=LR_TAU, rmax=LR_RMAX):
    """V fp16 [r, K], r <= rmax: the unit eigenvectors of the input second moment H [K, K] whose eigenvalue is at least tau of
    the trace, largest first (reference nq_encode.py:507-520 without its sparsification step, which production leaves off)"""
    w, Q = torch.linalg.eigh(H.double())
    w, Q = w.flip(0), Q.flip(1)
    share = w / w.clamp_min(0).sum()
    r = int((share[:rmax] >= tau).sum())
    return Q[:, :r].T.contiguous().half()


def lr_metric(H, V):
    """the input metric for the trellis fit when the error inside span(V) is corrected afterwards by the low-rank plane:
    (I - P) H (I - P) + m P with P the projector on span(V) and m the mean diagonal of the first term, which keeps the metric
    positive definite without asking the fit for anything inside the span (reference nq_encode.py:527-537)"""
    if V.shape[0] == 0:
        return H
    Vd = V.to(H.device).double()
    P = Vd.T @ torch.linalg.solve(Vd @ Vd.T, Vd)
    R = torch.eye(H.shape[0], dtype=torch.float64, device=H.device) - P
    Hp = R @ H.double() @ R
    return (Hp + Hp.diagonal().mean() * P).to(H.dtype)


def lr_fit(W, dense2, dense4, V):
    """least-squares coefficients of the low-rank plane on the decoded levels (reference nq_encode.py:540-556): U2 fp16 [r, N]
    minimises |W - dense2 - U2^T V| over matrices of that form (normal equations (V V^T) U = V E^T), U4 does the same for what
    level 4 leaves once the U2 term has been added. -> (U2, U4, dense2 + U2^T V, dense4 + (U2 + U4)^T V); the last two, fp32
    [N, K], are what the layer multiplies at levels 2 and 4 (both terms use the fp16-rounded coefficients)."""
    Vd = V.to(W.device).double()
    gram = Vd @ Vd.T

    def coefficients(err):
        return torch.linalg.solve(gram, Vd @ err.double().T).half()
    term = lambda U: (U.double().T @ Vd).float()
    Wf = W.float()
    U2 = coefficients(Wf - dense2)
    with2 = dense2 + term(U2)
    base4 = dense4 + term(U2)
    U4 = coefficients(Wf - base4)
    return U2, U4, with2, base4 + term(U4)


class EncodedProj(Proj):
    """a Proj (nestquant_amd.format) holding encoded planes: the level-2 base plane and, when given, the refinement planes
    p3 / d3 (level 3, the one-bit nested plane), p4 / d4 (level 4, wide plane of window code 0) and the sign plane var"""

    def __init__(s, N, K, base, p3=None, d3=None, p4=None, d4=None, var=None, p4n=None, d4n=None):
        """p4n / d4n: plane P4 and the block words of the nested two-plane level 4; with them the projection is `nested` (its
        level-4 row then points at P3 followed by P4 in one buffer, `slot`, read with the expert's l4code)"""
        s.z = proj_sizes(N, K)
        s.N, s.K, s.rk, s.bk, s.nested = N, K, 0, 0, p4n is not None
        s.base = base
        zero = lambda: torch.zeros(1, dtype=torch.int32, device=base.device)
        s.p4 = zero() if p4 is None else p4
        s.d4 = zero() if d4 is None else d4
        s.p4w = s.Mb = s.Nn = s.flags = s.fl = None
        s.var = var
        s.p3, s.d3 = p3, d3
        s.p4n, s.d4n = p4n, d4n
        s.p3w = s.p4nw = None
        if s.nested:
            s.slot = torch.cat([p3, p4n])
