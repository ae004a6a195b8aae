"""Minimal level-2 encoder: dense weight [N, K] -> 2-bit trellis base plane + fp16 sign/scale vectors.

It exists to produce honest planes for the CPU-plumbing configuration (one 512 x 256 weight, encode -> decode -> GEMV);
it is not the reference's production encoder. What it restates, in plain torch that runs on CPU or GPU:
  * the quick-fit preprocessing with identity Hessian, where LDLQ feedback vanishes (reference sm120/quickfit/fit_quick.py:1-4,
    threads/12-reference-encoder/nq_encode.py:135-172): seeded +-1 signs, per-channel scales, Hadamard-128 on both sides,
    so that  W ~= D(sv) B_N Q B_K D(su)  with B the 128-blocked orthonormal Hadamard;
  * the tail-biting Viterbi over the 16-bit shift-register trellis with the mul1 codebook (reference
    threads/05-exl3-harness/harness.py:297-364: pass 1 rolled by half a ring finds the state entering step 0, pass 2 is
    constrained to start from and end in it), Viterbi step i <-> ring position p = (-i) mod 256
    (threads/12-reference-encoder/nq_encode.py:54-58);
  * the LSB-first packing of ring states into lane records (threads/12-reference-encoder/nq_decode.py:101-109).
The reference's encoder depends on exllamav3 1.5.1, which is not available here, so bit parity with it is not claimed;
the tests pin this encoder by brute force on a small trellis, by decode(encode) self-consistency and by the Gaussian
distortion the reference reports for this code (MSE 0.068 at 2 bits, threads/03-nested-trellis-code/REPORT.md:21).
"""
import torch

from .format import Proj, proj_sizes

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


def encode_level2(W, seed=0, chunk=64):
    """W [N, K] float (N % 16 == 0, K % 128 == 0; N % 128 == 0 for the output rotation) ->
    dict(base int32 [nrec*4], su fp16 [K], sv fp16 [N], states int64 [units, 8, 256] (ring position order), Q fp32 [N, K])
    with  W ~= D(sv) B_N Q B_K D(su)  and Q the matrix the decoder reproduces bit for bit from `base`."""
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
    target = blocked_had(blocked_had(Wn, 1), 0).float()          # B_N Wn B_K
    S, C = N // 16, K // 128
    RI = ring_index(dev)
    units = target.reshape(S, 16, C, 128).permute(0, 2, 3, 1).reshape(S * C, 2048)   # [unit, column * 16 + row]
    rings = units[:, RI.reshape(-1)].reshape(S * C * 8, 256)     # ring position order
    ip = (-torch.arange(256, device=dev)) % 256                  # Viterbi step i <-> position p = (-i) mod 256
    lut = codebook(dev)
    st = torch.empty(rings.shape, dtype=torch.int64, device=dev)
    for a in range(0, rings.shape[0], chunk):
        sv_i = viterbi_ring(rings[a:a + chunk][:, ip].contiguous(), lut)
        st[a:a + chunk] = sv_i[:, ip]                            # back to position order (ip is its own inverse)
    # stream bit 2p + b = bit b of state(p): the low 2 bits of each state are the 2 new bits of its step
    bits = torch.stack([st & 1, (st >> 1) & 1], -1).reshape(-1, 512)
    chk = (bits.reshape(-1, 256, 2) * torch.tensor([1, 2], device=dev)).sum(-1)
    idx = (torch.arange(256, device=dev)[:, None] + torch.arange(8, device=dev)[None]) % 256
    assert torch.equal((chk[:, idx] << (2 * torch.arange(8, device=dev))).sum(-1), st), "ring states are not tail-biting"
    words = (bits.reshape(-1, 16, 32) << torch.arange(32, device=dev)).sum(-1)       # [rings, 16 words]; lane t4 = words 4 t4..
    base = words.reshape(S * C, 8, 4, 4).reshape(-1)                                  # record = (unit, lane 4 g + t4): 4 words
    base = torch.where(base >= 2**31, base - 2**32, base).to(torch.int32)
    Qr = lut[st]                                                 # decoded values, ring position order
    Qu = torch.empty(S * C, 2048, device=dev)
    Qu[:, RI.reshape(-1)] = Qr.reshape(S * C, 2048)
    Q = Qu.reshape(S, C, 128, 16).permute(0, 3, 1, 2).reshape(N, K)
    return dict(base=base, su=su, sv=sv, states=st.reshape(S * C, 8, 256), Q=Q, target=target)


class EncodedProj(Proj):
    """a Proj (nestquant_amd.format) holding an encoded level-2 base plane; the residual planes are absent"""

    def __init__(s, N, K, base):
        s.z = proj_sizes(N, K)
        s.N, s.K, s.rk, s.bk, s.nested = N, K, 0, 0, False
        s.base = base
        s.p4 = torch.zeros(1, dtype=torch.int32, device=base.device); s.d4 = torch.zeros(1, dtype=torch.int32, device=base.device)
        s.p4w = s.Mb = s.Nn = s.var = s.flags = s.fl = None
        s.p3 = s.d3 = s.p4n = s.d4n = s.p3w = s.p4nw = None
