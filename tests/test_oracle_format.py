"""Pins the oracle's format arithmetic and code->value map to facts stated in the reference's text (no imports of it).

Each check is chosen so that a plausible slip (wrong mask, dropped pad, transposed operand, wrong rounding order) fails.
"""
import numpy as np
import pytest

from oracle import nq_oracle as O


def test_record_bits_table():
    # reference threads/13-moe-layer-kernel/INTEGRATION.md:43-44 and sm120/NQ_RES_V2.md:24
    want = {0: 128, 1: 112, 2: 160, 3: 144, 4: 192, 5: 96, 6: 124, 7: 148, 8: 120, 9: 164, 10: 64, 11: 128, 12: 128}
    assert {c: O.rbits(c) for c in O.RKP} == want


@pytest.mark.parametrize("code", sorted(O.RKP))
def test_step_offsets_cover_the_ring(code):
    ka, mask = O.RKP[code]
    off = O.step_off(np.arange(257), ka, mask)
    assert off[0] == 0 and np.all(np.diff(off) >= ka) and np.all(np.diff(off) <= ka + 1)
    assert off[256] == 4 * O.rbits(code)                    # reference sm120/moe.py:121 invariant (G = 4 lanes)
    assert off[64] == O.rbits(code)                         # one lane = 64 steps = one record
    # the last window of a lane ends inside record + the neighbour's first word
    assert off[63] + 16 <= O.rbits(code) + 32
    # every step's width follows the mask bit of its position
    assert all(off[p + 1] - off[p] == ka + ((mask >> (p % 16)) & 1) for p in range(256))


def test_published_plane_sizes():
    # TP8 shard I = 256 (reference threads/13-moe-layer-kernel/INTEGRATION.md:26-33): gate|up [512, 6144], down [6144, 256]
    gu, dn = O.proj_sizes(512, 6144, rk=6), O.proj_sizes(6144, 256, rk=7)
    assert (gu["base"], dn["base"]) == (786432, 393216)
    assert (gu["p4"] - 4, dn["p4"] - 4) == (761856, 454656)           # payload; the tail sub-array adds a 4-byte pad
    assert (gu["d4"], dn["d4"]) == (6144, 3072)
    assert O.proj_sizes(512, 6144, rk=1)["p4"] == 688128 and O.proj_sizes(6144, 256, rk=2)["p4"] == 491520
    # TP4 shard I = 512 record segments (reference sm120/NQ_RES_V2.md:66-68): code 3 gate|up, code 9 down (with pad)
    assert O.proj_sizes(1024, 6144, rk=3)["p4"] == 1769472
    assert O.proj_sizes(6144, 512, rk=9)["p4"] == 1007620
    # full-shape expert (H 6144, I 2048): base 9,437,184 B; block words 73,728 B
    g, d = O.proj_sizes(4096, 6144), O.proj_sizes(6144, 2048)
    assert g["base"] + d["base"] == 9437184 and g["d4"] + d["d4"] == 73728


@pytest.mark.parametrize("code", sorted(O.RKP))
@pytest.mark.parametrize("nrec", [32, 96, 416])
def test_pack_round_trip(code, nrec):
    rng = np.random.default_rng(code * 1000 + nrec)
    bits = O.rbits(code); nw = (bits + 31) // 32
    w = rng.integers(0, 2**32, (nrec, nw), dtype=np.uint64).astype(np.uint32)
    if bits % 32:
        w[:, -1] &= np.uint32((1 << (bits % 32)) - 1)
    for split in ((False, True) if code == 11 else (False,)):
        buf = O.pack_words(w, bits, split)
        assert buf.size == O.plane_bytes(nrec, code)
        assert np.array_equal(O.unpack_words(buf, nrec, bits, split), w)


def test_codebook_known_answers():
    st = np.arange(65536)
    S = O.hash_sum(st)
    assert S.min() >= 0 and S.max() <= 1020
    # brute force on a few states with Python integers
    for s in (0, 1, 2, 255, 256, 4097, 65535, 0xBEEF):
        x = (s * 0x83DCD12D) & 0xFFFFFFFF
        assert S[s] == sum((x >> (8 * i)) & 255 for i in range(4))
    q = O.q2_value(S).astype(np.float64)
    assert q[0] == -3.453125 == O.K0                          # reference sm120/ref15_spec.py:35
    # unit-variance, zero-mean codebook: sum of 4 uniform bytes has mean 510 and std sqrt(4 (256^2 - 1) / 12) = 147.8,
    # and the reference documents the map as (1024 + bytesum) * (1 / 147.7) - 10.39 (threads/05-exl3-harness/harness.py:261)
    assert abs(1.0 / O.A_ - 147.7) < 0.1 and abs(O.B_ + 10.39) < 0.01
    assert abs(q.mean()) < 0.01 and abs(np.sqrt((q ** 2).mean()) - 1.0) < 0.01
    assert abs(S.mean() - 510.0) < 1.0 and abs(S.std() - 147.8) < 1.0
    # the fp16 bit pattern 0x6400 + S is exactly 1024 + S
    h = (0x6400 + S).astype(np.uint16).view(np.float16).astype(np.float64)
    assert np.array_equal(h, 1024.0 + S)
    # single rounding: exact rational arithmetic vs the float64 path on every S
    from fractions import Fraction
    A, B = Fraction(0x6EE, 1 << 18), Fraction(float(O.B16))
    for s in range(0, 1021, 7):
        exact = A * (1024 + s) + B
        assert float(np.float16(float(exact))) == float(O.q2_value(np.array([s]))[0])
    assert float(O.A16) == float(Fraction(1774, 1 << 18))      # reference sm120/ref15_spec.py:17: A = 1774 / 2^18


def test_block_words_and_fold_constants():
    L = O.all_block_words()
    assert len(L) == 33149                                    # reference sm120/results/verify_ext_I512.txt:2
    Mb, N = L[:, 0], L[:, 1]
    Ah, Ch = O.fold_consts(Mb, N)
    # The reference holds two textual variants of C: its torch decoder and its kernel subtract 1024 A' in fp32
    # (sm120/moe.py:132, sm120/nqmoe.cu:267-268, verified equal to each other on all 33149 words by the reference's
    # verify_ext.py), its numpy spec subtracts in float64 (sm120/ref15_spec.py:83). The oracle follows the fp32 pair.
    # The two variants differ only by double rounding, on a handful of words; A' never differs.
    rcp = (np.float32(1) / Mb.astype(np.float32))
    Ah64 = (np.float32(1.732421875) * rcp).astype(np.float64).astype(np.float16)
    t = (N.astype(np.float32) * rcp) * np.float32(O.K0) + np.float32(O.K0)
    Ch64 = (t.astype(np.float64) - 1024.0 * Ah64.astype(np.float64)).astype(np.float16)
    assert np.array_equal(Ah.view(np.uint16), Ah64.view(np.uint16))
    differ = Ch.view(np.uint16) != Ch64.view(np.uint16)
    assert differ.sum() == 11 and np.abs(Ch.view(np.int16).astype(int) - Ch64.view(np.int16).astype(int)).max() == 1   # one fp16 ulp
    assert {tuple(x) for x in L[differ][:4].tolist()} == {(7, 105), (13, 71), (14, 98), (15, 45)}
    # N = 0: the fold must reproduce level 2 up to the fold's own rounding of Sb (F = round-half-up(Mb Sb / 256) ...)
    S = np.arange(0, 1021)
    v = O.fold_value(S, np.zeros_like(S), 256 - 1, 0).astype(np.float64)        # Mb = 255
    assert np.abs(v - O.q2_value(S).astype(np.float64)).max() < 0.02
    # additive form bound |Q4 - (Q2 + delta (A Sr + K0))| <= 0.024 (reference threads/15-level4-decode/REPORT.md:178-186)
    rng = np.random.default_rng(0)
    idx = rng.integers(0, len(L), 4000)
    sb, sr = rng.integers(0, 1021, 4000), rng.integers(0, 1021, 4000)
    m, n = Mb[idx], N[idx]
    ok = (m >= 120) & (n <= 0.8 * m)                          # the realistic range the bound was measured on
    q4 = O.fold_value(sb, sr, m, n).astype(np.float64)
    add = O.q2_value(sb).astype(np.float64) + (n / m) * (O.A_ * sr + O.K0)
    assert np.abs(q4 - add)[ok].max() <= 0.03
    # F stays below 1024 so that 0x6400 + F is the fp16 of 1024 + F
    F = (m * sb + n * sr + 128) >> 8
    assert F.max() <= 1023 and ((Mb + N) <= 257).all()


def test_fold_exact_vs_fractions():
    """value = fp16(A' (1024 + F) + C) with ONE rounding: compare with exact rational arithmetic"""
    from fractions import Fraction
    rng = np.random.default_rng(1)
    L = O.all_block_words()
    for i in rng.integers(0, len(L), 300):
        m, n = int(L[i, 0]), int(L[i, 1])
        sb, sr = int(rng.integers(0, 1021)), int(rng.integers(0, 1021))
        Ah, Ch = O.fold_consts(np.array([m]), np.array([n]))
        F = (m * sb + n * sr + 128) >> 8
        exact = Fraction(float(Ah[0])) * (1024 + F) + Fraction(float(Ch[0]))
        want = np.float16(float(exact)) if exact.denominator.bit_length() < 60 else None
        got = O.fold_value(np.array([sb]), np.array([sr]), np.array([m]), np.array([n]))[0]
        # float(exact) is exact here: the sum has <= 24 significant bits (checked), so one rounding to fp16 remains
        num = exact.numerator
        assert abs(num).bit_length() - (abs(num) & -abs(num)).bit_length() + 1 <= 24
        assert want is not None and want == got


def test_geometry_is_a_bijection():
    row, col = O.lane_to_rowcol()
    idx = (row * 128 + col).reshape(-1)
    assert sorted(idx.tolist()) == list(range(2048))           # reference nq_decode.py:83 / ref15_spec.py:118-125
    # lanes of one quad share rows; a lane owns rows g and g + 8 only
    for lane in range(32):
        assert set(row[lane].tolist()) == {lane >> 2, (lane >> 2) + 8}


@pytest.mark.parametrize("code", sorted(O.RKP))
def test_lane_view_equals_ring_view(code):
    rng = np.random.default_rng(100 + code)
    bits = O.rbits(code); nw = (bits + 31) // 32
    w = rng.integers(0, 2**32, (64, nw), dtype=np.uint64).astype(np.uint32)
    if bits % 32:
        w[:, -1] &= np.uint32((1 << (bits % 32)) - 1)
    lane = O.lane_sums(w, code)                                # [64 records, 64]
    ring = O.hash_sum(O.ring_states(w, code))                  # [16 rings, 256], position p = t4 * 64 + j
    assert np.array_equal(lane.reshape(16, 256), ring)
    # rings of two records (the reference's G = 2 reading of the same planes): both walks agree there too, and differ from G = 4
    lane2 = O.lane_sums(w, code, G=2)
    assert np.array_equal(lane2.reshape(32, 128), O.hash_sum(O.ring_states(w, code, G=2)))
    assert not np.array_equal(lane2, lane)


def test_tail_biting_is_real():
    """the last windows of lane 3 of a ring must read lane 0's first bits (a decoder without the wrap fails this)"""
    w = np.zeros((4, 4), np.uint32)
    w[0, 0] = 0xFFFF                                           # only the ring's first 16 bits are set
    s = O.lane_sums(w, 0)
    zero = O.hash_sum(np.array([0]))[0]
    assert (s[3, 57:] != zero).all() and (s[3, :56] == zero).all() and (s[1] == zero).all()


def test_hadamard_and_layer_invariants():
    Hm = O.hadamard(128)
    assert np.allclose(Hm @ Hm.T, np.eye(128), atol=1e-6) and np.allclose(Hm, Hm.T)
    rng = np.random.default_rng(3)
    H = I = 256
    Wgu = rng.standard_normal((2 * I, H)).astype(np.float16).astype(np.float32)
    Wdn = rng.standard_normal((H, I)).astype(np.float16).astype(np.float32)
    signs = (rng.integers(0, 2, 3 * H + 3 * I) * 2 - 1).astype(np.float16)
    x = (rng.standard_normal((2, H)) * 0.05).astype(np.float32)
    y = O.expert_forward(x, Wgu, Wdn, signs, round_acts=False)
    # the layer equals a plain SwiGLU MLP with effective weights D(sv) B W B D(su) (reference sm120/eval/nqeff.py:5-11)
    s = O.split_signs(signs, H, I)
    Bh = np.kron(np.eye(H // 128), Hm).astype(np.float64); Bi = np.kron(np.eye(I // 128), Hm).astype(np.float64)
    Wg = np.diag(s["sv_g"]) @ Bi @ Wgu[:I].astype(np.float64) @ Bh @ np.diag(s["su_g"])
    Wu = np.diag(s["sv_u"]) @ Bi @ Wgu[I:].astype(np.float64) @ Bh @ np.diag(s["su_u"])
    Wd = np.diag(s["sv_o"]) @ Bh @ Wdn.astype(np.float64) @ Bi @ np.diag(s["su_d"])
    g = x.astype(np.float64) @ Wg.T; u = x.astype(np.float64) @ Wu.T
    ref = (g / (1 + np.exp(-g)) * u) @ Wd.T
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-5


def test_route_runs_semantics():
    sel = np.array([[5, 2, 7, 2], [2, 9, 5, 1]])
    rw = np.array([[.25, .25, .25, .25], [.5, 0., .25, .25]], np.float16)
    levels = {5: 2, 2: 4, 7: 0, 9: 4, 1: 2}
    runs = O.route_runs(sel, rw, levels)
    assert [r["e"] for r in runs] == [5, 2, 1]                # first-occurrence order; level 0 and rw == 0 dropped
    assert runs[0]["slots"] == [0, 6] and runs[1]["slots"] == [1, 3, 4] and runs[2]["slots"] == [7]


def test_mailbox_state_machine():
    table = np.zeros((4, O.TBL_W), np.int64); stage = np.arange(4 * O.TBL_W).reshape(4, -1).astype(np.int64)
    seq = np.array([0, 1, 0, 2], np.int32); applied = np.array([0, 0, 0, 2], np.int32)
    assert O.mailbox_apply(table, stage, seq, applied) == 1
    assert np.array_equal(table[1], stage[1]) and not table[[0, 2, 3]].any() and np.array_equal(applied, seq)
    assert O.mailbox_apply(table, stage, seq, applied) == 0


@pytest.mark.parametrize("code", [0, 1, 3, 7, 9])
def test_ring_streams_to_lane_words(code):
    """the loader's repack step (ring byte streams -> lane records) against a window walk done directly on the byte streams:
    state p of a ring = the 16 bits at step_off(p) of its tail-biting stream, LSB-first bytes"""
    import torch
    from nestquant_amd import format as F
    rng = np.random.default_rng(300 + code)
    bits = O.rbits(code); ka, mask = O.RKP[code]
    nrings = 24
    raw = rng.integers(0, 256, (nrings, 4 * bits // 8), dtype=np.uint8)
    w = F.lane_words_from_rings(torch.from_numpy(raw.reshape(-1)), bits)
    assert w.shape == (nrings * 4, (bits + 31) // 32) and int(w.max()) < 2**32
    if bits % 32:
        assert int(w[:, -1].max()) < 1 << (bits % 32)
    assert np.array_equal(F.rings_from_lane_words(w, bits).numpy(), raw)
    # direct walk over the bytes, no lane view involved
    L = 4 * bits
    stream = np.unpackbits(raw, axis=1, bitorder="little").astype(np.int64)          # [rings, L]
    off = np.asarray(O.step_off(np.arange(256), ka, mask))
    idx = (off[:, None] + np.arange(16)) % L
    states = (stream[:, idx] << np.arange(16)).sum(-1)                                 # [rings, 256]
    assert np.array_equal(O.ring_states(w.numpy().astype(np.uint32), code), states)
    assert np.array_equal(O.lane_sums(w.numpy().astype(np.uint32), code).reshape(nrings, 256), O.hash_sum(states))
    # and through the packer: pack_words -> unpack_words gives the records back
    assert torch.equal(F.unpack_words(F.pack_words(w, bits), nrings * 4, bits), w)
