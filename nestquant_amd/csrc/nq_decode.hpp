// Nested-trellis decode primitives for gfx950 (wave64). Header shared by the dequant, decode-GEMV and prefill kernels.
//
// Format being decoded (reference sm120/nqmoe.cu:14-25, sm120/ref15_spec.py:3-24):
//   unit   = 16 rows x 128 columns = 8 tail-biting rings x 256 weights; ring g = records of lanes 4g..4g+3
//   record = one lane's 64 weights in one plane; base record = 128 bits (2 bits / step); residual record = RBITS bits
//   state(j) = 16-bit window of the lane's record (extended by the ring neighbour's first word) at step_off(j)
//   hash     x = state * 0x83DCD12D mod 2^32 ; S = byte sum of x
//   level 2  w = fp16(A * (1024 + S_b) + B)                                      A = 0x1eee, B = 0xc931
//   level 3/4 F = (Mb S_b + N S_r + 128) >> 8 ; w = fp16(A' * (1024 + F) + C)   block word Mb | N << 8 per unit
//
// gfx950 instruction choices (every opcode of the chain issues at the same measured rate, so their count is what matters):
//   * one v_alignbit_b32 yields the register that holds two windows 16 bits apart; v_and / v_lshrrev (or one v_bfe_u32 where
//     the window lies inside a word) cuts the 16-bit state; the hash is ONE v_mul_lo_u32 by 0x83DCD12D;
//   * v_sad_u8 / v_sad_hi_u8 give the byte sums of two weights already packed as the fp16 pair (1024 + S);
//   * v_dot4_u32_u8 folds Mb * S_b + N * S_r with the rounding constant in its accumulator; v_perm_b32 packs a pair;
//   * v_pk_fma_f16 is the single-rounded fp16 FMA of the value map.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>

namespace nq {

constexpr int TBL_W = 20;                       // int64 words per table row (reference sm120/moe.py:6)
constexpr uint32_t HASH_MUL = 0x83DCD12Du;      // state -> 32-bit hash (reference sm120/moe.py:115, sm120/nqmoe.cu:79)
constexpr uint32_t MUL1_A2 = 0x1eee1eeeu;       // fp16 A twice
constexpr uint32_t MUL1_B2 = 0xc931c931u;       // fp16 B twice
constexpr int CODE_L3 = 10, CODE_L4N = 11, CODE_L4B = 12;   // nested planes of this build: K=1 plane P3; P3 record || P4 record;
                                                            // P3 and P4 records interleaved bit by bit
constexpr int NCODES = 13;

// plane pointers come out of int64 table words; naming the global address space keeps their loads off the flat path
// (flat loads also tick the LDS counter, so a prefetch in flight would stall every LDS read behind it)
#define NQ_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // native vectors: loadable through any address space
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const NQ_GLOBAL u32x4* gp_u4;
typedef const NQ_GLOBAL u32x2* gp_u2;
typedef const NQ_GLOBAL uint32_t* gp_u32;
typedef const NQ_GLOBAL uint16_t* gp_u16;
typedef const NQ_GLOBAL uint8_t* gp_u8;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

template <int C> struct CodeTag { static constexpr int value = C; };        // a compile-time integer passed to generic lambdas

// ---- window patterns (reference sm120/moe.py:10-12, sm120/nqmoe.cu:128-138) ----------------------------------------
template <int CODE> struct Pat;
template <> struct Pat<0>  { static constexpr int KA = 2, M = 0x0000; static constexpr bool SPLIT = false; };
template <> struct Pat<1>  { static constexpr int KA = 1, M = 0xEEEE; static constexpr bool SPLIT = false; };
template <> struct Pat<2>  { static constexpr int KA = 2, M = 0xAAAA; static constexpr bool SPLIT = false; };
template <> struct Pat<3>  { static constexpr int KA = 2, M = 0x8888; static constexpr bool SPLIT = false; };
template <> struct Pat<4>  { static constexpr int KA = 3, M = 0x0000; static constexpr bool SPLIT = false; };
template <> struct Pat<5>  { static constexpr int KA = 1, M = 0xAAAA; static constexpr bool SPLIT = false; };
template <> struct Pat<6>  { static constexpr int KA = 1, M = 0xFFFE; static constexpr bool SPLIT = false; };
template <> struct Pat<7>  { static constexpr int KA = 2, M = 0x9248; static constexpr bool SPLIT = false; };
template <> struct Pat<8>  { static constexpr int KA = 1, M = 0xFEFE; static constexpr bool SPLIT = false; };
template <> struct Pat<9>  { static constexpr int KA = 2, M = 0xD5AA; static constexpr bool SPLIT = false; };
template <> struct Pat<10> { static constexpr int KA = 1, M = 0x0000; static constexpr bool SPLIT = false; };
template <> struct Pat<11> { static constexpr int KA = 2, M = 0x0000; static constexpr bool SPLIT = true; };
template <> struct Pat<12> { static constexpr int KA = 2, M = 0x0000; static constexpr bool SPLIT = true; };
template <int CODE> constexpr bool interleaved_planes = CODE == CODE_L4B;

__host__ __device__ constexpr int popc16(int m) { int c = 0; for (int i = 0; i < 16; ++i) c += (m >> i) & 1; return c; }
__host__ __device__ constexpr int step_off(int j, int KA, int M)
{
    int s = (j >> 4) * (16 * KA + popc16(M));
    for (int i = 0; i < (j & 15); ++i) s += KA + ((M >> i) & 1);
    return s;
}
template <int CODE> struct Rec
{
    static constexpr int KA = Pat<CODE>::KA, M = Pat<CODE>::M;
    static constexpr int BITS = 4 * (16 * KA + popc16(M));
    static constexpr int NW = (BITS + 31) / 32;
    static constexpr int off(int j) { return step_off(j, KA, M); }
};
__host__ inline int rec_bits(int code)
{
    constexpr int ka[NCODES] = {2, 1, 2, 2, 3, 1, 1, 2, 1, 2, 1, 2, 2};
    constexpr int mk[NCODES] = {0, 0xEEEE, 0xAAAA, 0x8888, 0, 0xAAAA, 0xFFFE, 0x9248, 0xFEFE, 0xD5AA, 0, 0, 0};
    return 4 * (16 * ka[code] + popc16(mk[code]));
}

// ---- record loads ---------------------------------------------------------------------------------------------------
// A residual plane stores the BITS bits of a record as a series of sub-arrays, each contiguous over all nrec records so that
// the loads of a wavefront stay coalesced whatever BITS is: as many 128-bit elements as fit, then at most one 64-bit, one
// 32-bit and one 16-bit element, then a tail of BITS % 16 bits per record, bit-packed over the records and followed by a
// 4-byte pad (reference sm120/moe.py:36-49, sm120/nqmoe.cu:17-20). SubArrays is that layout as a compile-time table: for
// every piece its width, the bit position it fills inside the record, and the bytes per record that all earlier sub-arrays
// take (so piece i of record r starts at byte nrec * before[i] + r * width[i] / 8 of the plane).
struct SubArrays { int n; int width[8]; int pos[8]; int before[8]; int tail, tail_pos, tail_before; };
constexpr SubArrays sub_arrays(int bits)
{
    SubArrays L{};
    int pos = 0;
    for (int w = 128; w >= 16; w >>= 1)
        while (bits - pos >= w)                                  // several 128-bit elements, at most one of each smaller width
        {
            L.width[L.n] = w; L.pos[L.n] = pos; L.before[L.n] = pos / 8; ++L.n;
            pos += w;
        }
    L.tail = bits - pos; L.tail_pos = pos; L.tail_before = pos / 8;
    return L;
}

template <int... Is, class F> __device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) { (f(CodeTag<Is>{}), ...); }
template <int N, class F> __device__ __forceinline__ void static_for(F&& f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }

// 32 bits of the interleaved stream: bit 2 i = bit i of the 16-bit piece of plane P3, bit 2 i + 1 = bit i of the piece of P4.
// z holds, from its low byte up, (P3 byte, P4 byte, next P3 byte, next P4 byte); each 16-bit half is shuffled by swapping its
// middle nibbles, then the middle bit pairs of every byte, then the middle bits of every nibble (a perfect shuffle in three
// stages of five instructions: shift, and, the same again the other way, or).
__device__ __forceinline__ uint32_t shuffle_halves(uint32_t z)
{
    z = (z & 0xF00FF00Fu) | ((z & 0x00F000F0u) << 4) | ((z >> 4) & 0x00F000F0u);
    z = (z & 0xC3C3C3C3u) | ((z & 0x0C0C0C0Cu) << 2) | ((z >> 2) & 0x0C0C0C0Cu);
    z = (z & 0x99999999u) | ((z & 0x22222222u) << 1) | ((z >> 1) & 0x22222222u);
    return z;
}

// What is left to do on a loaded record before its windows are cut, kept apart from load_record so that a record requested one
// chunk ahead is not waited for at the point of the request. Code 12: w = (P3 lo, P3 hi, P4 lo, P4 hi) -> the interleaved
// 128 bits. Every other code: nothing.
template <int CODE>
__device__ __forceinline__ void prepare_record(uint32_t* w)
{
    if constexpr (interleaved_planes<CODE>)
    {
        const uint32_t a0 = w[0], a1 = w[1], b0 = w[2], b1 = w[3];
        w[0] = shuffle_halves(__builtin_amdgcn_perm(b0, a0, 0x05010400u));
        w[1] = shuffle_halves(__builtin_amdgcn_perm(b0, a0, 0x07030602u));
        w[2] = shuffle_halves(__builtin_amdgcn_perm(b1, a1, 0x05010400u));
        w[3] = shuffle_halves(__builtin_amdgcn_perm(b1, a1, 0x07030602u));
    }
}

// the record `rec` of a plane at p, as 32-bit words w[0 .. NW). Codes 11 and 12 take the 64-bit record of plane P3 and, nrec
// records further on, the 64-bit record of plane P4: code 11's 128-bit record is the first followed by the second, code 12's
// is the two interleaved bit by bit (stream bit 2 i = bit i of P3's record, bit 2 i + 1 = bit i of P4's), so that every
// 16-bit window holds eight bits of each plane.
template <int CODE>
__device__ __forceinline__ void load_record(uint32_t* w, gp_u8 p, size_t rec, size_t nrec)
{
    if constexpr (Pat<CODE>::SPLIT)
    {
        const u32x2 lo = ((gp_u2)p)[rec], hi = ((gp_u2)(p + nrec * 8))[rec];
        w[0] = lo.x; w[1] = lo.y; w[2] = hi.x; w[3] = hi.y;   // code 12: interleaved by prepare_record() where the record is used
    }
    else
    {
        static constexpr SubArrays L = sub_arrays(Rec<CODE>::BITS);
        static_for<L.n>([&](auto tag) {
            constexpr int i = decltype(tag)::value, W = L.width[i], at = L.pos[i] >> 5;
            const gp_u8 q = p + nrec * (size_t)L.before[i] + rec * (size_t)(W / 8);
            if constexpr (W == 128) { const u32x4 v = *(gp_u4)q; w[at] = v.x; w[at + 1] = v.y; w[at + 2] = v.z; w[at + 3] = v.w; }
            else if constexpr (W == 64) { const u32x2 v = *(gp_u2)q; w[at] = v.x; w[at + 1] = v.y; }
            else if constexpr (W == 32) w[at] = *(gp_u32)q;
            else w[at] = *(gp_u16)q;                              // a 16-bit piece always starts a word
        });
        if constexpr (L.tail != 0)
        {
            // bits [rec * tail, + tail) of the bit-packed tail array; a field that can straddle two words (tail does not divide
            // 32) takes the second word too, which for the last record is the pad
            const size_t bit = rec * (size_t)L.tail;
            const gp_u32 q = (gp_u32)(p + nrec * (size_t)L.tail_before) + (bit >> 5);
            const int sh = (int)(bit & 31);
            uint32_t v = (32 % L.tail) ? __builtin_amdgcn_alignbit(q[1], q[0], sh) : q[0] >> sh;
            v &= (1u << L.tail) - 1u;
            if constexpr ((L.tail_pos & 31) == 0) w[L.tail_pos >> 5] = v;       // the tail opens a word of its own,
            else w[L.tail_pos >> 5] |= v << (L.tail_pos & 31);                 // or sits above the 16-bit piece
        }
    }
}

// A lane's stream continues, after the BITS bits of its own record, with the record of the next lane of its ring (the rings
// are tail-biting): the windows of the last steps reach at most 32 bits into it, so its first word nb is spliced in at bit
// BITS and the word after that cleared. w holds NW + 2 words.
template <int BITS, int NW>
__device__ __forceinline__ void ext_words(uint32_t* w, uint32_t nb)
{
    constexpr int at = BITS >> 5, s = BITS & 31;
    if constexpr (s == 0) w[at] = nb;
    else
    {
        w[at] = (w[at] & ((1u << s) - 1u)) | (nb << s);
        w[at + 1] = nb >> (32 - s);
    }
    w[NW + 1] = 0;
}

// ---- hash -----------------------------------------------------------------------------------------------------------
// x = st * 0x83DCD12D mod 2^32 for the 16-bit window st at bit offset O of the extended record w[]. Windows O and O + 16 share
// one register (window_reg); state() takes the low or the high half of it (an and / a shift, which the compiler merges with
// the funnel shift into one bit-field extract where the window lies inside a word), times_hash() is the 32-bit multiply
// (on gfx950 it issues at the rate of the 16-bit multiply-adds it replaces, two per weight before). The
// multiply is volatile asm so that code which lays several weights side by side keeps that order (weight_pairs2).
template <int O> __device__ __forceinline__ uint32_t window_reg(const uint32_t* w)
{
    constexpr int o = (O & 31) >= 16 ? O - 16 : O, i = o >> 5, s = o & 31;
    if constexpr (s == 0) return w[i]; else return __builtin_amdgcn_alignbit(w[i + 1], w[i], s);
}
template <int O> __device__ __forceinline__ uint32_t state(uint32_t r)
{
    if constexpr ((O & 31) < 16) return r & 0xFFFFu; else return r >> 16;
}
__device__ __forceinline__ uint32_t times_hash(uint32_t st)
{
    uint32_t x;
    const uint32_t hc = HASH_MUL;
    asm volatile("v_mul_lo_u32 %0, %1, %2" : "=v"(x) : "v"(st), "s"(hc));
    return x;
}
template <int O> __device__ __forceinline__ uint32_t hash_at(const uint32_t* w) { return times_hash(state<O>(window_reg<O>(w))); }

// ---- per-unit constants ---------------------------------------------------------------------------------------------
struct FoldK { uint32_t Mrep, Nrep, A2, C2; };      // Mb and N replicated into 4 bytes; fp16 A', C replicated twice

// IEEE 1.0f / i, i = 1..255 (entry 0 unused)
struct RcpTable { float v[256]; };
constexpr RcpTable make_rcp() { RcpTable t{}; t.v[0] = 0.f; for (int i = 1; i < 256; ++i) t.v[i] = 1.0f / (float)i; return t; }
static __device__ __constant__ const RcpTable c_rcp = make_rcp();

// level-2 constants with the ring's sign (sgm = 0x80008000 negates exactly)
__device__ __forceinline__ FoldK consts_l2(uint32_t sgm) { return FoldK{0u, 0u, MUL1_A2 ^ sgm, MUL1_B2 ^ sgm}; }
// fold constants, fp32 operations in the spec's order without contraction (reference sm120/ref15_spec.py:79-84)
__device__ __forceinline__ FoldK consts_fold(uint32_t dw, uint32_t sgm)
{
    const uint32_t Mb = dw & 0xFFu, N = (dw >> 8) & 0xFFu;
    const float rc = c_rcp.v[Mb];
    const _Float16 Ah = (_Float16)__fmul_rn(1.732421875f, rc);
    const float t = __fadd_rn(__fmul_rn(__fmul_rn((float)N, rc), -3.453125f), -3.453125f);
    const _Float16 Ch = (_Float16)__fsub_rn(t, __fmul_rn(1024.f, (float)Ah));
    const uint32_t a = (uint32_t)__builtin_bit_cast(uint16_t, Ah), c = (uint32_t)__builtin_bit_cast(uint16_t, Ch);
    return FoldK{Mb * 0x01010101u, N * 0x01010101u, (a * 0x00010001u) ^ sgm, (c * 0x00010001u) ^ sgm};
}

__device__ __forceinline__ uint32_t pk_fma(uint32_t h, uint32_t a, uint32_t c)
{
    const half2_t r = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, h), __builtin_bit_cast(half2_t, a),
                                                __builtin_bit_cast(half2_t, c));
    return __builtin_bit_cast(uint32_t, r);
}

// ---- pair decode ----------------------------------------------------------------------------------------------------
// fp16 pair (1024 + S or 1024 + F) of lane weights JA (low half) and JB (high half); exact integers in fp16.
// RES = false: base only. wb: extended base record (6 words); wr: extended residual record.
// BK = window code of the base plane (0: two bits per step; 1: the 1.75-bit pattern), wb extended accordingly.
template <bool RES, int CODE, int JA, int JB, int BK = 0>
__device__ __forceinline__ uint32_t code_pair(const uint32_t* wb, const uint32_t* wr, const FoldK& k)
{
    const uint32_t xa = hash_at<Rec<BK>::off(JA)>(wb), xb = hash_at<Rec<BK>::off(JB)>(wb);
    if constexpr (!RES)
    {
        const uint32_t t = __builtin_amdgcn_sad_u8(xa, 0u, 0x64006400u);
        return __builtin_amdgcn_sad_hi_u8(xb, 0u, t);
    }
    else
    {
        uint32_t ta = __builtin_amdgcn_udot4(xa, k.Mrep, 0x640080u, false);
        uint32_t tb = __builtin_amdgcn_udot4(xb, k.Mrep, 0x640080u, false);
        ta = __builtin_amdgcn_udot4(hash_at<Rec<CODE>::off(JA)>(wr), k.Nrep, ta, false);
        tb = __builtin_amdgcn_udot4(hash_at<Rec<CODE>::off(JB)>(wr), k.Nrep, tb, false);
        return __builtin_amdgcn_perm(tb, ta, 0x06050201u);          // bits [8, 24) of ta, then of tb
    }
}
// decoded fp16 weight pair (bit-exact values)
template <bool RES, int CODE, int JA, int JB, int BK = 0>
__device__ __forceinline__ uint32_t weight_pair(const uint32_t* wb, const uint32_t* wr, const FoldK& k)
{
    return pk_fma(code_pair<RES, CODE, JA, JB, BK>(wb, wr, k), k.A2, k.C2);
}

// ---- two pairs at once, stage by stage --------------------------------------------------------------------------------
// A wavefront cannot issue an instruction right behind the one whose result it needs, and a SIMD that holds only two to four
// wavefronts then idles part of the time. The decode of one weight is a chain of five to seven dependent instructions, but
// the weights are independent of each other: here the four weights (JA, JA + 8, JB, JB + 8) go through the
// chain side by side, each stage for all four before the next, so that four independent instructions separate an instruction
// from the one that needs its result. The hash multiplies are volatile asm: the compiler keeps them in this order and fits
// the rest around them (measured at two wavefronts per SIMD: 2.39 -> 2.02 ns per instruction; at four 2.03 -> 1.85). Values
// and roundings are those of weight_pair.
// RAW: stop before the value map and hand out the fp16 pairs (1024 + S) or (1024 + F) themselves -- exact integers -- for a
// caller that applies the affine map to its accumulated products instead of to every weight (gemv_chunks<..., RAW>).
template <bool RES, int CODE, int JA, int JB, int BK = 0, bool RAW = false>
__device__ __forceinline__ void weight_pairs2(const uint32_t* wb, const uint32_t* wr, const FoldK& k, uint32_t& ua, uint32_t& ub)
{
    constexpr int B0 = Rec<BK>::off(JA), B1 = Rec<BK>::off(JA + 8), B2 = Rec<BK>::off(JB), B3 = Rec<BK>::off(JB + 8);
    const uint32_t r0 = window_reg<B0>(wb), r1 = window_reg<B1>(wb), r2 = window_reg<B2>(wb), r3 = window_reg<B3>(wb);
    const uint32_t y0 = state<B0>(r0), y1 = state<B1>(r1), y2 = state<B2>(r2), y3 = state<B3>(r3);
    if constexpr (!RES)
    {
        const uint32_t x0 = times_hash(y0), x1 = times_hash(y1), x2 = times_hash(y2), x3 = times_hash(y3);
        const uint32_t ta = __builtin_amdgcn_sad_u8(x0, 0u, 0x64006400u), tb = __builtin_amdgcn_sad_u8(x2, 0u, 0x64006400u);
        const uint32_t ca = __builtin_amdgcn_sad_hi_u8(x1, 0u, ta), cb = __builtin_amdgcn_sad_hi_u8(x3, 0u, tb);
        if constexpr (RAW) { ua = ca; ub = cb; }
        else { ua = pk_fma(ca, k.A2, k.C2); ub = pk_fma(cb, k.A2, k.C2); }
    }
    else
    {
        constexpr int R0 = Rec<CODE>::off(JA), R1 = Rec<CODE>::off(JA + 8), R2 = Rec<CODE>::off(JB), R3 = Rec<CODE>::off(JB + 8);
        const uint32_t q0 = window_reg<R0>(wr), q1 = window_reg<R1>(wr), q2 = window_reg<R2>(wr), q3 = window_reg<R3>(wr);
        const uint32_t z0 = state<R0>(q0), z1 = state<R1>(q1), z2 = state<R2>(q2), z3 = state<R3>(q3);
        const uint32_t x0 = times_hash(y0), x1 = times_hash(y1), x2 = times_hash(y2), x3 = times_hash(y3);
        const uint32_t v0 = times_hash(z0), v1 = times_hash(z1), v2 = times_hash(z2), v3 = times_hash(z3);
        uint32_t t0 = __builtin_amdgcn_udot4(x0, k.Mrep, 0x640080u, false), t1 = __builtin_amdgcn_udot4(x1, k.Mrep, 0x640080u, false);
        uint32_t t2 = __builtin_amdgcn_udot4(x2, k.Mrep, 0x640080u, false), t3 = __builtin_amdgcn_udot4(x3, k.Mrep, 0x640080u, false);
        t0 = __builtin_amdgcn_udot4(v0, k.Nrep, t0, false); t1 = __builtin_amdgcn_udot4(v1, k.Nrep, t1, false);
        t2 = __builtin_amdgcn_udot4(v2, k.Nrep, t2, false); t3 = __builtin_amdgcn_udot4(v3, k.Nrep, t3, false);
        const uint32_t ca = __builtin_amdgcn_perm(t1, t0, 0x06050201u), cb = __builtin_amdgcn_perm(t3, t2, 0x06050201u);
        if constexpr (RAW) { ua = ca; ub = cb; }
        else { ua = pk_fma(ca, k.A2, k.C2); ub = pk_fma(cb, k.A2, k.C2); }
    }
}

// ---- table row ------------------------------------------------------------------------------------------------------
// int64[20] per expert (reference sm120/moe.py:216-229, sm120/nqmoe.cu:26-45):
//   [0] level 0/2/3/4  [1..4] gate|up base, residual plane, block words, flags (mask mode, 0 = dense)  [5..8] down  [9] sign/scale vector
//   [10],[11] residual window code of gate|up, down  [12],[13] sign-variant planes  [14..17] low-rank plane (buffers, ranks)
//   [18] in_had_down (0 / 128 / 512)  [19] base window codes, gate|up | down << 8 (0 or 1)
typedef const NQ_GLOBAL uint64_t* gp_u64;
struct Planes { gp_u4 base; gp_u8 res; gp_u32 dw; gp_u8 var; gp_u64 flags; int code; int bcode; };

// Base record of a lane: code 0 = one uint4 per record; other codes = the residual plane's sub-array layout at
// Rec<BK>::BITS bits per record (reference sm120/NQ_RES_V2.md:38-46), at most 128 bits.
template <int BK>
__device__ __forceinline__ u32x4 load_base(const Planes& P, size_t rec, size_t nrec)
{
    if constexpr (BK == 0) return P.base[rec];
    else
    {
        static_assert(Rec<BK>::BITS <= 128, "base records are at most four words");
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        load_record<BK>(w, (gp_u8)P.base, rec, nrec);
        return u32x4{w[0], w[1], w[2], w[3]};
    }
}
// wb[0..3] = the record's words -> wb[0..5] = the record followed by the ring neighbour's first word `nb`
template <int BK>
__device__ __forceinline__ void ext_base(uint32_t* wb, uint32_t nb) { ext_words<Rec<BK>::BITS, Rec<BK>::NW>(wb, nb); }
template <class F>
__device__ __forceinline__ void dispatch_base(int bcode, F&& f)
{
    if (bcode == 1) f(CodeTag<1>{}); else f(CodeTag<0>{});
}

// Mask mode (reference sm120/nqmoe.cu:22-24,202-206): flags = one uint64 per strip, bit c = chunk c is refined; the residual
// plane and its block words are compact over the nm = popcount(flags) refined chunks of every strip, in chunk order, and
// the other chunks decode at level 2. Flags are equal over the 8 strips of a 128-row group.
struct MaskedUnit { bool on; size_t unit; size_t nrec; };     // refined?; residual unit index; residual records of the plane
__device__ __forceinline__ MaskedUnit masked_unit(uint64_t f, size_t strip, int c, size_t nstrips)
{
    const int nm = __popcll(f);
    return MaskedUnit{((f >> c) & 1ull) != 0, strip * nm + __popcll(f & ((1ull << c) - 1ull)), nstrips * nm * 32};
}
__device__ __forceinline__ Planes planes_of(const int64_t* ent, int mode)
{
    const int o = mode == 0 ? 1 : 5;
    Planes P;
    P.base = (gp_u4)ent[o]; P.res = (gp_u8)ent[o + 1]; P.dw = (gp_u32)ent[o + 2];
    P.var = (gp_u8)ent[mode == 0 ? 12 : 13]; P.code = (int)ent[10 + mode]; P.flags = (gp_u64)ent[o + 3];
    P.bcode = (int)((ent[19] >> (8 * mode)) & 0xFF);
    return P;
}

// compile-time dispatch over the residual code; F is a generic lambda taking std::integral_constant<int, CODE>
template <class F>
__device__ __forceinline__ void dispatch_code(int code, F&& f)
{
    switch (code)
    {
        case 1: f(CodeTag<1>{}); break;   case 2: f(CodeTag<2>{}); break;   case 3: f(CodeTag<3>{}); break;
        case 4: f(CodeTag<4>{}); break;   case 5: f(CodeTag<5>{}); break;   case 6: f(CodeTag<6>{}); break;
        case 7: f(CodeTag<7>{}); break;   case 8: f(CodeTag<8>{}); break;   case 9: f(CodeTag<9>{}); break;
        case 10: f(CodeTag<10>{}); break; case 11: f(CodeTag<11>{}); break; case 12: f(CodeTag<12>{}); break;
        default: f(CodeTag<0>{}); break;
    }
}

}  // namespace nq
