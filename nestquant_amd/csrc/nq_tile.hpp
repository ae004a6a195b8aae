// Pieces shared by the decode-path GEMV (nq_moe.hip) and the prefill grouped GEMM (nq_prefill.hip): the wavefront
// Hadamard-128, the B-operand column order, and the stream of MFMA A operands decoded from trellis records.
//
// Lane mapping (wave64): lane = 16 * t4 + 8 * ss + g decodes the record of lane (4 g + t4) of unit (strip0 + ss, chunk).
// It holds 32 weights of row g and 32 of row g + 8, in columns 16 t + 2 t4 + {0,1,8,9}. v_mfma_f32_16x16x32_f16 takes 8
// fp16 per lane; lanes with equal (ss, g) and different t4 are the four k-groups of one A row, so the decoded pairs
// (w_j, w_{j+8}) are A operands as they leave the decoder. MFMA (MM, RHO) covers rows g + 8 RHO and the columns of
// t = 2 MM, 2 MM + 1; its B operand (16 tokens) holds the same columns, see bop_index().
#pragma once
#include "nq_decode.hpp"
#include <utility>

namespace nq {

// ---- Hadamard-128 on one wavefront: lane holds elements 2 lane, 2 lane + 1 --------------------------------------------
// One in-lane butterfly, then six cross-lane stages: lanes l and l ^ m exchange, the lane with bit m clear keeps a + a',
// the other a' - a (a' = the partner's value), all in fp32 in this order. The exchanges use no LDS: DPP lane selects for
// m = 1, 2, 4, 8 (quad permutes, a half-row mirror, a row rotate), and for m = 16, 32 the row / half swaps of gfx950, which
// leave both partners' values in both lanes. The per-lane sign is a sign-bit flip (or a factor +-1 in an FMA), so every sum
// is the same single rounding as a plain add or subtract. All 64 lanes must be active.
template <int CTRL> __device__ __forceinline__ float dpp_lane(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float flip_sign(float v, uint32_t m) { return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) ^ m); }
// lo / hi = the value of the lane with bit 16 (bit 32) clear / set, in both lanes. The swap exchanges the odd 16-lane rows
// (the upper half) of its first register with the even rows (the lower half) of its second; the two read-write operands
// force two distinct registers that start as the same value. Written as asm because the compiler's builtin for it hands
// back the first register for both results; the compiler therefore does not see the instruction and cannot place the wait
// states it needs after the writes that feed it and before the reads of its results, so they are written out here.
__device__ __forceinline__ void swap_rows16(float v, float& lo, float& hi)
{
    lo = v; hi = v;
    asm volatile("s_nop 3\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 3" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ void swap_halves32(float v, float& lo, float& hi)
{
    lo = v; hi = v;
    asm volatile("s_nop 3\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 3" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ void wht128(float& a, float& b, int lane)
{
    const float s = a + b, d = a - b; a = s; b = d;
    const uint32_t l = (uint32_t)lane;
    const uint32_t n1 = (l << 31) & 0x80000000u, n2 = (l << 30) & 0x80000000u, n4 = (l << 29) & 0x80000000u, n8 = (l << 28) & 0x80000000u;
    a = dpp_lane<0xB1>(a) + flip_sign(a, n1); b = dpp_lane<0xB1>(b) + flip_sign(b, n1);                   // quad_perm [1,0,3,2]
    a = dpp_lane<0x4E>(a) + flip_sign(a, n2); b = dpp_lane<0x4E>(b) + flip_sign(b, n2);                   // quad_perm [2,3,0,1]
    a = dpp_lane<0x141>(dpp_lane<0x1B>(a)) + flip_sign(a, n4);                                            // l ^ 3 then l ^ 7 = l ^ 4
    b = dpp_lane<0x141>(dpp_lane<0x1B>(b)) + flip_sign(b, n4);
    a = dpp_lane<0x128>(a) + flip_sign(a, n8); b = dpp_lane<0x128>(b) + flip_sign(b, n8);                 // row_ror 8
    const float s16 = (lane & 16) ? -1.f : 1.f, s32 = (lane & 32) ? -1.f : 1.f;
    float lo, hi;
    swap_rows16(a, lo, hi); a = __builtin_fmaf(hi, s16, lo);
    swap_rows16(b, lo, hi); b = __builtin_fmaf(hi, s16, lo);
    swap_halves32(a, lo, hi); a = __builtin_fmaf(hi, s32, lo);
    swap_halves32(b, lo, hi); b = __builtin_fmaf(hi, s32, lo);
    a *= 0.08838834764f; b *= 0.08838834764f;
}

// LDS position (in halfs) of column c of a 128-column chunk in the B-operand order:
// 16-byte block (mm, kg) holds, for i = 0..3, columns 32 mm + 2 kg + 8 (i >> 1) + (i & 1) and that + 16
__device__ __forceinline__ int bop_index(int c)
{
    const int mm = c >> 5, hi = (c >> 4) & 1, kg = (c >> 1) & 3, i = 2 * ((c >> 3) & 1) + (c & 1);
    return (mm * 4 + kg) * 8 + 2 * i + hi;
}

// A operand of MFMA (MM, RHO): rows g + 8 RHO, columns of t = 2 MM and 2 MM + 1
template <bool RES, int CODE, int MM, int RHO, int BK = 0, bool RAW = false>
__device__ __forceinline__ half8_t a_operand(const uint32_t* wb, const uint32_t* wr, const FoldK& k)
{
    constexpr int J = 16 * MM + 2 * RHO;
    uint32_t u[4];
    weight_pairs2<RES, CODE, J + 0, J + 1, BK, RAW>(wb, wr, k, u[0], u[1]);
    weight_pairs2<RES, CODE, J + 4, J + 5, BK, RAW>(wb, wr, k, u[2], u[3]);
    return __builtin_bit_cast(half8_t, *(u32x4*)u);
}

// Wavefront priority by progress through the k-slice. The SIMD's arbiter picks the highest user priority and, among equals,
// the oldest wavefront, so of the co-resident wavefronts (one per workgroup, all with the same amount of work) the oldest
// would finish far ahead of the youngest, and the SIMD would spend the end of the launch with one or two wavefronts, which
// cannot keep the vector ALU busy. Lowering a wavefront's priority as it nears its end lets the others catch up, so that
// they finish together; a wavefront of lower priority still issues whenever the others wait.
// Measured (decode layer, B = 1): gate|up launch 48.2 -> 44.2 us with k-slices of 12 chunks; the down launch gains with
// k-slices of 8 chunks (31.8 -> 29.8 us) and loses with 4, where the steps are too coarse, so short slices keep one priority.
// The thresholds (a half, a quarter, an eighth of the slice left) were the best of six sets tried.
__device__ __forceinline__ void progress_priority(int c, int NC)
{
    if (NC < 8) return;
    const int left = 8 * (NC - c);                               // eighths of chunks left, this chunk included
    if (left > 4 * NC) __builtin_amdgcn_s_setprio(3);
    else if (left > 2 * NC) __builtin_amdgcn_s_setprio(2);
    else if (left > NC) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

struct LaneCtx
{
    size_t rec0;          // record index of this lane in chunk 0 of its k-slice: (unit0) * 32 + 4 g + t4
    size_t unit0;         // unit index (strip * C + chunk0)
    size_t nrec;          // records of the whole projection (sub-array stride)
    int src;              // lane holding the next record of the ring
    int g;                // ring index (sign-variant bit)
    const char* xs;       // this lane's B-operand base in LDS (bytes), kg folded in
    int xstep;            // bytes per chunk (0 for lanes without a token)
    size_t strip, nstrips; int chunk0;   // mask mode: this lane's strip, strips of the projection, first chunk of the k-slice
};

// mask mode: chunk by chunk either the folded decode (refined chunks, residual records compact over them) or the level-2
// decode; the choice is the same for every lane of the workgroup. Residual records are fetched when needed (no prefetch).
template <int CODE, int BK>
__device__ __forceinline__ void gemv_chunks_masked(const Planes& P, const LaneCtx& L, int NC, float4_t* acc, u32x4 nb)
{
    constexpr int NW = Rec<CODE>::NW;
    const uint64_t f = P.flags[L.strip];
    uint32_t nvar = P.var ? (uint32_t)P.var[L.unit0] : 0u;
    for (int c = 0; c < NC; ++c)
    {
        progress_priority(c, NC);
        uint32_t wb[6], wr[NW + 2] = {0};
        wb[0] = nb.x; wb[1] = nb.y; wb[2] = nb.z; wb[3] = nb.w;
        const uint32_t var = nvar;
        const MaskedUnit m = masked_unit(f, L.strip, L.chunk0 + c, L.nstrips);
        const bool on = __builtin_amdgcn_readfirstlane((int)m.on) != 0;
        uint32_t dw = 0;
        if (on) { load_record<CODE>(wr, P.res, m.unit * 32 + (L.rec0 & 31), m.nrec); dw = P.dw[m.unit]; }
        if (c + 1 < NC)
        {
            nb = load_base<BK>(P, L.rec0 + (size_t)(c + 1) * 32, L.nrec);
            if (P.var) nvar = P.var[L.unit0 + c + 1];
        }
        ext_base<BK>(wb, __shfl(wb[0], L.src));
        const uint32_t sgm = ((var >> L.g) & 1u) * 0x80008000u;
        const char* xp = L.xs + c * L.xstep;
        if (on)
        {
            prepare_record<CODE>(wr);
            ext_words<Rec<CODE>::BITS, Rec<CODE>::NW>(wr, __shfl(wr[0], L.src));
            const FoldK k = consts_fold(dw, sgm);
            static_for<4>([&](auto mm) {
                constexpr int MM = decltype(mm)::value;
                const half8_t b = *(const half8_t*)(xp + MM * 64);
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<true, CODE, MM, 0, BK>(wb, wr, k), b, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<true, CODE, MM, 1, BK>(wb, wr, k), b, acc[1], 0, 0, 0);
            });
        }
        else
        {
            const FoldK k = consts_l2(sgm);
            static_for<4>([&](auto mm) {
                constexpr int MM = decltype(mm)::value;
                const half8_t b = *(const half8_t*)(xp + MM * 64);
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<false, 0, MM, 0, BK>(wb, wr, k), b, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<false, 0, MM, 1, BK>(wb, wr, k), b, acc[1], 0, 0, 0);
            });
        }
    }
}

// MASKOK = false leaves the mask-mode loop out (the caller has made sure that P.flags is null)
// RAW (level 2 without a sign plane only: one affine map for the whole plane): the MFMAs multiply the integers 1024 + S, exact in
// fp16, and the value map w = A (1024 + S) + B is applied once to the sums: sum_k w_k x_k = A sum_k (1024 + S_k) x_k + B sum_k x_k,
// with sum_k x_k from one more MFMA per operand against a row of ones. That removes the packed FMA of every weight pair (32 of the
// loop's ~276 vector instructions per chunk) and, with it, the rounding of each weight to fp16: the result is that of the
// UNROUNDED weights, ~2e-4 (relative, l2) from the product with the exact fp16 weights that the other form and the reference
// compute -- inside the layer's 1e-3, outside the 5e-5 that the exact form holds, hence an option the caller has to ask for.
template <bool RES, int CODE, int BK = 0, bool MASKOK = true, bool RAW = false>
__device__ __forceinline__ void gemv_chunks(const Planes& P, const LaneCtx& L, int NC, float4_t* acc, u32x4 nb)
{
    static_assert(!RAW || BK == 0, "the hoisted value map is built for base window code 0");
    float4_t accx = {0.f, 0.f, 0.f, 0.f};
    // RAW at levels 3 / 4: the value map differs from unit to unit, w = A'_u (1024 + F) + C_u, so it is applied chunk by chunk: the
    // chunk's integer products go to accumulators of their own (zero at the chunk's start) and enter the running sums times A'_u;
    // C_u sum_k x_k comes from two more MFMAs per operand whose A operand is C_u in every place (the rows a lane decodes and the
    // rows it supplies to the MFMA are the same, so its own unit's C_u is the right one). The accumulator rows a lane HOLDS belong
    // to the strip (lane >> 5), whose A' it fetches from a lane that decodes that strip.
    const int lane_of_out_strip = (int)((threadIdx.x & 0x37u) | ((threadIdx.x >> 2) & 8u));
    const half8_t ones = {(_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1, (_Float16)1};
    if constexpr (RES && MASKOK)
        if (P.flags) { gemv_chunks_masked<CODE, BK>(P, L, NC, acc, nb); return; }     // block-uniform
    constexpr int NW = RES ? Rec<CODE>::NW : 1;
    uint32_t nr[NW + 2] = {0}, ndw = 0, nvar = 0;
    if constexpr (RES) { load_record<CODE>(nr, P.res, L.rec0, L.nrec); ndw = P.dw[L.unit0]; }
    if (P.var) nvar = P.var[L.unit0];
    for (int c = 0; c < NC; ++c)
    {
        progress_priority(c, NC);
        uint32_t wb[6], wr[NW + 2];
        wb[0] = nb.x; wb[1] = nb.y; wb[2] = nb.z; wb[3] = nb.w;
#pragma unroll
        for (int i = 0; i < NW; ++i) wr[i] = nr[i];
        const uint32_t dw = ndw, var = nvar;
        if (c + 1 < NC)                                         // prefetch the next chunk's records
        {
            nb = load_base<BK>(P, L.rec0 + (size_t)(c + 1) * 32, L.nrec);
            if constexpr (RES) { load_record<CODE>(nr, P.res, L.rec0 + (size_t)(c + 1) * 32, L.nrec); ndw = P.dw[L.unit0 + c + 1]; }
            if (P.var) nvar = P.var[L.unit0 + c + 1];
        }
        ext_base<BK>(wb, __shfl(wb[0], L.src));
        const uint32_t sgm = ((var >> L.g) & 1u) * 0x80008000u;
        FoldK k;
        if constexpr (RES)
        {
            prepare_record<CODE>(wr);
            ext_words<Rec<CODE>::BITS, Rec<CODE>::NW>(wr, __shfl(wr[0], L.src));
            k = consts_fold(dw, sgm);
        }
        else k = consts_l2(sgm);
        const char* xp = L.xs + c * L.xstep;
        if constexpr (RAW && RES)
        {
            float4_t c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};
            const u32x4 cu = {k.C2, k.C2, k.C2, k.C2};
            const half8_t cop = __builtin_bit_cast(half8_t, cu);
            static_for<4>([&](auto mm) {
                constexpr int MM = decltype(mm)::value;
                const half8_t b = *(const half8_t*)(xp + MM * 64);
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<RES, CODE, MM, 0, BK, true>(wb, wr, k), b, c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<RES, CODE, MM, 1, BK, true>(wb, wr, k), b, c1, 0, 0, 0);
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cop, b, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cop, b, acc[1], 0, 0, 0);
            });
            const float Amine = (float)__builtin_bit_cast(_Float16, (uint16_t)(k.A2 & 0xFFFFu));
            const float Aout = __shfl(Amine, lane_of_out_strip);
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                acc[0][i] = __builtin_fmaf(Aout, c0[i], acc[0][i]);
                acc[1][i] = __builtin_fmaf(Aout, c1[i], acc[1][i]);
            }
        }
        else
            static_for<4>([&](auto mm) {
                constexpr int MM = decltype(mm)::value;
                const half8_t b = *(const half8_t*)(xp + MM * 64);
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<RES, CODE, MM, 0, BK, RAW>(wb, wr, k), b, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_operand<RES, CODE, MM, 1, BK, RAW>(wb, wr, k), b, acc[1], 0, 0, 0);
                if constexpr (RAW) accx = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, b, accx, 0, 0, 0);
            });
    }
    if constexpr (RAW && !RES)
    {   // every row of accx holds the token's sum of x over the k-slice; A and B as the fp32 values of the fp16 constants
        const float A = 0.00676727294921875f /* fp16 0x1eee = 1774 / 2^18 */, B = -10.3828125f /* fp16 0xc931 */;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            acc[0][i] = __builtin_fmaf(A, acc[0][i], B * accx[i]);
            acc[1][i] = __builtin_fmaf(A, acc[1][i], B * accx[i]);
        }
    }
}


}  // namespace nq
