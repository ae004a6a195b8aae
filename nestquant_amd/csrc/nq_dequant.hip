// Dense decode of trellis planes to the rotated-domain fp16 weight matrix [N][K].
//   nq_dequant_k   : one projection of one expert (the reference's NQ_WDUMP debug dump, sm120/nqmoe.cu:246-288,852-853)
//   nq_pf_decode_k : G experts, both projections (reference nq_pf_decode, sm120/nqmoe.cu:1013-1080)
// A wavefront decodes two adjacent units (64 records = 1 KiB of base codes, one coalesced load), stages the 2 x 16 x 128
// fp16 tile in LDS and writes 256-byte row segments. HBM-bound on the fp16 writes: 2 B written per 0.25-0.5 B read.
#include "nq_decode.hpp"
#include "nq_host.hpp"

namespace nq {

constexpr int TS = 68;                        // LDS tile row stride in 32-bit words (64 + 4: conflict-free pair stores)

template <bool RES, int CODE, int BK>
__device__ __forceinline__ void decode_to_tile(const uint32_t* wb, const uint32_t* wr, const FoldK& k, uint32_t* tile, int lane32)
{
    const int g = lane32 >> 2, t4 = lane32 & 3;
#pragma unroll
    for (int t = 0; t < 8; ++t)
    {
        uint32_t a[4];
        // a switch keeps every window offset a compile-time constant while t stays a loop variable
        switch (t)
        {
#define NQ_T(T) case T: a[0] = weight_pair<RES, CODE, 8 * T + 0, 8 * T + 1, BK>(wb, wr, k); \
                        a[1] = weight_pair<RES, CODE, 8 * T + 2, 8 * T + 3, BK>(wb, wr, k); \
                        a[2] = weight_pair<RES, CODE, 8 * T + 4, 8 * T + 5, BK>(wb, wr, k); \
                        a[3] = weight_pair<RES, CODE, 8 * T + 6, 8 * T + 7, BK>(wb, wr, k); break;
            NQ_T(0) NQ_T(1) NQ_T(2) NQ_T(3) NQ_T(4) NQ_T(5) NQ_T(6) default: NQ_T(7)
#undef NQ_T
        }
        // pair index pp = 4 t + r: row g + 8 (r & 1), columns 16 t + 2 t4 + 8 (r >> 1) + {0, 1}
#pragma unroll
        for (int r = 0; r < 4; ++r) tile[(g + 8 * (r & 1)) * TS + 8 * t + t4 + 4 * (r >> 1)] = a[r];
    }
}

// decode unit `unit` of projection planes P (level lv) into tile; all 64 lanes of the wave call this together
template <int BK>
__device__ __forceinline__ void decode_unit_bk(const Planes& P, int lv, size_t unit, size_t nrec, int C, uint32_t* tile, int lane);
__device__ __forceinline__ void decode_unit(const Planes& P, int lv, size_t unit, size_t nrec, int C, uint32_t* tile, int lane)
{
    dispatch_base(P.bcode, [&](auto bk) { decode_unit_bk<decltype(bk)::value>(P, lv, unit, nrec, C, tile, lane); });
}

template <int BK>
__device__ __forceinline__ void decode_unit_bk(const Planes& P, int lv, size_t unit, size_t nrec, int C, uint32_t* tile, int lane)
{
    const int lane32 = lane & 31;
    const int src = (lane & ~3) | ((lane + 1) & 3);           // next lane of the ring
    uint32_t wb[6];
    {
        const u32x4 v = load_base<BK>(P, unit * 32 + lane32, nrec);
        wb[0] = v.x; wb[1] = v.y; wb[2] = v.z; wb[3] = v.w;
        ext_base<BK>(wb, __shfl(wb[0], src));
    }
    const uint32_t sgm = P.var ? (((uint32_t)P.var[unit] >> (lane32 >> 2)) & 1u) * 0x80008000u : 0u;
    size_t runit = unit, rnrec = nrec;                          // residual unit / records: compact in mask mode
    bool on = lv != 2;
    if (on && P.flags)
    {   // the two halves of a wavefront may sit in different strips or chunks: this branch may diverge between them, and the
        // ring neighbour of a lane is always in its own half
        const size_t strip = unit / C;
        const MaskedUnit m = masked_unit(P.flags[strip], strip, (int)(unit - strip * C), nrec / 32 / C);
        on = m.on; runit = m.unit; rnrec = m.nrec;
    }
    if (!on)
    {
        decode_to_tile<false, 0, BK>(wb, wb, consts_l2(sgm), tile, lane32);
        return;
    }
    const uint32_t dw = P.dw[runit];
    const FoldK k = consts_fold(dw, sgm);
    dispatch_code(P.code, [&](auto tag) {
        constexpr int CODE = decltype(tag)::value;
        uint32_t wr[Rec<CODE>::NW + 2];
        load_record<CODE>(wr, P.res, runit * 32 + lane32, rnrec);
        prepare_record<CODE>(wr);
        ext_words<Rec<CODE>::BITS, Rec<CODE>::NW>(wr, __shfl(wr[0], src));
        decode_to_tile<true, CODE, BK>(wb, wr, k, tile, lane32);
    });
}

__device__ __forceinline__ void store_tile(const uint32_t* tile, _Float16* out, int K, int lane)
{
    // 16 rows x 256 B; each lane moves 16 B, 16 lanes per row
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const int i = lane + 64 * j, row = i >> 4, c8 = i & 15;
        *(uint4*)(out + (size_t)row * K + c8 * 8) = *(const uint4*)(tile + row * TS + c8 * 4);
    }
}

// planes of projection `mode` (0 gate|up [2I][H], 1 down [H][I]) of the expert described by ent -> out
__device__ __forceinline__ void dequant_body(const int64_t* ent, int mode, int lv, int H, int I, _Float16* out,
                                             int pair, uint32_t* tiles)
{
    const int lane = threadIdx.x & 63, half = lane >> 5;
    const int N = mode == 0 ? 2 * I : H, K = mode == 0 ? H : I, C = K / 128;
    const size_t nunits = (size_t)(N / 16) * C, nrec = nunits * 32;
    size_t unit = (size_t)pair * 2 + half;
    const bool live = unit < nunits;
    if (!live) unit = nunits - 1;                              // keep the wave convergent for the shuffles
    uint32_t* tile = tiles + half * 16 * TS;
    _Float16* dst = out + (size_t)(unit / C) * 16 * K + (size_t)(unit % C) * 128;
    if (lv <= 0)
    {
        if (live) for (int i = lane & 31; i < 256; i += 32) *(uint4*)(dst + (size_t)(i >> 4) * K + (i & 15) * 8) = make_uint4(0, 0, 0, 0);
        return;
    }
    const Planes P = planes_of(ent, mode);
    decode_unit(P, lv, unit, nrec, C, tile, lane);
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    // each half-wave wrote its own tile; the whole wave now drains both tiles
    for (int h = 0; h < 2; ++h)
    {
        const size_t u = (size_t)pair * 2 + h;
        if (u >= nunits) break;
        store_tile(tiles + h * 16 * TS, out + (size_t)(u / C) * 16 * K + (size_t)(u % C) * 128, K, lane);
    }
}

__global__ void __launch_bounds__(256) nq_dequant_k(const int64_t* __restrict__ ent, int mode, int level, int H, int I, _Float16* out)
{
    __shared__ __align__(16) uint32_t tiles[4][2 * 16 * TS];
    const int warp = threadIdx.x >> 6;
    const int N = mode == 0 ? 2 * I : H, K = mode == 0 ? H : I;
    const int npairs = ((N / 16) * (K / 128) + 1) / 2;
    const int pair = blockIdx.x * 4 + warp;
    if (pair >= npairs) return;                                 // wave-uniform
    const int lv = level ? level : (int)ent[0];
    dequant_body(ent, mode, lv, H, I, out, pair, tiles[warp]);
}

// grid (ceil(pairs / 4), G, 2): Wgu [G][2I][H], Wdn [G][H][I]; level from the live table row; level <= 0 -> zeros
__global__ void __launch_bounds__(256) nq_pf_decode_k(const int64_t* __restrict__ table, const int32_t* __restrict__ experts,
                                                       _Float16* Wgu, _Float16* Wdn, int H, int I)
{
    __shared__ __align__(16) uint32_t tiles[4][2 * 16 * TS];
    const int mode = blockIdx.z, gi = blockIdx.y, warp = threadIdx.x >> 6;
    const int N = mode == 0 ? 2 * I : H, K = mode == 0 ? H : I;
    const int npairs = ((N / 16) * (K / 128) + 1) / 2;
    const int pair = blockIdx.x * 4 + warp;
    if (pair >= npairs) return;
    const int64_t* ent = table + (int64_t)experts[gi] * TBL_W;
    _Float16* out = (mode == 0 ? Wgu : Wdn) + (size_t)gi * N * K;
    dequant_body(ent, mode, (int)ent[0], H, I, out, pair, tiles[warp]);
}

int launch_dequant(const int64_t* row, int proj, int level, int H, int I, void* out, hipStream_t st)
{
    const int N = proj == 0 ? 2 * I : H, K = proj == 0 ? H : I;
    const int npairs = ((N / 16) * (K / 128) + 1) / 2;
    nq_dequant_k<<<dim3((npairs + 3) / 4), 256, 0, st>>>(row, proj, level, H, I, (_Float16*)out);
    NQ_LAUNCH_CHECK("nq_dequant");
    return 0;
}

int launch_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu, void* Wdn, int H, int I, hipStream_t st)
{
    if (!G) return 0;
    const int pgu = ((2 * I / 16) * (H / 128) + 1) / 2, pdn = ((H / 16) * (I / 128) + 1) / 2;
    const int np = pgu > pdn ? pgu : pdn;
    nq_pf_decode_k<<<dim3((np + 3) / 4, G, 2), 256, 0, st>>>(table, experts, (_Float16*)Wgu, (_Float16*)Wdn, H, I);
    NQ_LAUNCH_CHECK("nq_pf_decode");
    return 0;
}

}  // namespace nq
