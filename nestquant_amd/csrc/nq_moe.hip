// Decode-path MoE layer for 1..8 tokens (reference sm120/nqmoe.cu:375-449 route, :493-771 do_item, :858-907 moe_forward,
// :908-929 mailbox). Three launches on one stream, every routing / level / pointer decision read on the device:
//
//   nq_prep_k        routing once per call (picks -> runs of distinct experts, their table rows -> run headers in RouteWs) and
//                 the rotation of the activations of every active pick (x * su -> Hadamard-128 -> fp16, B-operand order).
//   nq_gemv_k<0, *>  gate|up: grid (strip-pair blocks, k-slices, runs). A run = one distinct routed expert + the tokens that
//                 picked it. The block copies those tokens' rotated x into LDS, then every wavefront decodes the records of
//                 two strips chunk by chunk straight into MFMA A operands (v_mfma_f32_16x16x32_f16, tokens as the N
//                 dimension) and writes its k-slice partial sums. In a call of both launches that is all; in a gate|up-only
//                 call (and for rows with a low-rank plane or the 512-wide rotation) the block that arrives last at a
//                 (run, 128-column group) counter finishes the group: Hadamard * sv, SwiGLU, * su_d, Hadamard -> h fp16.
//   nq_gemv_k<1, *>  down: staging forms h from the gate|up partial sums (or reads it), same decode loop; the last block of a
//                 128-row output group (counter over all runs) combines:
//                 out[b] = sum_k rw[b,k] * sv_o (.) Hadamard(sum of partials).
//   A call with a mailbox: one workgroup of an extra plane of blocks of the call's LAST projection launch applies it
//   (table <- stage, device applied <- seq); the NEXT routing launch publishes applied to the host. See mailbox_apply.
//
// Lane mapping of the GEMV (wave64): lane = 16 * t4 + 8 * ss + g decodes the record of lane (4 g + t4) of unit
// (strip0 + ss, chunk); it holds 32 weights of row g and 32 of row g + 8, in columns 16 t + 2 t4 + {0,1,8,9}. An MFMA
// 16x16x32 takes 8 fp16 per lane: lanes with equal (ss, g) and different t4 are the k-groups of one A row, so the decoded
// pairs are A operands as they leave the decoder, with no cross-lane movement. The B operand (tokens) comes from LDS,
// staged in the matching column order. Partial sums instead of float atomics make the layer output bitwise repeatable;
// the arrival counters are zero on entry and are reset by the block that consumes them.
#include "nq_tile.hpp"
#include "nq_host.hpp"
#include <algorithm>
#include <mutex>
#include "../../include/nq_moe_hip.h"

namespace nq {

// Partial sums cross workgroups (and XCDs, whose L2s are not coherent with each other) inside one kernel. They are
// written and read with device-scope relaxed atomics (sc1: write-through / read-through to the device coherence point)
// and ordered by "all my stores are acknowledged (vmcnt 0) -> bump the group's arrival counter". A full device-scope
// fence would also be correct but writes back and invalidates the whole L2 once per workgroup, which costs several times
// the kernel's own run time.
// The compiler waits after every atomic load, which serialises the finisher's reads (one memory round trip per k-slice),
// so the loads are issued as a batch of sc0 sc1 loads and waited for once; the wait names the destination registers so
// that no use can move above it.
__device__ __forceinline__ void st_dev4(float* p, float4_t v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st_dev2(float* p, float2 v)
{
    asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ float2 ld_dev2_issue(const float* p)
{
    float2 v;
    asm volatile("global_load_dwordx2 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void ld_wait(float2& a, float2& b, float2& c, float2& d)
{
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) :: "memory");
}
// sums over k-slices y of the two floats at p[q] + y * stride, for NR rows q at once: the reads of all rows are in flight
// together, four slices per row at a time (device-coherent reads)
template <int NR>
__device__ __forceinline__ void sum_partials(const float* const* p, size_t stride, int NY, float2* out)
{
#pragma unroll
    for (int q = 0; q < NR; ++q) out[q] = make_float2(0.f, 0.f);
    for (int y = 0; y < NY; y += 4)
    {
        float2 v[NR][4];
#pragma unroll
        for (int q = 0; q < NR; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) v[q][i] = ld_dev2_issue(p[q] + (size_t)(y + i < NY ? y + i : y) * stride);
#pragma unroll
        for (int q = 0; q < NR; ++q) ld_wait(v[q][0], v[q][1], v[q][2], v[q][3]);
#pragma unroll
        for (int q = 0; q < NR; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) if (y + i < NY) { out[q].x += v[q][i].x; out[q].y += v[q][i].y; }
    }
}

// ---- caller dtypes: the casts a caller would otherwise launch as separate kernels (x.half(), ids.long(), w.half(),
// out.to(x.dtype); reference sm120/serve/nq_vllm.py:522,560,573) happen at the loads and the final store, with the same
// roundings: activations and routing weights pass through fp16, the fp32 result is rounded once to the output type.
constexpr int DT_BF16 = 1, DT_F32 = 2, DT_I32 = 1, DT_OUT_F16 = 1, DT_OUT_BF16 = 2;   // 0 = the default type of each argument (fp16, int64, fp32 out)
__device__ __forceinline__ float bf16_to_f(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float f)           // round to nearest even; NaN stays NaN
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ long long sel_at(const MoeArgs& a, int i)
{
    return a.sel_dtype == DT_I32 ? (long long)((const int32_t*)a.sel)[i] : (long long)((const int64_t*)a.sel)[i];
}
__device__ __forceinline__ float rw_at(const MoeArgs& a, int i)   // the weight as fp16 would hold it
{
    if (a.rw_dtype == DT_BF16) return (float)(_Float16)bf16_to_f(((const uint16_t*)a.rw)[i]);
    if (a.rw_dtype == DT_F32) return (float)(_Float16)((const float*)a.rw)[i];
    return (float)((const _Float16*)a.rw)[i];
}
__device__ __forceinline__ half2_t x2_at(const MoeArgs& a, size_t i)   // x[i], x[i + 1] (i even) as fp16
{
    if (a.x_dtype == DT_BF16)
    {
        const uint32_t v = *(const uint32_t*)((const uint16_t*)a.x + i);
        return half2_t{(_Float16)bf16_to_f((uint16_t)v), (_Float16)bf16_to_f((uint16_t)(v >> 16))};
    }
    if (a.x_dtype == DT_F32) { const float2 v = *(const float2*)((const float*)a.x + i); return half2_t{(_Float16)v.x, (_Float16)v.y}; }
    return *(const half2_t*)((const _Float16*)a.x + i);
}
__device__ __forceinline__ void out2_store(const MoeArgs& a, size_t i, float v0, float v1)   // out[i], out[i + 1] (i even)
{
    if (a.out_dtype == DT_OUT_F16) { half2_t h; h.x = (_Float16)v0; h.y = (_Float16)v1; *(half2_t*)((_Float16*)a.out + i) = h; }
    else if (a.out_dtype == DT_OUT_BF16) *(uint32_t*)((uint16_t*)a.out + i) = (uint32_t)f_to_bf16(v0) | ((uint32_t)f_to_bf16(v1) << 16);
    else *(float2*)((float*)a.out + i) = make_float2(v0, v1);
}

constexpr int MAXTOK = 8;                      // tokens of one run = tokens of one call (the MFMA N dimension holds 16)
// What the projection launches need to know about run r, written once per call by nq_prep_k (one per projection: the plane
// addresses differ). A run = one distinct routed expert + the tokens that picked it.
struct alignas(64) RunHdr
{
    Planes P;                     // this projection of the run's expert
    const _Float16* signs;        // su_g | sv_g | sv_u | su_d | sv_o | su_u
    const _Float16* lr; const _Float16* lr4;      // low-rank plane of the run's expert (lr == nullptr: none)
    int level, ntok;
    int had;                      // width of the Hadamard on the down projection's input: 128 or 512
    int rg, rd;
    int q0;                       // rotated activations of the run's token j: row q0 + j of MoeArgs::xrot
    unsigned char slot[MAXTOK];   // pick index (token * topk + k) of the run's tokens
    __device__ __forceinline__ int slot_of(int j) const       // by shifts: a run-time index into slot[] would put the header into scratch memory
    {
        unsigned long long v;
        __builtin_memcpy(&v, slot, 8);
        return (int)((v >> (8 * j)) & 0xFFull);
    }
};
struct PickInfo                   // per pick, for the down launch's combine
{
    float w[64];                  // routing weight, 0 for picks that contribute nothing
    const _Float16* signs[64];
    const _Float16* lr[64]; const _Float16* lr4[64]; unsigned char rg[64], rd[64], lv[64];
};
struct RouteWs { int nruns; int ny_gu; int pad[14]; PickInfo picks; RunHdr run[2][64]; };   // ny_gu: k-slices of the gate|up launch that filled part_gu
static_assert(sizeof(RunHdr) == 128, "RunHdr is read as 32 scalar words");
static_assert(sizeof(RouteWs) <= NQ_ROUTE_WS_BYTES, "NQ_ROUTE_WS_BYTES in include/nq_moe_hip.h is too small");

// ---- mailbox rows: 20 int64 read past every cache (a copy engine may have written them while kernels ran), all in flight
// together and waited for once (the compiler would wait after each atomic load: twenty round trips)
__device__ __forceinline__ void ld_sys_row(const int64_t* p, int64_t* f)
{
#pragma unroll
    for (int i = 0; i < TBL_W; ++i) asm volatile("global_load_dwordx2 %0, %1, off offset:%2 sc0 sc1" : "=v"(f[i]) : "v"(p), "n"(8 * i) : "memory");
#pragma unroll
    for (int i = 0; i < TBL_W; i += 4) asm volatile("s_waitcnt vmcnt(0)" : "+v"(f[i]), "+v"(f[i + 1]), "+v"(f[i + 2]), "+v"(f[i + 3]) :: "memory");
}

// ---- routing dedup: picks -> runs (refined experts first, then by first occurrence); slots in pick order ----------------
// One wavefront per workgroup of nq_prep_k; lane s owns pick s (S <= 64). A run takes at most one pick per token: a token
// that names the same expert twice opens a second run of that expert, so a run never has more than B tokens. Every lane
// requests all fields of its own pick's table row together, so the leader's fields cost no second round trip. The routing
// reads the table and nothing else: no kernel writes the table while a routing launch runs (the mailbox of a call is applied
// by its last projection launch, see mailbox_apply), so every workgroup of the launch sees the same rows and the rows cannot
// be torn.
struct PrepRows { int nq; unsigned char tok[64]; const _Float16* signs[64]; };    // LDS: the rows of xrot, one per active pick
__device__ __forceinline__ void route(const MoeArgs& a, RouteWs* W, int lane, bool writer, PrepRows* Q)
{
    const int S = a.B * a.topk;
    int e = -1, lv = 0; bool ok = false, inrange = false;
    int64_t f[TBL_W];
#pragma unroll
    for (int i = 0; i < TBL_W; ++i) f[i] = 0;
    if (lane < S)
    {
        const long long ee = sel_at(a, lane);
        if (ee >= 0 && ee < a.E)
        {
            e = (int)ee; inrange = true;
            const int64_t* ent = a.table + (size_t)e * TBL_W;
#pragma unroll
            for (int i = 0; i < TBL_W; ++i) f[i] = ent[i];
            lv = (int)f[0];
            ok = rw_at(a, lane) != 0.f && lv > 0;
        }
    }
    if (writer && a.hits && inrange && rw_at(a, lane) != 0.f)
        __hip_atomic_fetch_add(a.hits + e, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const int level = a.force_level ? a.force_level : lv;
    // Runs of refined experts (level 3, 4: twice the decode work per chunk) are numbered before the level-2 ones, each group
    // by first occurrence: workgroups are dispatched in run order, so the long ones start first and spread over all CUs, and
    // the short ones fill in around them (gate|up 44.0 -> 42.6 us, down 28.4 -> 27.2 us on the benchmark's level mix).
    const unsigned long long okm = __ballot(ok);
    const unsigned long long heavy = __ballot(ok && level > 2);
    const unsigned long long below = (1ull << lane) - 1ull;
    const int tok = lane / a.topk, sh = tok * a.topk;
    const unsigned long long mytok = sh < 64 ? (a.topk >= 64 ? ~0ull : ((1ull << a.topk) - 1ull)) << sh : 0ull;
    int r = 0, cum = 0;
    int my_run = -1, my_pos = 0, my_ntok = 0, my_q0 = 0;         // the run this lane's pick went into, its place there; for the first lane of a run: its size
    for (int pass = 0; pass < 2; ++pass)
    {
        unsigned long long rem = pass == 0 ? heavy : okm & ~heavy;
        while (rem)
        {
            const int leader = __ffsll((long long)rem) - 1;
            const int ev = __shfl(e, leader);
            const unsigned long long same = __ballot(((rem >> lane) & 1ull) && e == ev);
            const unsigned long long m = __ballot(((same >> lane) & 1ull) && (same & mytok & below) == 0ull);   // first pick per token
            if ((m >> lane) & 1ull)
            {
                my_run = r; my_pos = __popcll(m & below); my_ntok = __popcll(m); my_q0 = cum;
                Q->tok[cum + my_pos] = (unsigned char)tok; Q->signs[cum + my_pos] = (const _Float16*)f[9];
            }
            rem &= ~m; ++r; cum += __popcll(m);
        }
    }
    if (lane == 0) Q->nq = cum;
    if (!writer) return;
    // the headers, after the numbering: every lane holds its own pick's row, so the first lanes of all runs write their runs'
    // headers side by side (inside the loop above the same stores would be issued once per run, one lane at a time)
    if (my_run >= 0)
    {
        W->run[0][my_run].slot[my_pos] = (unsigned char)lane; W->run[1][my_run].slot[my_pos] = (unsigned char)lane;
        if (my_pos == 0)
        {
#pragma unroll
            for (int mode = 0; mode < 2; ++mode)
            {
                RunHdr& R = W->run[mode][my_run];
                const int o = mode == 0 ? 1 : 5;
                R.P.base = (gp_u4)f[o]; R.P.res = (gp_u8)f[o + 1]; R.P.dw = (gp_u32)f[o + 2]; R.P.flags = (gp_u64)f[o + 3];
                R.P.var = (gp_u8)f[12 + mode]; R.P.code = (int)f[10 + mode]; R.P.bcode = (int)((f[19] >> (8 * mode)) & 0xFF);
                R.signs = (const _Float16*)f[9];
                R.level = level;
                R.had = f[18] == 512 ? 512 : 128;
                R.lr = (const _Float16*)f[14]; R.lr4 = (const _Float16*)f[15]; R.rg = (int)f[16]; R.rd = (int)f[17];
                R.ntok = my_ntok; R.q0 = my_q0;
            }
        }
    }
    PickInfo& K = W->picks;
    K.w[lane] = ok ? rw_at(a, lane) : 0.f; K.signs[lane] = (const _Float16*)f[9];
    K.lr[lane] = (const _Float16*)f[14]; K.lr4[lane] = (const _Float16*)f[15];
    K.rg[lane] = (unsigned char)f[16]; K.rd[lane] = (unsigned char)f[17]; K.lv[lane] = (unsigned char)level;
    if (lane == 0) W->nruns = r;
}

// The mailbox of a layer call (reference nq_mailbox, sm120/nqmoe.cu:908-923, a launch of its own there), in two halves that
// keep the reference's rule "once applied_host[e] == seq[e] no later kernel can reference the old row's slot":
//   apply   -- one workgroup of the call's LAST projection launch: for every e with seq[e] != applied[e], table[e] <- stage[e]
//              and the device copy applied[e] <- seq[e]. This is the call's only reading of seq / stage (a single observer),
//              it comes after the call's routing launch has ended (the routing of this call used the old rows, identically in
//              all its workgroups), and neither projection launch reads the table, so a row cannot be torn and no two parts of
//              the call can disagree about a row. Nothing is published to the host here: this call's launches may still be
//              decoding from the slot that the old row names.
//   publish -- the routing launch of the NEXT call (publish_applied): applied_host[e] <- applied[e] for every e. It runs after
//              every launch of the earlier calls has ended (stream order), and from this routing launch on every launch works
//              from rows read after the apply, so a slot released by a published row is no longer referenced by anything.
// A row whose seq lands while call n runs is therefore used from call n + 1 on and published at the head of call n + 1, which is
// when the reference's mailbox launch at the head of call n + 1 would have applied and published it.
__device__ __forceinline__ void mailbox_apply(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int E)
{
    for (int e = threadIdx.x; e < E; e += blockDim.x)
    {
        const int32_t ap = applied[e];
        const int32_t sq = __hip_atomic_load(seq + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (sq == ap) continue;                                  // the row is requested only after seq has been seen (the copy
        int64_t row[TBL_W];                                      // stream wrote the row before seq)
        ld_sys_row(stage + (size_t)e * TBL_W, row);
#pragma unroll
        for (int i = 0; i < TBL_W; ++i) table[(size_t)e * TBL_W + i] = row[i];
        applied[e] = sq;                                         // read again only by later launches on this stream
    }
}
// host mirror of the device's applied[]: plain re-publication of every entry (values only ever grow, equal values are harmless)
__device__ __forceinline__ void publish_applied(const int32_t* applied, int32_t* applied_host, int E, int first, int step)
{
    for (int e = first; e < E; e += step)
        __hip_atomic_store(applied_host + e, applied[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// First launch of every layer call. Every workgroup repeats the routing (its first wavefront; workgroup 0 writes the result:
// run headers for both projection launches, which then read one header each instead of repeating the dependent loads
// sel -> table row in every one of their ~1800 workgroups, the per-pick data of the combine, the hits export); then the
// wavefronts of the grid share the rotation of the activations: one task per (active pick q, gate or up, 128-column chunk):
// xrot[q][gate|up][chunk] = fp16(Hadamard-128(x[token] * su)) in the MFMA B-operand column order, which the gate|up launch
// copies into LDS (before, each of the 32 row blocks of a run repeated these rotations: 9 % of the launch's vector
// instructions). With a mailbox in the call the other three wavefronts of workgroup 0 first publish what earlier calls applied
// (publish_applied); nothing here reads seq or stage and nothing writes the table.
__global__ void __launch_bounds__(256) nq_prep_k(MoeArgs a)
{
    __shared__ PrepRows Q;
    const int lane = threadIdx.x & 63;
    if (threadIdx.x < 64) route(a, a.route, lane, blockIdx.x == 0, &Q);
    else if (blockIdx.x == 0 && a.mb_table && a.mb_applied_host) publish_applied(a.mb_applied, a.mb_applied_host, a.E, threadIdx.x - 64, 192);
    __syncthreads();
    // workgroup 0 has the result to write (it ends ~1 us after the others' routing): with more than one workgroup in the grid the
    // rotation tasks go to the others, so that it is not also the last to finish
    const int C = a.H / 128, ntask = Q.nq * 2 * C, nrot = gridDim.x > 1 ? gridDim.x - 1 : 1, rot = gridDim.x > 1 ? (int)blockIdx.x - 1 : 0;
    if (rot < 0) return;
    for (int t = rot * 4 + (threadIdx.x >> 6); t < ntask; t += nrot * 4)
    {
        const int q = t / (2 * C), r = t - q * 2 * C, up = r / C, c = r - up * C, kk = c * 128 + 2 * lane;
        const _Float16* su = Q.signs[q] + (up ? 2 * a.H + 3 * a.I : 0);
        const half2_t xv = x2_at(a, (size_t)Q.tok[q] * a.H + kk), sv = *(const half2_t*)(su + kk);
        float v0 = (float)xv.x * (float)sv.x, v1 = (float)xv.y * (float)sv.y;
        wht128(v0, v1, lane);
        _Float16* dst = a.xrot + ((size_t)q * 2 + up) * a.H + c * 128;
        dst[bop_index(2 * lane)] = (_Float16)v0; dst[bop_index(2 * lane + 1)] = (_Float16)v1;
    }
}

// finisher of gate|up for (run z, 128-column group grp): h[slot] = fp16(WHT(silu(g) * u * su_d)), g = WHT(sum_y part_g) * sv_g.
// With a 512-wide Hadamard on the down projection's input (in_had_down, reference sm120/nqmoe.cu:36-40,673-712;
// WHT_512 = H_4 (x) WHT_128 / 2) the group's WHT_128 result goes, in fp32, into the gate columns of k-slice 0 that this
// finisher has just consumed, and the last of the four groups of a 512-column block combines them with the Sylvester H_4
// and rounds to fp16 once.
__device__ __forceinline__ void finish_gu(const MoeArgs& a, const RunHdr& R, float (*zl)[4], int z, int grp, int NY, int warp, int SB, int lane, int& last)
{
    const _Float16 *sv_g = R.signs + a.H, *sv_u = sv_g + a.I, *su_d = sv_u + a.I;
    const int S = a.B * a.topk, col = grp * 128 + 2 * lane;
    const bool wide = R.had == 512;
    // low-rank plane (reference sm120/nqmoe.cu:41-45,611-645): lr = V_gu [rg][H] | U2_g [rg][I] | U2_u [rg][I] | V_dn [rd][I] |
    // U2_d [rd][H], lr4 = U4_g | U4_u | U4_d (level 4 only). z = x V_gu^T over the raw activations, one wavefront per token
    const bool lowrank = R.lr != nullptr;                        // block-uniform
    const int rg = lowrank ? R.rg : 0, rd = lowrank ? R.rd : 0;
    if (rg)
    {
        for (int j = warp; j < R.ntok; j += SB)
        {
            const int tok = R.slot_of(j) / a.topk;
            float zz[4] = {0.f, 0.f, 0.f, 0.f};
            for (int k = 2 * lane; k < a.H; k += 128)
            {
                const half2_t xv = x2_at(a, (size_t)tok * a.H + k);
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (r < rg) { const half2_t vv = *(const half2_t*)(R.lr + (size_t)r * a.H + k); zz[r] += (float)xv.x * (float)vv.x + (float)xv.y * (float)vv.y; }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
#pragma unroll
                for (int m = 32; m >= 1; m >>= 1) zz[r] += __shfl_xor(zz[r], m);
                if (lane == 0) zl[j][r] = zz[r];
            }
        }
        __syncthreads();
    }
    const _Float16* U2g = R.lr + (size_t)rg * a.H, *U2u = U2g + (size_t)rg * a.I, *Vd = U2u + (size_t)rg * a.I;
    const _Float16* U4g = R.lr4, *U4u = U4g + (size_t)rg * a.I;
    for (int j = warp; j < R.ntok; j += SB)
    {
        const int s = R.slot_of(j);
        const float* p = a.part_gu + (size_t)s * 2 * a.I + col;
        const half2_t svg = *(const half2_t*)(sv_g + col), svu = *(const half2_t*)(sv_u + col), sud = *(const half2_t*)(su_d + col);
        const float* const rows2[2] = {p, p + a.I};
        float2 pq[2];
        sum_partials<2>(rows2, (size_t)S * 2 * a.I, NY, pq);
        float g0 = pq[0].x, g1 = pq[0].y, u0 = pq[1].x, u1 = pq[1].y;
        wht128(g0, g1, lane); wht128(u0, u1, lane);
        g0 *= (float)svg.x; g1 *= (float)svg.y; u0 *= (float)svu.x; u1 *= (float)svu.y;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (r < rg)
            {
                const float zr = zl[j][r];
                half2_t ug = *(const half2_t*)(U2g + (size_t)r * a.I + col), uu = *(const half2_t*)(U2u + (size_t)r * a.I + col);
                g0 += zr * (float)ug.x; g1 += zr * (float)ug.y; u0 += zr * (float)uu.x; u1 += zr * (float)uu.y;
                if (R.level == 4)
                {
                    ug = *(const half2_t*)(U4g + (size_t)r * a.I + col); uu = *(const half2_t*)(U4u + (size_t)r * a.I + col);
                    g0 += zr * (float)ug.x; g1 += zr * (float)ug.y; u0 += zr * (float)uu.x; u1 += zr * (float)uu.y;
                }
            }
        const float sw0 = g0 / (1.f + __expf(-g0)) * u0, sw1 = g1 / (1.f + __expf(-g1)) * u1;
        if (rd)
        {   // this group's share of z_d = sw V_dn^T, summed over the groups by the down combine
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                float t = 0.f;
                if (r < rd) { const half2_t vv = *(const half2_t*)(Vd + (size_t)r * a.I + col); t = sw0 * (float)vv.x + sw1 * (float)vv.y; }
#pragma unroll
                for (int m = 32; m >= 1; m >>= 1) t += __shfl_xor(t, m);
                if (lane == 0) a.zd[((size_t)s * (a.I / 128) + grp) * 4 + r] = t;
            }
        }
        float v0 = sw0 * (float)sud.x, v1 = sw1 * (float)sud.y;
        wht128(v0, v1, lane);
        // h = fp16 of the fp32 rotation result (two roundings, as the reference's kernel and its torch restatement). Left alone,
        // the compiler merges the rotation's last multiply into the conversion (v_fma_mixlo_f16: one rounding) at some call
        // sites and not at others; this one and the down launch's staging must give the same bits.
        asm volatile("" : "+v"(v0), "+v"(v1));
        if (wide) st_dev2(a.part_gu + (size_t)s * 2 * a.I + col, make_float2(v0, v1));
        else
        {
            half2_t hv; hv.x = (_Float16)v0; hv.y = (_Float16)v1;
            *(half2_t*)(a.h + (size_t)s * a.I + col) = hv;       // read by the next kernel on the stream
        }
    }
    if (!wide) return;                                           // block-uniform
    int* cnt = a.cnt_h + z * (a.I / 128) + grp / 4;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) last = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 3;
    __syncthreads();
    if (!last) return;
    const int c0 = (grp / 4) * 512 + 2 * lane;
    for (int j = warp; j < R.ntok; j += SB)
    {
        const int s = R.slot_of(j);
        float2 w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) w[q] = ld_dev2_issue(a.part_gu + (size_t)s * 2 * a.I + c0 + q * 128);
        ld_wait(w[0], w[1], w[2], w[3]);
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            float h0 = 0.f, h1 = 0.f;
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
            {
                const float sg = (__builtin_popcount(q & pp) & 1) ? -0.5f : 0.5f;
                h0 += sg * w[pp].x; h1 += sg * w[pp].y;
            }
            half2_t hv; hv.x = (_Float16)h0; hv.y = (_Float16)h1;
            *(half2_t*)(a.h + (size_t)s * a.I + c0 + q * 128) = hv;
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// combine of the down projection for output rows [grp * 128, +128): out[b] = sum_k rw[b,k] * sv_o[e] (.) WHT(sum_y part_d[slot])
// picks of a token are spread over the block's wavefronts and reduced through LDS (red: SB * 128 floats)
__device__ __forceinline__ void finish_dn(const MoeArgs& a, const PickInfo& R, int grp, int NY, int warp, int SB, int lane, float* red)
{
    const int S = a.B * a.topk, col = grp * 128 + 2 * lane;
    for (int b = 0; b < a.B; ++b)
    {
        float o0 = 0.f, o1 = 0.f;
        for (int k = warp; k < a.topk; k += 2 * SB)              // two picks of this wavefront at a time, their reads in flight together
        {
            float2 pv[2] = {make_float2(0.f, 0.f), make_float2(0.f, 0.f)};
            float w[2] = {0.f, 0.f};
            half2_t sv[2] = {};
            const float* rows2[2] = {a.part_d, a.part_d};
#pragma unroll
            for (int q = 0; q < 2; ++q)
            {
                const int kq = k + q * SB, s = b * a.topk + kq;
                if (kq >= a.topk || R.w[s] == 0.f) continue;     // what route() saw: no second look at the table
                w[q] = R.w[s]; rows2[q] = a.part_d + (size_t)s * a.H + col;

                sv[q] = *(const half2_t*)(R.signs[s] + a.H + 3 * a.I + col);
            }
            if (w[0] == 0.f && w[1] == 0.f) continue;
            sum_partials<2>(rows2, (size_t)S * a.H, NY, pv);
#pragma unroll
            for (int q = 0; q < 2; ++q)
            {
                float v0 = pv[q].x, v1 = pv[q].y;
                wht128(v0, v1, lane);
                if (w[q] == 0.f) continue;
                v0 *= (float)sv[q].x; v1 *= (float)sv[q].y;
                const int s = b * a.topk + k + q * SB, prd = R.lr[s] ? R.rd[s] : 0;
                if (prd)
                {   // y += (sw V_dn^T) (U2_d [+ U4_d]): z_d summed over the I / 128 groups written by the gate|up finishers
                    const int prg = R.rg[s];
                    const _Float16* U2d = R.lr[s] + (size_t)prg * (a.H + 2 * a.I) + (size_t)prd * a.I;
                    const _Float16* U4d = R.lr4[s] + (size_t)prg * 2 * a.I;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (r < prd)
                        {
                            float zr = 0.f;
                            for (int gq = 0; gq < a.I / 128; ++gq) zr += a.zd[((size_t)s * (a.I / 128) + gq) * 4 + r];
                            half2_t ud = *(const half2_t*)(U2d + (size_t)r * a.H + col);
                            v0 += zr * (float)ud.x; v1 += zr * (float)ud.y;
                            if (R.lv[s] == 4) { ud = *(const half2_t*)(U4d + (size_t)r * a.H + col); v0 += zr * (float)ud.x; v1 += zr * (float)ud.y; }
                        }
                }
                o0 += w[q] * v0; o1 += w[q] * v1;
            }
        }
        red[warp * 128 + 2 * lane] = o0; red[warp * 128 + 2 * lane + 1] = o1;
        __syncthreads();
        if (warp == 0)
        {
            float r0 = 0.f, r1 = 0.f;
            for (int w2 = 0; w2 < SB; ++w2) { r0 += red[w2 * 128 + 2 * lane]; r1 += red[w2 * 128 + 2 * lane + 1]; }
            out2_store(a, (size_t)b * a.H + col, r0, r1);
        }
        __syncthreads();
    }
}

// MODE 0: gate|up (N = 2I, K = H, input x rotated here). MODE 1: down (N = H, K = I, input h).
// grid (N / 32 / SB, C / NC, S); block 64 * SB threads (SB = 1, 2 or 4: a block covers at most one 128-row group);
// dynamic LDS = rows * (NC * 256 + 16) + 256 bytes (>= SB * 512 for the combine), one row per token of the call
// ANYROW = false: the kernel of a layer whose rows are all of the common kind, base window code 0 and no mask-mode flags (the
// host says so, MoeArgs::common_rows). A run whose row is nevertheless of another kind is not decoded as if it were common:
// its plane is not read and its partial sums are NaN, so every token that picked it comes out NaN. ANYROW = true also
// carries the decode loops of the other base codes and of mask mode, which cost ~35 registers that the common kernel does
// not have to pay for. Four wavefronts per SIMD is the measured optimum for the gate|up launch (three: +4 us per layer; five,
// which the common kernel reaches at 92 registers: +1.5 us), so the register allocator is told to aim at exactly that. The
// common down launch gains from five (96 registers, three of them spilled): its 1536 workgroups then need 1.2 rounds instead of
// 1.5 (-0.4 us per layer at one token, -2.5 us at four); six spills sixteen registers and loses 0.9 us.
template <int MODE, bool ANYROW>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MODE == 1 && !ANYROW ? 5 : 4, MODE == 1 && !ANYROW ? 5 : 4)))
nq_gemv_k(MoeArgs a, int NC)
{
    extern __shared__ __align__(16) char smem[];
    __builtin_amdgcn_s_setprio(3);                               // the head is a chain of latencies (see progress_priority)
    __shared__ float zl[MAXTOK][4];                              // gate|up finisher: x V_gu^T of the run's tokens (low-rank plane)
    __shared__ int last;
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6, SB = blockDim.x >> 6;
    if (a.mb_apply && blockIdx.z == gridDim.z - 1)
    {   // the extra plane of blocks of the last projection launch of a call with a mailbox: one of them applies it
        if (blockIdx.x == 0 && blockIdx.y == 0) mailbox_apply(a.mb_table, a.mb_stage, a.mb_seq, a.mb_applied, a.E);
        return;
    }
    // the run's header, written by nq_prep_k: block-uniform, read through the scalar cache (constant address space)
    typedef const __attribute__((address_space(4))) RouteWs* cws_t;
    const cws_t W = (cws_t)a.route;
    struct RawHdr { uint32_t w[sizeof(RunHdr) / 4]; } raw;       // requested together with nruns: one round trip, not two
    {
        const __attribute__((address_space(4))) uint32_t* src = (const __attribute__((address_space(4))) uint32_t*)&a.route->run[MODE][blockIdx.z];
#pragma unroll
        for (int i = 0; i < (int)(sizeof(RunHdr) / 4); ++i) raw.w[i] = src[i];
    }
    const int nruns = W->nruns;
    const int ny_gu = W->ny_gu;                                  // MODE 1: how many k-slices the gate|up launch that filled part_gu wrote
    const int N = MODE == 0 ? 2 * a.I : a.H, K = MODE == 0 ? a.H : a.I, C = K / 128;
    if (MODE == 1 && nruns == 0 && blockIdx.z == 0 && blockIdx.y == 0)
    {   // no active pick at all: nobody will arrive last, so the first plane of blocks writes the zero output
        for (int i = threadIdx.x; i < a.B * SB * 16; i += blockDim.x)
            out2_store(a, (size_t)(i / (SB * 16)) * a.H + blockIdx.x * SB * 32 + 2 * (i % (SB * 16)), 0.f, 0.f);
    }
    if ((int)blockIdx.z >= nruns) return;                        // block-uniform
    const RunHdr R = __builtin_bit_cast(RunHdr, raw);
    const int NY = C / NC;
    if (MODE == 0 && threadIdx.x == 0 && blockIdx.x + blockIdx.y + blockIdx.z == 0) a.route->ny_gu = NY;   // for the down launch's fused staging
    const int ntok = R.ntok, chunk0 = blockIdx.y * NC, k0 = chunk0 * 128;
    const int rowstride = NC * 256 + 16;                         // bytes per staged token (+16: spread tokens over banks)
    char* zero = smem + ntok * rowstride;                        // 256 zero bytes after the token rows
    const _Float16* signs = R.signs;

    // ---- lane context; the first base record is requested now so that its latency overlaps the staging below
    const int t4 = lane >> 4, ss = (lane >> 3) & 1, g = lane & 7, n = lane & 15;
    const int strip = 2 * (blockIdx.x * SB + warp) + ss;
    const Planes P = R.P;                                        // block-uniform: the plane addresses stay in scalar registers
    LaneCtx L;
    L.unit0 = (size_t)strip * C + chunk0; L.rec0 = L.unit0 * 32 + 4 * g + t4;
    L.nrec = (size_t)(N / 16) * C * 32;
    L.src = a.G == 2 ? lane ^ 16 : (lane + 16) & 63;             // next record of the ring: rings of four lanes, or of two
    L.g = g; L.strip = (size_t)strip; L.nstrips = (size_t)(N / 16); L.chunk0 = chunk0;
    L.xs = (n < ntok ? smem + n * rowstride : zero) + t4 * 16; L.xstep = n < ntok ? 256 : 0;
    // block-uniform: a row the common kernel has no loop for (its plane is not read: the records have another size or order)
    const bool foreign = !ANYROW && (P.bcode != 0 || (P.flags != nullptr && R.level != 2));
    u32x4 nb0 = {0u, 0u, 0u, 0u};
    if constexpr (ANYROW) { if (P.bcode == 1) nb0 = load_base<1>(P, L.rec0, L.nrec); else nb0 = P.base[L.rec0]; }
    else if (!foreign) nb0 = P.base[L.rec0];

    // ---- stage the run's tokens for this k-slice in B-operand order
    if constexpr (MODE == 0)
    {
        // rotated by nq_prep_k, already in B-operand order: 16 bytes per thread and step
        const bool up = (int)(blockIdx.x * SB * 32) >= a.I;      // gate rows were rotated with su_g, up rows with su_u
        const _Float16* xr = a.xrot + ((size_t)R.q0 * 2 + (up ? 1 : 0)) * a.H + k0;
        for (int i = threadIdx.x; i < ntok * NC * 16; i += blockDim.x)
        {
            const int j = i / (NC * 16), r = i - j * NC * 16;
            *(u32x4*)(smem + j * rowstride + r * 16) = *(const u32x4*)(xr + (size_t)j * 2 * a.H + r * 8);
        }
    }
    else if (a.fuse && R.had != 512 && R.lr == nullptr)
    {
        // The gate|up finisher, done here for this k-slice's columns of the run's tokens: g = WHT(sum of gate partials) * sv_g,
        // u likewise, h = fp16(WHT(silu(g) * u * su_d)), written straight into the B-operand rows (same operations in the same
        // order as finish_gu, so the same bits). Every column block of the run repeats it; in exchange the gate|up launch ends
        // with its last partial sum and h makes no round trip through memory. Runs whose row has a low-rank plane or the
        // 512-wide rotation keep the finisher in the gate|up launch: both launches read the same row, so they agree.
        const _Float16 *sv_g = signs + a.H, *sv_u = sv_g + a.I, *su_d = sv_u + a.I;
        const int Sgu = a.B * a.topk;
        for (int task = warp; task < ntok * NC; task += SB)
        {
            const int j = task / NC, c = task - j * NC, col = k0 + c * 128 + 2 * lane;
            const float* p = a.part_gu + (size_t)R.slot_of(j) * 2 * a.I + col;
            const float* const rows2[2] = {p, p + a.I};
            const half2_t svg = *(const half2_t*)(sv_g + col), svu = *(const half2_t*)(sv_u + col), sud = *(const half2_t*)(su_d + col);
            float2 pq[2];
            sum_partials<2>(rows2, (size_t)Sgu * 2 * a.I, ny_gu, pq);
            float g0 = pq[0].x, g1 = pq[0].y, u0 = pq[1].x, u1 = pq[1].y;
            wht128(g0, g1, lane); wht128(u0, u1, lane);
            g0 *= (float)svg.x; g1 *= (float)svg.y; u0 *= (float)svu.x; u1 *= (float)svu.y;
            const float sw0 = g0 / (1.f + __expf(-g0)) * u0, sw1 = g1 / (1.f + __expf(-g1)) * u1;
            float v0 = sw0 * (float)sud.x, v1 = sw1 * (float)sud.y;
            wht128(v0, v1, lane);
            asm volatile("" : "+v"(v0), "+v"(v1));            // as in finish_gu: the scaled fp32 value is rounded to fp16, in two steps
            _Float16* dst = (_Float16*)(smem + j * rowstride + c * 256);
            dst[bop_index(2 * lane)] = (_Float16)v0; dst[bop_index(2 * lane + 1)] = (_Float16)v1;
            if (blockIdx.x == 0)                                 // h stays inspectable, as the gate|up finisher leaves it
            {
                half2_t hv; hv.x = (_Float16)v0; hv.y = (_Float16)v1;
                *(half2_t*)(a.h + (size_t)R.slot_of(j) * a.I + col) = hv;
            }
        }
    }
    else
    {
        for (int i = threadIdx.x; i < ntok * NC * 64; i += blockDim.x)
        {
            const int j = i / (NC * 64), r = i % (NC * 64), c = r >> 6, p = r & 63;
            const half2_t hv = *(const half2_t*)(a.h + (size_t)R.slot_of(j) * a.I + k0 + c * 128 + 2 * p);
            _Float16* dst = (_Float16*)(smem + j * rowstride + c * 256);
            dst[bop_index(2 * p)] = hv.x; dst[bop_index(2 * p + 1)] = hv.y;
        }
    }
    if (threadIdx.x < 64) ((uint32_t*)zero)[threadIdx.x] = 0u;
    __syncthreads();

    // ---- decode + MFMA over the k-slice
    float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if constexpr (ANYROW)
        dispatch_base(P.bcode, [&](auto bk) {
            constexpr int BK = decltype(bk)::value;
            if (R.level == 2) gemv_chunks<false, 0, BK>(P, L, NC, acc, nb0);
            else dispatch_code(P.code, [&](auto tag) { gemv_chunks<true, decltype(tag)::value, BK>(P, L, NC, acc, nb0); });
        });
    else if (foreign)
    {
        const float nan = __builtin_nanf("");
        acc[0] = float4_t{nan, nan, nan, nan}; acc[1] = acc[0];
    }
    else if (R.level == 2)
    {
        if (a.hoist && P.var == nullptr) gemv_chunks<false, 0, 0, false, true>(P, L, NC, acc, nb0);   // block-uniform: the caller's option
        else gemv_chunks<false, 0, 0, false>(P, L, NC, acc, nb0);
    }
    else if (a.hoist && P.var == nullptr) dispatch_code(P.code, [&](auto tag) { gemv_chunks<true, decltype(tag)::value, 0, false, true>(P, L, NC, acc, nb0); });
    else dispatch_code(P.code, [&](auto tag) { gemv_chunks<true, decltype(tag)::value, 0, false>(P, L, NC, acc, nb0); });

    __builtin_amdgcn_s_setprio(3);                               // the tail is a chain of latencies: nothing should wait behind decoders

    // ---- k-slice partial sums: lane (t4, n) holds rows 16 (strip0 + t4 / 2) + 4 (t4 & 1) + i (+ 8 for acc[1]) of token n
    if (n < ntok)
    {
        const int S = a.B * a.topk;
        float* part = (MODE == 0 ? a.part_gu : a.part_d) + ((size_t)blockIdx.y * S + R.slot_of(n)) * N;
        const int row = 16 * (2 * (blockIdx.x * SB + warp) + (t4 >> 1)) + 4 * (t4 & 1);
        st_dev4(part + row, acc[0]);
        st_dev4(part + row + 8, acc[1]);
    }

    // fused finisher: the down launch's staging forms h from these partial sums itself (no arrival counter, no finisher here)
    if (MODE == 0 && a.fuse && R.had != 512 && R.lr == nullptr) return;   // block-uniform (a property of the run's row)

    // ---- arrival counter of the 128-row group this block belongs to; the last block to arrive finishes the group
    const int rows0 = blockIdx.x * SB * 32;
    const int grp = MODE == 0 ? (rows0 % a.I) / 128 : rows0 / 128;
    int* cnt = MODE == 0 ? a.cnt_gu + blockIdx.z * (a.I / 128) + grp : a.cnt_d + grp;
    const int expect = (MODE == 0 ? 2 : nruns) * NY * (128 / (SB * 32));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");             // this wavefront's partial sums are acknowledged
    __syncthreads();
    if (threadIdx.x == 0)
        last = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == expect - 1;
    __syncthreads();
    if (!last) return;                                           // block-uniform
    if constexpr (MODE == 0) finish_gu(a, R, zl, blockIdx.z, grp, NY, warp, SB, lane, last);
    else finish_dn(a, a.route->picks, grp, NY, warp, SB, lane, (float*)smem);
    if (threadIdx.x == 0) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The stand-alone mailbox (reference nq_mailbox, sm120/nqmoe.cu:914-923): table[e] <- stage[e] where seq[e] != applied[e], then
// applied[e] <- seq[e]; the host mirror gets every entry of applied, changed or not, so that rows applied by the mailbox block
// of an earlier layer call (which publishes nothing itself) are published here too. Safe to publish at once: this launch
// follows every earlier launch on the stream, and every later one reads the table after it.
__global__ void nq_mailbox_k(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const int32_t sq = __hip_atomic_load(seq + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    int32_t ap = applied[e];
    if (sq != ap)
    {
#pragma unroll
        for (int i = 0; i < TBL_W; ++i)
            table[(size_t)e * TBL_W + i] = __hip_atomic_load(stage + (size_t)e * TBL_W + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __threadfence();
        applied[e] = ap = sq;
    }
    if (applied_host) __hip_atomic_store(applied_host + e, ap, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

int launch_moe(const MoeArgs& a, const int* cfg_gu, const int* cfg_dn, int which, hipStream_t st)
{
    const int S = a.B * a.topk;
    const bool reuse = (which & 4) != 0;                          // the routing launch of an earlier call left route_ws / xrot as this call needs them
    const bool defer = (which & 8) != 0;                          // two-call form of the one-call arithmetic: h is formed by the down launch
    which &= 3;
    if (!reuse)
    {
        const int ntask = S * 2 * (a.H / 128);                   // upper bound: every pick active
        nq_prep_k<<<std::min((ntask + 3) / 4, 1023) + 1, 256, 0, st>>>(a);       // one workgroup per four rotation tasks, plus the writer
        NQ_LAUNCH_CHECK("moe_forward (routing)");
    }
    // a call with a mailbox and no projection launch: the apply half as a launch of its own (nothing is published here either)
    if (a.mb_table && which == 0) return launch_mailbox(a.mb_table, a.mb_stage, a.mb_seq, a.mb_applied, nullptr, a.E, st);
    const int last_mode = (which & 2) ? 1 : 0;
    for (int mode = 0; mode < 2; ++mode)
    {
        if (!((which >> mode) & 1)) continue;
        const int* cf = mode == 0 ? cfg_gu : cfg_dn;
        const int NC = cf[0] * cf[2], SB = cf[1];
        const int N = mode == 0 ? 2 * a.I : a.H, K = mode == 0 ? a.H : a.I, C = K / 128;
        const int NX = N / 32 / SB, NY = C / NC;
        const int shm = std::max(a.B * (NC * 256 + 16) + 256, SB * 512);
        const bool any = a.common_rows != 1;
        MoeArgs b = a;
        b.fuse = which == 3 || defer;                             // both launches belong to this call (or the caller says the other one follows)
        b.mb_apply = a.mb_table != nullptr && mode == last_mode;  // the call's last projection launch carries the mailbox block
        auto kern = mode == 0 ? (any ? nq_gemv_k<0, true> : nq_gemv_k<0, false>) : (any ? nq_gemv_k<1, true> : nq_gemv_k<1, false>);
        if (shm > 48 * 1024)
        {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, shm);
            if (e != hipSuccess) return set_error("moe_forward: LDS %d bytes: %s", shm, hipGetErrorString(e));
        }
        kern<<<dim3(NX, NY, S + (b.mb_apply ? 1 : 0)), 64 * SB, shm, st>>>(b, NC);
        NQ_LAUNCH_CHECK("moe_forward");
    }
    return 0;
}

// ---- nq_moe_forward_static: the same two launches with every workspace carved from one built-in device array --------------
// For callers that cannot allocate (stream capture, serving loops, harnesses that forbid hipMalloc). Each GPU holds its own
// copy of the array at its own address; in host code the array's name is only a handle for hipGetSymbolAddress, which is
// asked once per device, with that device current, and the address it returns is what the kernels are given. Calls on one
// GPU share the array: two calls that overlap on one GPU (different streams) race.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)NQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static unsigned char* g_scratch_ptr[MAX_DEVICES] = {};
static std::mutex g_scratch_mu;

__global__ void nq_clear_k(int* p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

int launch_moe_static(MoeArgs a, const int* cfg_gu, const int* cfg_dn, int which, hipStream_t st)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return set_error("nq_moe_forward_static: current device %d: %s", dev, hipGetErrorString(e));
    unsigned char* base;
    {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (!g_scratch_ptr[dev])
        {
            void* ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !ptr) return set_error("nq_moe_forward_static: address of the built-in scratch on device %d: %s", dev, hipGetErrorString(e));
            g_scratch_ptr[dev] = (unsigned char*)ptr;
        }
        base = g_scratch_ptr[dev];
    }
    const size_t S = (size_t)a.B * a.topk, G128 = (size_t)a.I / 128;
    const size_t ny_gu = (size_t)(a.H / 128) / (cfg_gu[0] * cfg_gu[2]), ny_dn = (size_t)(a.I / 128) / (cfg_dn[0] * cfg_dn[2]);
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += (bytes + 255) & ~(size_t)255; return o; };
    const size_t o_cnt = take((2 * S * G128 + (size_t)a.H / 128) * sizeof(int));       // cnt_gu | cnt_h | cnt_d: cleared below
    const size_t o_gu = take(ny_gu * S * 2 * a.I * sizeof(float)), o_d = take(ny_dn * S * a.H * sizeof(float));
    const size_t o_h = take(S * a.I * sizeof(_Float16)), o_zd = take(S * G128 * 4 * sizeof(float)), o_route = take(sizeof(RouteWs)), o_xrot = take(S * 2 * a.H * sizeof(_Float16));
    if (off > STATIC_SCRATCH_BYTES)
        return set_error("nq_moe_forward_static: this call needs %zu bytes of workspace (B=%d topk=%d H=%d I=%d, %zu and %zu k-slices), the built-in "
                         "scratch holds %zu: use coarser k-slices, or nq_moe_forward with workspaces of the caller's", off, a.B, a.topk, a.H, a.I, ny_gu, ny_dn,
                         STATIC_SCRATCH_BYTES);
    a.cnt_gu = (int*)(base + o_cnt); a.cnt_h = a.cnt_gu + S * G128; a.cnt_d = a.cnt_h + S * G128;
    a.part_gu = (float*)(base + o_gu); a.part_d = (float*)(base + o_d); a.h = (_Float16*)(base + o_h); a.zd = (float*)(base + o_zd);
    a.route = (RouteWs*)(base + o_route); a.xrot = (_Float16*)(base + o_xrot);
    // the counters must be zero on entry; a fill kernel, not hipMemsetAsync, so that the call can be recorded into a graph
    const int ncnt = (int)(2 * S * G128 + (size_t)a.H / 128);
    nq_clear_k<<<(ncnt + 255) / 256, 256, 0, st>>>(a.cnt_gu, ncnt);
    NQ_LAUNCH_CHECK("nq_moe_forward_static");
    return launch_moe(a, cfg_gu, cfg_dn, which, st);
}

// resident workgroups per CU, registers and spill bytes of a decode kernel for a launch shape
int query_occ(int mode, int any_rows, int sb, int shm, int* out)
{
    auto kern = mode == 0 ? (any_rows ? nq_gemv_k<0, true> : nq_gemv_k<0, false>) : (any_rows ? nq_gemv_k<1, true> : nq_gemv_k<1, false>);
    hipError_t e;
    if (shm > 48 * 1024 && (e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, shm)) != hipSuccess)
        return set_error("nq_occ: LDS %d bytes: %s", shm, hipGetErrorString(e));
    int nb = 0;
    if ((e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, (const void*)kern, 64 * sb, (size_t)shm)) != hipSuccess)
        return set_error("nq_occ: %s", hipGetErrorString(e));
    hipFuncAttributes fa;
    if ((e = hipFuncGetAttributes(&fa, (const void*)kern)) != hipSuccess) return set_error("nq_occ: %s", hipGetErrorString(e));
    out[0] = nb; out[1] = fa.numRegs; out[2] = (int)fa.localSizeBytes;
    return 0;
}

int launch_mailbox(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E, hipStream_t st)
{
    nq_mailbox_k<<<(E + 127) / 128, 128, 0, st>>>(table, stage, seq, applied, applied_host, E);
    NQ_LAUNCH_CHECK("nq_mailbox");
    return 0;
}

}  // namespace nq
