// Decode-path MoE layer for 1..8 tokens (reference sm120/nqmoe.cu:375-449 route, :493-771 do_item, :858-907 moe_forward,
// :908-929 mailbox). Two launches on one stream, every routing / level / pointer decision read on the device:
//
//   nq_gemv_k<0>  gate|up: grid (strip-pair blocks, k-slices, runs). A run = one distinct routed expert + the tokens that
//                 picked it. The block rotates those tokens' x (x * su -> Hadamard-128 -> fp16) into LDS, then every
//                 wavefront decodes the records of two strips chunk by chunk straight into MFMA A operands
//                 (v_mfma_f32_16x16x32_f16, tokens as the N dimension) and writes its k-slice partial sums. The block
//                 that arrives last at a (run, 128-column group) counter sums the partials and finishes them:
//                 Hadamard * sv, SwiGLU, * su_d, Hadamard -> h fp16.
//   nq_gemv_k<1>  down: same kernel on h; the last block of a 128-row output group (counter over all runs) combines:
//                 out[b] = sum_k rw[b,k] * sv_o (.) Hadamard(sum of partials).
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
// sum over k-slices y of the two floats at p + y * stride (device-coherent reads, four in flight at a time)
__device__ __forceinline__ float2 sum_partials(const float* p, size_t stride, int NY)
{
    float2 acc = make_float2(0.f, 0.f);
    for (int y = 0; y < NY; y += 4)
    {
        float2 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ld_dev2_issue(p + (size_t)(y + i < NY ? y + i : y) * stride);
        ld_wait(v[0], v[1], v[2], v[3]);
#pragma unroll
        for (int i = 0; i < 4; ++i) if (y + i < NY) { acc.x += v[i].x; acc.y += v[i].y; }
    }
    return acc;
}

#ifndef NQ_OCC
#define NQ_OCC
#endif
constexpr int MAXTOK = 16;                     // MFMA N: tokens of one run (B <= 8 -> at most 8 with distinct top-k ids)
struct RunInfo { int e, level, ntok, nruns; int slot[MAXTOK]; const int64_t* ent; };

// ---- routing dedup: picks -> runs, numbered by first occurrence; slots in pick order ---------------------------------
// called by one full wavefront; lane s owns pick s (S <= 64). Fills run z.
__device__ __forceinline__ void route(const MoeArgs& a, int z, RunInfo* R, int lane, int rows)
{
    const int S = a.B * a.topk;
    int e = -1; bool ok = false;
    if (lane < S)
    {
        const long long ee = a.sel[lane];
        if (ee >= 0 && ee < a.E)
        {
            e = (int)ee;
            ok = (float)a.rw[lane] != 0.f && a.table[(size_t)e * TBL_W] > 0;
        }
    }
    unsigned long long rem = __ballot(ok);
    const unsigned long long below = (1ull << lane) - 1ull;
    int r = 0;
    while (rem)
    {
        const int leader = __ffsll((long long)rem) - 1;
        const int ev = __shfl(e, leader);
        const unsigned long long m = __ballot(ok && e == ev);
        if (r == z && ((m >> lane) & 1ull))
        {
            const int pos = __popcll(m & below);
            if (pos < rows) R->slot[pos] = lane;
            if (pos == 0)
            {
                R->e = e; R->ent = a.table + (size_t)e * TBL_W;
                const int lv = (int)R->ent[0];
                R->level = a.force_level ? a.force_level : lv;
                const int n = __popcll(m);
                R->ntok = n < rows ? n : rows;
            }
        }
        rem &= ~m; ++r;
    }
    if (lane == 0) R->nruns = r;
}

// finisher of gate|up for (run, 128-column group grp): h[slot] = fp16(WHT(silu(g) * u * su_d)), g = WHT(sum_y part_g) * sv_g
__device__ __forceinline__ void finish_gu(const MoeArgs& a, const RunInfo& R, int grp, int NY, int warp, int SB, int lane)
{
    const _Float16* signs = (const _Float16*)R.ent[9];
    const _Float16 *sv_g = signs + a.H, *sv_u = sv_g + a.I, *su_d = sv_u + a.I;
    const int S = a.B * a.topk, col = grp * 128 + 2 * lane;
    for (int j = warp; j < R.ntok; j += SB)
    {
        const int s = R.slot[j];
        const float* p = a.part_gu + (size_t)s * 2 * a.I + col;
        const float2 pg = sum_partials(p, (size_t)S * 2 * a.I, NY), pu = sum_partials(p + a.I, (size_t)S * 2 * a.I, NY);
        float g0 = pg.x, g1 = pg.y, u0 = pu.x, u1 = pu.y;
        wht128(g0, g1, lane); wht128(u0, u1, lane);
        const half2_t svg = *(const half2_t*)(sv_g + col), svu = *(const half2_t*)(sv_u + col), sud = *(const half2_t*)(su_d + col);
        g0 *= (float)svg.x; g1 *= (float)svg.y; u0 *= (float)svu.x; u1 *= (float)svu.y;
        float v0 = g0 / (1.f + __expf(-g0)) * u0 * (float)sud.x, v1 = g1 / (1.f + __expf(-g1)) * u1 * (float)sud.y;
        wht128(v0, v1, lane);
        half2_t hv; hv.x = (_Float16)v0; hv.y = (_Float16)v1;
        *(half2_t*)(a.h + (size_t)s * a.I + col) = hv;           // read by the next kernel on the stream
    }
}

// combine of the down projection for output rows [grp * 128, +128): out[b] = sum_k rw[b,k] * sv_o[e] (.) WHT(sum_y part_d[slot])
// picks of a token are spread over the block's wavefronts and reduced through LDS (red: SB * 128 floats)
__device__ __forceinline__ void finish_dn(const MoeArgs& a, int grp, int NY, int warp, int SB, int lane, float* red)
{
    const int S = a.B * a.topk, col = grp * 128 + 2 * lane;
    for (int b = 0; b < a.B; ++b)
    {
        float o0 = 0.f, o1 = 0.f;
        for (int k = warp; k < a.topk; k += SB)
        {
            const int s = b * a.topk + k;
            const long long ee = a.sel[s];
            const float w = (float)a.rw[s];
            if (ee < 0 || ee >= a.E || w == 0.f) continue;
            const int64_t* ent = a.table + (size_t)ee * TBL_W;
            if (ent[0] <= 0) continue;
            const float2 pv = sum_partials(a.part_d + (size_t)s * a.H + col, (size_t)S * a.H, NY);
            float v0 = pv.x, v1 = pv.y;
            wht128(v0, v1, lane);
            const half2_t sv = *(const half2_t*)((const _Float16*)ent[9] + a.H + 3 * a.I + col);
            o0 += w * (v0 * (float)sv.x); o1 += w * (v1 * (float)sv.y);
        }
        red[warp * 128 + 2 * lane] = o0; red[warp * 128 + 2 * lane + 1] = o1;
        __syncthreads();
        if (warp == 0)
        {
            float r0 = 0.f, r1 = 0.f;
            for (int w2 = 0; w2 < SB; ++w2) { r0 += red[w2 * 128 + 2 * lane]; r1 += red[w2 * 128 + 2 * lane + 1]; }
            *(float2*)(a.out + (size_t)b * a.H + col) = make_float2(r0, r1);
        }
        __syncthreads();
    }
}

// MODE 0: gate|up (N = 2I, K = H, input x rotated here). MODE 1: down (N = H, K = I, input h).
// grid (N / 32 / SB, C / NC, S); block 64 * SB threads (SB = 1, 2 or 4: a block covers at most one 128-row group);
// dynamic LDS = rows * (NC * 256 + 16) + 256 bytes (>= SB * 512 for the combine), rows = min(B * topk, MAXTOK) staged tokens
template <int MODE>
__global__ void __launch_bounds__(256) NQ_OCC nq_gemv_k(MoeArgs a, int NC, int rows)
{
    extern __shared__ __align__(16) char smem[];
    __shared__ RunInfo R;
    __shared__ int last;
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6, SB = blockDim.x >> 6;
    if (warp == 0) route(a, blockIdx.z, &R, lane, rows);
    if (MODE == 0 && a.hits && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x < a.B * a.topk)
    {
        const long long ee = a.sel[threadIdx.x];
        if ((float)a.rw[threadIdx.x] != 0.f && ee >= 0 && ee < a.E)
            __hip_atomic_fetch_add(a.hits + ee, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    __syncthreads();
    const int nruns = R.nruns;
    const int N = MODE == 0 ? 2 * a.I : a.H, K = MODE == 0 ? a.H : a.I, C = K / 128, NY = C / NC;
    if (MODE == 1 && nruns == 0 && blockIdx.z == 0 && blockIdx.y == 0)
    {   // no active pick at all: nobody will arrive last, so the first plane of blocks writes the zero output
        for (int i = threadIdx.x; i < a.B * SB * 32; i += blockDim.x)
            a.out[(size_t)(i / (SB * 32)) * a.H + blockIdx.x * SB * 32 + i % (SB * 32)] = 0.f;
    }
    if ((int)blockIdx.z >= nruns) return;                        // block-uniform
    const int ntok = R.ntok, chunk0 = blockIdx.y * NC, k0 = chunk0 * 128;
    const int rowstride = NC * 256 + 16;                         // bytes per staged token (+16: spread tokens over banks)
    char* zero = smem + ntok * rowstride;                        // 256 zero bytes after the token rows
    const _Float16* signs = (const _Float16*)R.ent[9];

    // ---- lane context; the first base record is requested now so that its latency overlaps the staging below
    const int t4 = lane >> 4, ss = (lane >> 3) & 1, g = lane & 7, n = lane & 15;
    const int strip = 2 * (blockIdx.x * SB + warp) + ss;
    const Planes P = planes_of(R.ent, MODE);
    LaneCtx L;
    L.unit0 = (size_t)strip * C + chunk0; L.rec0 = L.unit0 * 32 + 4 * g + t4;
    L.nrec = (size_t)(N / 16) * C * 32;
    L.src = (lane + 16) & 63; L.g = g;
    L.xs = (n < ntok ? smem + n * rowstride : zero) + t4 * 16; L.xstep = n < ntok ? 256 : 0;
    const u32x4 nb0 = P.base[L.rec0];

    // ---- stage the run's tokens for this k-slice in B-operand order
    if constexpr (MODE == 0)
    {
        const bool up = (int)(blockIdx.x * SB * 32) >= a.I;      // gate rows use su_g, up rows su_u
        const _Float16* su = up ? signs + 2 * a.H + 3 * a.I : signs;
        for (int task = warp; task < ntok * NC; task += SB)
        {
            const int j = task / NC, c = task % NC, kk = k0 + c * 128 + 2 * lane;
            const int tok = R.slot[j] / a.topk;
            const half2_t xv = *(const half2_t*)(a.x + (size_t)tok * a.H + kk), sv = *(const half2_t*)(su + kk);
            float v0 = (float)xv.x * (float)sv.x, v1 = (float)xv.y * (float)sv.y;
            wht128(v0, v1, lane);
            _Float16* dst = (_Float16*)(smem + j * rowstride + c * 256);
            dst[bop_index(2 * lane)] = (_Float16)v0; dst[bop_index(2 * lane + 1)] = (_Float16)v1;
        }
    }
    else
    {
        for (int i = threadIdx.x; i < ntok * NC * 64; i += blockDim.x)
        {
            const int j = i / (NC * 64), r = i % (NC * 64), c = r >> 6, p = r & 63;
            const half2_t hv = *(const half2_t*)(a.h + (size_t)R.slot[j] * a.I + k0 + c * 128 + 2 * p);
            _Float16* dst = (_Float16*)(smem + j * rowstride + c * 256);
            dst[bop_index(2 * p)] = hv.x; dst[bop_index(2 * p + 1)] = hv.y;
        }
    }
    if (threadIdx.x < 64) ((uint32_t*)zero)[threadIdx.x] = 0u;
    __syncthreads();

    // ---- decode + MFMA over the k-slice
    float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (R.level == 2) gemv_chunks<false, 0>(P, L, NC, acc, nb0);
    else dispatch_code(P.code, [&](auto tag) { gemv_chunks<true, decltype(tag)::value>(P, L, NC, acc, nb0); });

    // ---- k-slice partial sums: lane (t4, n) holds rows 16 (strip0 + t4 / 2) + 4 (t4 & 1) + i (+ 8 for acc[1]) of token n
    if (n < ntok)
    {
        const int S = a.B * a.topk;
        float* part = (MODE == 0 ? a.part_gu : a.part_d) + ((size_t)blockIdx.y * S + R.slot[n]) * N;
        const int row = 16 * (2 * (blockIdx.x * SB + warp) + (t4 >> 1)) + 4 * (t4 & 1);
        st_dev4(part + row, acc[0]);
        st_dev4(part + row + 8, acc[1]);
    }

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
    if constexpr (MODE == 0) finish_gu(a, R, grp, NY, warp, SB, lane);
    else finish_dn(a, grp, NY, warp, SB, lane, (float*)smem);
    if (threadIdx.x == 0) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// table[e] <- stage[e] where seq[e] != applied[e]; publish applied (device copy and optional host-mapped mirror)
__global__ void nq_mailbox_k(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const int32_t sq = __hip_atomic_load(seq + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (sq == applied[e]) return;
#pragma unroll
    for (int i = 0; i < TBL_W; ++i)
        table[(size_t)e * TBL_W + i] = __hip_atomic_load(stage + (size_t)e * TBL_W + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __threadfence();
    applied[e] = sq;
    if (applied_host) __hip_atomic_store(applied_host + e, sq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

int launch_moe(const MoeArgs& a, const int* cfg_gu, const int* cfg_dn, int which, hipStream_t st)
{
    const int S = a.B * a.topk;
    for (int mode = 0; mode < 2; ++mode)
    {
        if (!((which >> mode) & 1)) continue;
        const int* cf = mode == 0 ? cfg_gu : cfg_dn;
        const int NC = cf[0] * cf[2], SB = cf[1];
        const int N = mode == 0 ? 2 * a.I : a.H, K = mode == 0 ? a.H : a.I, C = K / 128;
        const int NX = N / 32 / SB, NY = C / NC;
        const int rows = S < MAXTOK ? S : MAXTOK;
        const int shm = std::max(rows * (NC * 256 + 16) + 256, SB * 512);
        auto kern = mode == 0 ? nq_gemv_k<0> : nq_gemv_k<1>;
        if (shm > 48 * 1024)
        {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, shm);
            if (e != hipSuccess) return set_error("moe_forward: LDS %d bytes: %s", shm, hipGetErrorString(e));
        }
        kern<<<dim3(NX, NY, S), 64 * SB, shm, st>>>(a, NC, rows);
        NQ_LAUNCH_CHECK("moe_forward");
    }
    return 0;
}

int launch_mailbox(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E, hipStream_t st)
{
    nq_mailbox_k<<<(E + 127) / 128, 128, 0, st>>>(table, stage, seq, applied, applied_host, E);
    NQ_LAUNCH_CHECK("nq_mailbox");
    return 0;
}

}  // namespace nq
