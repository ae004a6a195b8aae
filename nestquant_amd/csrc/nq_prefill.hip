// Prefill path (T > 8 tokens): every routed expert's weights are decoded once per 16..256-row tile of its tokens, inside
// the grouped GEMM itself, never written to HBM (reference: pf_decode to fp16 in HBM + Triton/cuBLAS grouped GEMM,
// sm120/nqmoe.cu:942-1240, sm120/pf_gemm.py:7-34, sm120/moe.py:282-326).
//
//   nq_pf_pre_k   per (token, expert) pair, sorted by expert: xg / xu = fp16(Hadamard-128(x * su_g / su_u)), written in
//                 B-operand column order so the GEMM stages them with straight 16-byte copies      (reference nq_pf_pre)
//   nq_pf_gemm_k  C[rows of expert j][N] = A[rows][K] @ W_j[N][K]^T: grid (N / 128, tiles); a tile = (expert, row0, rows
//                 <= 16 TG). Per 128-column chunk the block stages the tile's activations in LDS while each wavefront
//                 decodes two strips of the expert's records into MFMA A operands, then runs TG x 8 MFMAs
//                 (v_mfma_f32_16x16x32_f16, fp32 accumulate) over the staged tokens. Level from the live table row.
//   nq_pf_mid_k   Hadamard * sv, SwiGLU, * su_d, Hadamard -> h fp16 (B-operand order)               (reference nq_pf_mid)
//   nq_pf_post_k  out[token] += sum over its picks of rw * sv_o (.) Hadamard(y): gathered per token, no atomics  (reference nq_pf_post)
//   nq_pf_hits_k  hits[e] += counts[e]                                                            (reference nq_pf_hits)
#include "nq_tile.hpp"
#include "nq_host.hpp"

namespace nq {

constexpr int PF_ROW = 256;                    // LDS bytes per staged token and chunk; 16-byte column q of row r sits in slot q ^ (r & 15)

// lane holds columns 2 lane, 2 lane + 1 of a 128-column chunk; columns c and c + 16 are neighbours in the B-operand order,
// so lanes l and l ^ 8 swap one value each and every lane stores one aligned 4-byte pair
__device__ __forceinline__ void store_bop(_Float16* dst, float v0, float v1, int lane)
{
    const bool hi = (lane >> 3) & 1;
    const float mine = hi ? v1 : v0, give = hi ? v0 : v1;
    const float got = dpp_lane<0x128>(give);                      // lane ^ 8 (row rotate): low lanes get the partner's v0, high lanes the partner's v1
    half2_t w;
    w.x = (_Float16)(hi ? got : mine); w.y = (_Float16)(hi ? mine : got);
    const int c = hi ? 2 * (lane ^ 8) + 1 : 2 * lane;           // the pair's low column: (c, c + 16)
    *(half2_t*)(dst + bop_index(c)) = w;
}

// order the LDS accesses of one wavefront's lanes among themselves (a wavefront-private buffer needs no workgroup barrier)
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Is pair row p (of expert e) held by a tile of one of the heights in the bit mask `heights` (bit k = 16 << k)? tiles / cap:
// the lists of nq_pf_plan_k. The remainder tile of expert e sits at index e of the list of its height and starts at its
// first row; the rows before it belong to the expert's full 256-row tiles. Rows of no valid expert count as height 256.
__device__ __forceinline__ bool row_in_heights(const int32_t* __restrict__ tiles, int cap, int heights, int p, int e, int E)
{
    int k = 4;
    if (e >= 0 && e < E)
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int4 t = ((const int4*)tiles)[(size_t)q * cap + e];
            if (t.x == e && p >= t.y) k = q;
        }
    return (heights >> k) & 1;
}

// grid (npairs), block 256: wave w handles the 512-column segments w, w + 4, ... of the pair's row, gate and up together.
// tiles (optional): work only on the rows of the tile heights in `heights`
__global__ void __launch_bounds__(256) nq_pf_pre_k(const _Float16* __restrict__ x, const int32_t* __restrict__ pt, const int32_t* __restrict__ pe,
                                                    const int64_t* __restrict__ table, _Float16* xg, _Float16* xu, float* zg, int E, int H, int I,
                                                    const int32_t* __restrict__ tiles, int cap, int heights)
{
    __shared__ float zsh[4][4];
    const int p = blockIdx.x, lane = threadIdx.x & 63, warp = threadIdx.x >> 6;
    const int e = pe[p];
    if (tiles && !row_in_heights(tiles, cap, heights, p, e, E)) return;       // block-uniform
    const int ng = H / 128;
    const bool live = e >= 0 && e < E && table[(size_t)e * TBL_W] > 0;
    const _Float16* signs = live ? (const _Float16*)table[(size_t)e * TBL_W + 9] : nullptr;
    const _Float16* xr = x + (size_t)pt[p] * H;
    // low-rank plane (table words 14, 16): zg[p] = x V_gu^T over the raw activations, for the mid kernel
    const _Float16* lr = live ? (const _Float16*)table[(size_t)e * TBL_W + 14] : nullptr;
    const int rg = lr ? (int)table[(size_t)e * TBL_W + 16] : 0;
    if (zg && rg)                                                // block-uniform
    {
        float zz[4] = {0.f, 0.f, 0.f, 0.f};
        for (int k = 2 * threadIdx.x; k < H; k += 512)
        {
            const half2_t xv = *(const half2_t*)(xr + k);
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < rg) { const half2_t vv = *(const half2_t*)(lr + (size_t)r * H + k); zz[r] += (float)xv.x * (float)vv.x + (float)xv.y * (float)vv.y; }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) zz[r] += __shfl_xor(zz[r], m);
            if (lane == 0) zsh[warp][r] = zz[r];
        }
        __syncthreads();
        if (threadIdx.x < 4) zg[(size_t)p * 4 + threadIdx.x] = zsh[0][threadIdx.x] + zsh[1][threadIdx.x] + zsh[2][threadIdx.x] + zsh[3][threadIdx.x];
    }
    // A wavefront takes 512-column segments: x and the two scale vectors arrive as one 16-byte load per lane each and pass
    // through a wavefront-private LDS buffer to the WHT's layout (lane = columns 2 lane, 2 lane + 1 of a 128-column chunk);
    // the eight rotated chunks (4 chunks x gate / up) go back through the same buffer in B-operand order and leave as
    // 16-byte stores. Full segments only when H is a multiple of 512; the remaining chunks take the narrow path below.
    __shared__ __align__(16) _Float16 seg[4][3 * 512];
    _Float16* sb = seg[warp];
    const int nseg = H / 512;
    for (int sgi = warp; sgi < nseg; sgi += 4)
    {
        const int k0 = sgi * 512;
        float v[2][4][2];
        if (live)
        {
            const _Float16* sug = signs, *suu = signs + 2 * H + 3 * I;
            const uint4 xi = *(const uint4*)(xr + k0 + 8 * lane), gi = *(const uint4*)(sug + k0 + 8 * lane), ui = *(const uint4*)(suu + k0 + 8 * lane);
            *(uint4*)(sb + 8 * lane) = xi; *(uint4*)(sb + 512 + 8 * lane) = gi; *(uint4*)(sb + 1024 + 8 * lane) = ui;
            wave_sync();
#pragma unroll
            for (int c = 0; c < 4; ++c)
            {
                const half2_t xv = *(const half2_t*)(sb + 128 * c + 2 * lane), sg = *(const half2_t*)(sb + 512 + 128 * c + 2 * lane),
                              su = *(const half2_t*)(sb + 1024 + 128 * c + 2 * lane);
                v[0][c][0] = (float)xv.x * (float)sg.x; v[0][c][1] = (float)xv.y * (float)sg.y;
                v[1][c][0] = (float)xv.x * (float)su.x; v[1][c][1] = (float)xv.y * (float)su.y;
            }
#pragma unroll
            for (int up = 0; up < 2; ++up)
#pragma unroll
                for (int c = 0; c < 4; ++c) wht128(v[up][c][0], v[up][c][1], lane);
        }
        else
        {
#pragma unroll
            for (int up = 0; up < 2; ++up)
#pragma unroll
                for (int c = 0; c < 4; ++c) v[up][c][0] = v[up][c][1] = 0.f;
        }
        wave_sync();       // every lane has read its inputs before the buffer is reused
#pragma unroll
        for (int up = 0; up < 2; ++up)
#pragma unroll
            for (int c = 0; c < 4; ++c) store_bop(sb + up * 512 + c * 128, v[up][c][0], v[up][c][1], lane);
        wave_sync();
        *(uint4*)(xg + (size_t)p * H + k0 + 8 * lane) = *(const uint4*)(sb + 8 * lane);
        *(uint4*)(xu + (size_t)p * H + k0 + 8 * lane) = *(const uint4*)(sb + 512 + 8 * lane);
        wave_sync();       // the stores' LDS reads are done before the next segment's writes
    }
    for (int task = 8 * nseg + warp; task < 2 * ng; task += 4)       // chunks beyond the last full segment (task = 2 * chunk + up)
    {
        const int up = task & 1, grp = task >> 1, k = grp * 128 + 2 * lane;
        _Float16* dst = (up ? xu : xg) + (size_t)p * H + grp * 128;
        float v0 = 0.f, v1 = 0.f;
        if (live)
        {
            const _Float16* su = up ? signs + 2 * H + 3 * I : signs;
            const half2_t xv = *(const half2_t*)(xr + k), sv = *(const half2_t*)(su + k);
            v0 = (float)xv.x * (float)sv.x; v1 = (float)xv.y * (float)sv.y;
            wht128(v0, v1, lane);
        }
        store_bop(dst, v0, v1, lane);
    }
}

// grid (npairs), block 256: acc_gu [P][2I] fp32 (gate | up) -> h [P][I] fp16 in B-operand order. With in_had_down = 512
// (table word 18) the four wavefronts hold the four 128-column groups of a 512-column block and combine their WHT_128
// results through LDS with the Sylvester H_4 / 2 before the single rounding to fp16.
// tiles (optional): work only on the rows of the tile heights in `heights`, as nq_pf_pre_k
__global__ void __launch_bounds__(256) nq_pf_mid_k(const float* __restrict__ acc_gu, const int32_t* __restrict__ pe,
                                                    const int64_t* __restrict__ table, _Float16* h, const float* zg, float* zd, int E, int H, int I,
                                                    const int32_t* __restrict__ tiles, int cap, int heights)
{
    __shared__ float wsh[4][128];
    __shared__ float zsh[4][4];
    const int p = blockIdx.x, lane = threadIdx.x & 63, warp = threadIdx.x >> 6;
    const int e = pe[p];
    if (tiles && !row_in_heights(tiles, cap, heights, p, e, E)) return;       // block-uniform
    const bool live = e >= 0 && e < E && table[(size_t)e * TBL_W] > 0;
    const _Float16* signs = live ? (const _Float16*)table[(size_t)e * TBL_W + 9] : nullptr;
    const bool wide = live && table[(size_t)e * TBL_W + 18] == 512;      // block-uniform
    // low-rank plane: g / u += zg (U2 [+ U4 at level 4]); zd[p] = sw V_dn^T for the post kernel
    const _Float16* lr = live ? (const _Float16*)table[(size_t)e * TBL_W + 14] : nullptr;
    const _Float16* lr4 = live ? (const _Float16*)table[(size_t)e * TBL_W + 15] : nullptr;
    const int rg = lr && zg ? (int)table[(size_t)e * TBL_W + 16] : 0, rd = lr && zd ? (int)table[(size_t)e * TBL_W + 17] : 0;
    const bool l4 = live && table[(size_t)e * TBL_W] == 4;
    const _Float16* U2g = lr + (size_t)rg * H, *U2u = U2g + (size_t)rg * I, *Vd = U2u + (size_t)rg * I, *U4g = lr4, *U4u = lr4 + (size_t)rg * I;
    float zr[4] = {0.f, 0.f, 0.f, 0.f}, zacc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r = 0; r < rg; ++r) zr[r] = zg[(size_t)p * 4 + r];
    for (int grp = warp; grp < I / 128; grp += 4)
    {
        const int col = grp * 128 + 2 * lane;
        _Float16* dst = h + (size_t)p * I + grp * 128;
        float v0 = 0.f, v1 = 0.f;
        if (live)
        {
            const _Float16 *sv_g = signs + H, *sv_u = sv_g + I, *su_d = sv_u + I;
            const float2 pg = *(const float2*)(acc_gu + (size_t)p * 2 * I + col), pu = *(const float2*)(acc_gu + (size_t)p * 2 * I + I + col);
            float g0 = pg.x, g1 = pg.y, u0 = pu.x, u1 = pu.y;
            wht128(g0, g1, lane); wht128(u0, u1, lane);
            const half2_t svg = *(const half2_t*)(sv_g + col), svu = *(const half2_t*)(sv_u + col), sud = *(const half2_t*)(su_d + col);
            g0 *= (float)svg.x; g1 *= (float)svg.y; u0 *= (float)svu.x; u1 *= (float)svu.y;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < rg)
                {
                    half2_t ug = *(const half2_t*)(U2g + (size_t)r * I + col), uu = *(const half2_t*)(U2u + (size_t)r * I + col);
                    g0 += zr[r] * (float)ug.x; g1 += zr[r] * (float)ug.y; u0 += zr[r] * (float)uu.x; u1 += zr[r] * (float)uu.y;
                    if (l4)
                    {
                        ug = *(const half2_t*)(U4g + (size_t)r * I + col); uu = *(const half2_t*)(U4u + (size_t)r * I + col);
                        g0 += zr[r] * (float)ug.x; g1 += zr[r] * (float)ug.y; u0 += zr[r] * (float)uu.x; u1 += zr[r] * (float)uu.y;
                    }
                }
            const float sw0 = g0 / (1.f + __expf(-g0)) * u0, sw1 = g1 / (1.f + __expf(-g1)) * u1;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < rd) { const half2_t vv = *(const half2_t*)(Vd + (size_t)r * I + col); zacc[r] += sw0 * (float)vv.x + sw1 * (float)vv.y; }
            v0 = sw0 * (float)sud.x; v1 = sw1 * (float)sud.y;
            wht128(v0, v1, lane);
        }
        if (wide)
        {   // I % 512 == 0, so all four wavefronts are in this iteration: grp = 4 * block + warp
            wsh[warp][2 * lane] = v0; wsh[warp][2 * lane + 1] = v1;
            __syncthreads();
            v0 = v1 = 0.f;
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
            {
                const float sg = (__builtin_popcount(warp & pp) & 1) ? -0.5f : 0.5f;
                v0 += sg * wsh[pp][2 * lane]; v1 += sg * wsh[pp][2 * lane + 1];
            }
            __syncthreads();
        }
        store_bop(dst, v0, v1, lane);
    }
    if (rd)                                                      // block-uniform
    {
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) zacc[r] += __shfl_xor(zacc[r], m);
            if (lane == 0) zsh[warp][r] = zacc[r];
        }
        __syncthreads();
        if (threadIdx.x < 4) zd[(size_t)p * 4 + threadIdx.x] = zsh[0][threadIdx.x] + zsh[1][threadIdx.x] + zsh[2][threadIdx.x] + zsh[3][threadIdx.x];
    }
}

// grid (T), block 256: out[t] += sum over the token's picks whose pair row lies in [row_lo, row_lo + nrows) of
// rw * sv_o (.) Hadamard(y[row]); pos[t][k] = row of pair (t, k) in the expert-sorted order. One block owns a token, so
// the sum needs no atomics and its order is fixed (the reference's pf_post adds with float atomics in arrival order).
__global__ void __launch_bounds__(256) nq_pf_post_k(const float* __restrict__ y, const int32_t* __restrict__ pos, const int64_t* __restrict__ sel,
                                                     const _Float16* __restrict__ rw, int topk, int row_lo, int nrows,
                                                     const int64_t* __restrict__ table, float* out, const float* zd, int E, int H, int I)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63, warp = threadIdx.x >> 6;
    // the token's live picks, gathered once: row, weight and sign vector (picks keep their order, so does the sum)
    __shared__ int p_row[64]; __shared__ float p_w[64]; __shared__ const _Float16* p_sv[64]; __shared__ int p_n;
    __shared__ const _Float16* p_u2[64]; __shared__ const _Float16* p_u4[64]; __shared__ int p_rd[64];   // low-rank plane: U2_d, U4_d (level 4) and r_dn
    if (warp == 0)
    {
        bool ok = false; int r = 0, rdn = 0; float w = 0.f; const _Float16* sv = nullptr; const _Float16* u2 = nullptr; const _Float16* u4 = nullptr;
        if (lane < topk)
        {
            r = pos[(size_t)t * topk + lane] - row_lo;
            const long long e = sel[(size_t)t * topk + lane];
            w = (float)rw[(size_t)t * topk + lane];
            if (r >= 0 && r < nrows && e >= 0 && e < E && w != 0.f && table[(size_t)e * TBL_W] > 0)
            {
                ok = true; sv = (const _Float16*)table[(size_t)e * TBL_W + 9] + H + 3 * I;
                const _Float16* lr = (const _Float16*)table[(size_t)e * TBL_W + 14];
                if (lr && zd)
                {
                    const int rg = (int)table[(size_t)e * TBL_W + 16];
                    rdn = (int)table[(size_t)e * TBL_W + 17];
                    u2 = lr + (size_t)rg * (H + 2 * I) + (size_t)rdn * I;
                    if (table[(size_t)e * TBL_W] == 4) u4 = (const _Float16*)table[(size_t)e * TBL_W + 15] + (size_t)rg * 2 * I;
                }
            }
        }
        const unsigned long long m = __ballot(ok);
        if (ok) { const int i = __popcll(m & ((1ull << lane) - 1ull)); p_row[i] = r; p_w[i] = w; p_sv[i] = sv; p_u2[i] = u2; p_u4[i] = u4; p_rd[i] = rdn; }
        if (lane == 0) p_n = __popcll(m);
    }
    __syncthreads();
    const int np = p_n;
    if (np == 0) return;
    for (int grp = warp; grp < H / 128; grp += 4)
    {
        const int col = grp * 128 + 2 * lane;
        float o0 = 0.f, o1 = 0.f;
        for (int k0 = 0; k0 < np; k0 += 4)                       // four picks at a time, reads first
        {
            float2 v[4]; half2_t sv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const int k = k0 + u < np ? k0 + u : k0;
                v[u] = *(const float2*)(y + (size_t)p_row[k] * H + col);
                sv[u] = *(const half2_t*)(p_sv[k] + col);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                if (k0 + u >= np) break;
                float v0 = v[u].x, v1 = v[u].y;
                wht128(v0, v1, lane);
                const float w = p_w[k0 + u];
                v0 *= (float)sv[u].x; v1 *= (float)sv[u].y;
                for (int r = 0; r < p_rd[k0 + u]; ++r)           // y += (sw V_dn^T) (U2_d [+ U4_d])
                {
                    const float zr = zd[(size_t)p_row[k0 + u] * 4 + r];
                    half2_t ud = *(const half2_t*)(p_u2[k0 + u] + (size_t)r * H + col);
                    v0 += zr * (float)ud.x; v1 += zr * (float)ud.y;
                    if (p_u4[k0 + u]) { ud = *(const half2_t*)(p_u4[k0 + u] + (size_t)r * H + col); v0 += zr * (float)ud.x; v1 += zr * (float)ud.y; }
                }
                o0 += w * v0; o1 += w * v1;
            }
        }
        float2* op = (float2*)(out + (size_t)t * H + col);
        float2 cur = *op; cur.x += o0; cur.y += o1; *op = cur;
    }
}

__global__ void nq_pf_hits_k(const int32_t* counts, int32_t* hits, int E)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < E && counts[e]) __hip_atomic_fetch_add(hits + e, counts[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// ---- tile lists on the device ------------------------------------------------------------------------------------------
// One workgroup. counts[e] = pairs of expert e over the whole call (pairs sorted by expert, so expert e owns the pair rows
// [sum of counts before e, + counts[e])); the chunk is the pair rows [row_lo, row_lo + nrows). Every expert's rows inside
// the chunk are cut into 256-row tiles; the remainder goes to the list of the smallest compiled height (16 << k) that holds
// it, at index e of list k; the full tiles follow at indices E.. of list 4. tiles: int32 [5][cap][4] = (expert, first row in
// the chunk, rows, 0); entries without a tile get expert -1, which the GEMM skips. Replaces the host loop over the expert
// counts and with it the call's one host synchronisation.
__device__ __forceinline__ void block_scan(int* a, int* b, int E)
{   // inclusive prefix sum of a[0..E) in place (b: scratch of the same size); all threads of the block call it
    int *src = a, *dst = b;
    for (int off = 1; off < E; off <<= 1)
    {
        for (int e = threadIdx.x; e < E; e += blockDim.x) dst[e] = src[e] + (e >= off ? src[e - off] : 0);
        __syncthreads();
        int* t = src; src = dst; dst = t;
    }
    if (src != a)
    {
        for (int e = threadIdx.x; e < E; e += blockDim.x) a[e] = src[e];
        __syncthreads();
    }
}

// hot (may be null): experts with at least hot_min rows in the chunk get a slot 0 .. hot_cap - 1 of the decoded-weight scratch (in
// expert order, as far as the slots reach), written to hot[e] (-1: none) and, plus one, into the fourth word of their tiles.
__global__ void __launch_bounds__(256) nq_pf_plan_k(const int32_t* __restrict__ counts, int E, int row_lo, int nrows, int32_t* tiles, int cap,
                                                    int32_t* hot, int hot_min, int hot_cap)
{
    extern __shared__ int plan_sh[];
    int *incl = plan_sh, *tmp = plan_sh + E, *full = plan_sh + 2 * E, *hrank = plan_sh + 3 * E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) incl[e] = counts[e] > 0 ? counts[e] : 0;
    __syncthreads();
    block_scan(incl, tmp, E);
    const int row_hi = row_lo + nrows;
    for (int e = threadIdx.x; e < E; e += blockDim.x)
    {
        const int c = counts[e] > 0 ? counts[e] : 0, start = incl[e] - c;
        const int u = start > row_lo ? start : row_lo, v = start + c < row_hi ? start + c : row_hi;
        const int n = v > u ? v - u : 0;
        full[e] = n / 256;
        hrank[e] = hot != nullptr && n >= hot_min ? 1 : 0;
    }
    __syncthreads();
    block_scan(hrank, tmp, E);                                   // inclusive: hot experts up to and including e
    int* fincl = tmp;                                            // inclusive scan of the full-tile counts
    for (int e = threadIdx.x; e < E; e += blockDim.x) fincl[e] = full[e];
    __syncthreads();
    block_scan(fincl, full, E);                                  // clobbers full[]: recomputed below
    int4* T4 = (int4*)tiles;
    for (int e = threadIdx.x; e < E; e += blockDim.x)
    {
        const int c = counts[e] > 0 ? counts[e] : 0, start = incl[e] - c;
        const int u = start > row_lo ? start : row_lo, v = start + c < row_hi ? start + c : row_hi;
        const int n = v > u ? v - u : 0, r0 = u - row_lo, nf = n / 256, rem = n % 256;
        const int k = rem == 0 ? -1 : rem <= 16 ? 0 : rem <= 32 ? 1 : rem <= 64 ? 2 : rem <= 128 ? 3 : 4;
        const bool is_hot = hot != nullptr && n >= hot_min && hrank[e] <= hot_cap;
        const int slot1 = is_hot ? hrank[e] : 0;                 // scratch slot + 1
        if (hot != nullptr) hot[e] = slot1 - 1;
#pragma unroll
        for (int q = 0; q < 5; ++q) T4[(size_t)q * cap + e] = q == k ? make_int4(e, r0 + 256 * nf, rem, slot1) : make_int4(-1, 0, 0, 0);
        const int base = E + fincl[e] - nf;
        for (int j = 0; j < nf; ++j) T4[(size_t)4 * cap + base + j] = make_int4(e, r0 + 256 * j, 256, slot1);
    }
    const int total = E + fincl[E - 1];
    for (int i = total + threadIdx.x; i < cap; i += blockDim.x) T4[(size_t)4 * cap + i] = make_int4(-1, 0, 0, 0);
}

int launch_pf_plan(const int32_t* counts, int E, int row_lo, int nrows, int32_t* tiles, int cap, int32_t* hot, int hot_min, int hot_cap, hipStream_t st)
{
    nq_pf_plan_k<<<1, 256, 4 * E * sizeof(int), st>>>(counts, E, row_lo, nrows, tiles, cap, hot, hot_min, hot_cap);
    NQ_LAUNCH_CHECK("nq_pf_plan");
    return 0;
}

struct PfGemm
{
    const int64_t* table; const int32_t* tiles;   // tiles [ntiles][4]: expert, first row, rows (<= 16 TG), unused
    const _Float16* A0; const _Float16* A1;         // activations in B-operand order: A0 for weight rows < I (or all rows of down), A1 above
    float* C; int mode, E, H, I;
    int solo;                                       // the other kernel variant will not be launched on these tiles: a tile that is its kind comes out NaN
    const u32x4* Wop;                               // decoded weights of hot experts in A-operand order (nq_pf_wdecode_k), or null
};

// ---- decoded-weight scratch of hot experts --------------------------------------------------------------------------------
// An expert with many pair rows is cut into several 256-row tiles, and every tile's workgroups would decode the expert again.
// Such experts are decoded once per call instead, into fp16 scratch laid out exactly as the grouped GEMM holds weights in
// registers: for strip pair sp (32 weight rows), chunk c, MFMA (mm, rho) one 1 KB block of 64 lanes x 16 bytes, the A operand of
// that MFMA. A tile of a hot expert then loads its operands (coalesced, 16 bytes per lane) where the others decode.
// Slot k of the scratch holds gate|up ([2I / 32][H / 128][8] blocks) followed by down ([H / 32][I / 128][8] blocks).
__device__ __forceinline__ size_t wop_base(int slot, int mode, int H, int I)
{   // in 16-byte units
    const size_t gu = (size_t)(2 * I / 32) * (H / 128) * 8 * 64, dn = (size_t)(H / 32) * (I / 128) * 8 * 64;
    return (size_t)slot * (gu + dn) + (mode ? gu : 0);
}

template <bool RES, int CODE>
__device__ __forceinline__ void wdecode_chunks(const Planes& P, const LaneCtx& L, int C, u32x4* dst, int lane)
{
    constexpr int NW = RES ? Rec<CODE>::NW : 1;
    u32x4 nb = P.base[L.rec0];
    uint32_t nr[NW + 2] = {0}, ndw = 0, nvar = 0;
    if constexpr (RES) { load_record<CODE>(nr, P.res, L.rec0, L.nrec); ndw = P.dw[L.unit0]; }
    if (P.var) nvar = P.var[L.unit0];
    for (int c = 0; c < C; ++c)
    {
        uint32_t wb[6], wr[NW + 2];
        wb[0] = nb.x; wb[1] = nb.y; wb[2] = nb.z; wb[3] = nb.w;
#pragma unroll
        for (int i = 0; i < NW; ++i) wr[i] = nr[i];
        const uint32_t dw = ndw, var = nvar;
        if (c + 1 < C)
        {
            nb = P.base[L.rec0 + (size_t)(c + 1) * 32];
            if constexpr (RES) { load_record<CODE>(nr, P.res, L.rec0 + (size_t)(c + 1) * 32, L.nrec); ndw = P.dw[L.unit0 + c + 1]; }
            if (P.var) nvar = P.var[L.unit0 + c + 1];
        }
        ext_base<0>(wb, __shfl(wb[0], L.src));
        const uint32_t sgm = ((var >> L.g) & 1u) * 0x80008000u;
        FoldK k;
        if constexpr (RES) { prepare_record<CODE>(wr); ext_words<Rec<CODE>::BITS, Rec<CODE>::NW>(wr, __shfl(wr[0], L.src)); k = consts_fold(dw, sgm); }
        else k = consts_l2(sgm);
        u32x4* d = dst + (size_t)c * 8 * 64 + lane;
        static_for<4>([&](auto mm) {
            constexpr int MM = decltype(mm)::value;
            d[(MM * 2 + 0) * 64] = __builtin_bit_cast(u32x4, a_operand<RES, CODE, MM, 0>(wb, wr, k));
            d[(MM * 2 + 1) * 64] = __builtin_bit_cast(u32x4, a_operand<RES, CODE, MM, 1>(wb, wr, k));
        });
    }
}

// grid (N / 128, E), block 256: block (x, e) decodes 128 weight rows of expert e if it has a scratch slot (hot[e] >= 0) and its
// row is of the common kind (K = 2 base plane, no mask-mode flags; others keep decoding inside the GEMM, whatever hot[] says)
__global__ void __launch_bounds__(256) nq_pf_wdecode_k(const int64_t* table, const int32_t* hot, int mode, u32x4* Wop, int H, int I)
{
    const int e = blockIdx.y, slot = hot[e];
    if (slot < 0) return;
    const int64_t* ent = table + (size_t)e * TBL_W;
    const int lv = (int)ent[0];
    if (lv <= 0) return;
    const Planes P = planes_of(ent, mode);
    if (P.bcode != 0 || P.flags != nullptr) return;
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6;
    const int N = mode == 0 ? 2 * I : H, K = mode == 0 ? H : I, C = K / 128;
    const int sp = blockIdx.x * 4 + warp, t4 = lane >> 4, ss = (lane >> 3) & 1, g = lane & 7;
    LaneCtx L;
    L.unit0 = (size_t)(2 * sp + ss) * C; L.rec0 = L.unit0 * 32 + 4 * g + t4;
    L.nrec = (size_t)(N / 16) * C * 32;
    L.src = (lane + 16) & 63; L.g = g; L.xs = nullptr; L.xstep = 0;
    L.strip = (size_t)(2 * sp + ss); L.nstrips = (size_t)(N / 16); L.chunk0 = 0;
    u32x4* dst = Wop + wop_base(slot, mode, H, I) + (size_t)sp * C * 8 * 64;
    if (lv == 2) wdecode_chunks<false, 0>(P, L, C, dst, lane);
    else dispatch_code(P.code, [&](auto tag) { wdecode_chunks<true, decltype(tag)::value>(P, L, C, dst, lane); });
}

int launch_pf_wdecode(const int64_t* table, const int32_t* hot, int E, int mode, void* Wop, int H, int I, hipStream_t st)
{
    const int N = mode == 0 ? 2 * I : H;
    nq_pf_wdecode_k<<<dim3(N / 128, E), 256, 0, st>>>(table, hot, mode, (u32x4*)Wop, H, I);
    NQ_LAUNCH_CHECK("nq_pf_wdecode");
    return 0;
}


// The MFMA phase of one chunk: TG x 8 MFMAs, tokens 16 tg + n as the N dimension (row groups beyond the tile multiply stale
// LDS rows whose results are never stored). Two row groups are interleaved so that four different accumulators separate an
// MFMA from the next one that depends on it, and the operand reads run one group (one mm of two row groups) ahead of the
// MFMAs that use them.
template <int TG>
__device__ __forceinline__ void pf_mfmas(const half8_t (*aop)[2], const char* smem, const uint32_t* boff, float4_t (*acc)[2])
{
    constexpr int TS = TG >= 2 ? 2 : 1, NGRP = TG / TS * 4;
    half8_t bq[2][TS];
    auto bread = [&](int grp, half8_t* dst) {
        const int tg = grp / 4 * TS, mm = grp % 4;
#pragma unroll
        for (int u = 0; u < TS; ++u) dst[u] = *(const half8_t*)(smem + boff[mm] + (tg + u) * 16 * PF_ROW);
    };
    bread(0, bq[0]);
#pragma unroll
    for (int gq = 0; gq < NGRP; ++gq)
    {
        if (gq + 1 < NGRP) bread(gq + 1, bq[(gq + 1) % 2]);
        __builtin_amdgcn_sched_barrier(0);
        const int tg = gq / 4 * TS, mm = gq % 4;
#pragma unroll
        for (int u = 0; u < TS; ++u)
        {
            const half8_t b = bq[gq % 2][u];
            acc[tg + u][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop[mm][0], b, acc[tg + u][0], 0, 0, 0);
            acc[tg + u][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop[mm][1], b, acc[tg + u][1], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Token staging shared by the GEMM bodies: wavefront w copies rows 16 u + 4 w + (lane >> 4), u = 0 .. TG - 1, of the tile, one
// 1 KB global -> LDS load per u (64 lanes x 16 bytes land in LDS in lane order, so a load fills 4 rows x 256 bytes). The lane
// picks which 16-byte column of its row it fetches: column (lane & 15) ^ (row & 15) goes to slot lane & 15, and the MFMA reads
// undo the XOR, which spreads the 16 tokens of an operand read over all banks without padding. Rows beyond the tile re-read
// its last row: their products are never stored.
// PART = 0 .. 3 issues a quarter of the loads (all of them in part 0 when there are fewer than four): the decode-fused body
// spreads them over its decode, because the texture path takes 16 clocks per 1 KB load and a wavefront that issues sixteen in
// a row stalls behind its own requests (measured: 1450 clocks per chunk at 256 rows) with the record loads queued after them.
template <int TG, int PART = -1>
__device__ __forceinline__ void pf_stage_tokens(const _Float16* A, int K, int row0, int nrows, int c, char* smem, int warp, int srow, uint32_t scol)
{
    typedef const __attribute__((address_space(1))) void* gvp;
    typedef __attribute__((address_space(3))) void* lvp;
    constexpr int U0 = PART < 0 ? 0 : (TG >= 4 ? PART * (TG / 4) : 0), U1 = PART < 0 ? TG : (TG >= 4 ? U0 + TG / 4 : (PART == 0 ? TG : 0));
    // uniform base of the tile's chunk (scalar registers) + a 32-bit lane offset inside the tile; the offset passes through an
    // empty asm so that the addresses of a part are formed when the part is issued, not sixteen of them ahead of the decode
    const char* base = (const char*)A + ((size_t)row0 * K + c * 128) * 2;
    uint32_t lane_off = (uint32_t)(srow * K * 2) + scol;
    asm volatile("" : "+v"(lane_off));
    const uint32_t ustep = (uint32_t)(16 * K * 2);
    const uint32_t last_off = (uint32_t)((nrows - 1) * K * 2) + scol;
#pragma unroll
    for (int u = U0; u < U1; ++u)
    {
        if constexpr (PART < 0) { if (16 * u >= nrows) break; }  // block-uniform; the spread parts stay free of branches
        uint32_t off = lane_off + (uint32_t)u * ustep;
        off = 16 * u + srow < nrows ? off : last_off;
        __builtin_amdgcn_global_load_lds((gvp)(base + off), (lvp)(smem + (16 * u + 4 * warp) * PF_ROW), 16, 0, 0);
    }
}

// body for a tile of a hot expert: the A operands of this wavefront's two strips come from the decoded-weight scratch
// (w: this strip pair's blocks, [C][8][64] x 16 bytes), one chunk ahead of the MFMAs that use them
template <int TG>
__device__ __forceinline__ void pf_chunks_pre(const u32x4* w, int C, const _Float16* A, int K, int row0, int nrows, char* smem, float4_t (*acc)[2])
{
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6, t4 = lane >> 4, n = lane & 15;
    const int srow = 4 * warp + t4;
    const uint32_t scol = (uint32_t)((n ^ srow) * 16);
    uint32_t boff[4];
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) boff[mm] = (uint32_t)(n * PF_ROW + (((4 * mm + t4) ^ n) << 4));
    u32x4 nx[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) nx[i] = w[(size_t)i * 64 + lane];
    for (int c = 0; c < C; ++c)
    {
        pf_stage_tokens<TG>(A, K, row0, nrows, c, smem, warp, srow, scol);
        half8_t aop[4][2];
#pragma unroll
        for (int i = 0; i < 8; ++i) aop[i >> 1][i & 1] = __builtin_bit_cast(half8_t, nx[i]);
        if (c + 1 < C)
        {
#pragma unroll
            for (int i = 0; i < 8; ++i) nx[i] = w[((size_t)(c + 1) * 8 + i) * 64 + lane];
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // the tokens have landed (and the next chunk's operands, requested with them)
        __syncthreads();
        pf_mfmas<TG>(aop, smem, boff, acc);
        __syncthreads();
    }
}

// body for one (RES, CODE): all K / 128 chunks of this wave's two strips against the tile's tokens
template <int TG, bool RES, int CODE, bool MASKED, int BK = 0>
__device__ __forceinline__ void pf_chunks(const Planes& P, const LaneCtx& L, int C, const _Float16* A, int K, int row0, int nrows,
                                          char* smem, float4_t (*acc)[2])
{
    constexpr int NW = RES ? Rec<CODE>::NW : 1;
    u32x4 nb = load_base<BK>(P, L.rec0, L.nrec);
    uint32_t nr[NW + 2] = {0}, ndw = 0, nvar = 0;
    constexpr bool masked = RES && MASKED;                       // the kernel variant for experts in mask mode
    // an expert without flags that comes through this variant (base code other than 0) reads as "every chunk refined",
    // for which the compact residual indexing is the dense one
    const uint64_t mflags = masked ? (P.flags ? P.flags[L.strip] : (C >= 64 ? ~0ull : (1ull << C) - 1ull)) : 0ull;
    if constexpr (RES && !masked) { load_record<CODE>(nr, P.res, L.rec0, L.nrec); ndw = P.dw[L.unit0]; }
    if (P.var) nvar = P.var[L.unit0];
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6, t4 = lane >> 4, n = lane & 15;
    // Staging: wavefront w copies rows 16 u + 4 w + (lane >> 4), u = 0 .. TG - 1, of the tile, one 1 KB
    // global -> LDS load per u (64 lanes x 16 bytes land in LDS in lane order, so a load fills 4 rows x 256 bytes). The
    // lane picks which 16-byte column of its row it fetches: column (lane & 15) ^ (row & 15) goes to slot lane & 15, and
    // the MFMA reads undo the XOR, which spreads the 16 tokens of an operand read over all banks without padding.
    // Rows beyond the tile re-read its last row: their products are never stored.
    const int srow = 4 * warp + t4;                              // row & 15 of every row this lane stages
    const uint32_t scol = (uint32_t)((n ^ srow) * 16);           // byte offset of the fetched column inside the chunk
    uint32_t boff[4];                                            // B-operand read offsets of this lane for mm = 0..3
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) boff[mm] = (uint32_t)(n * PF_ROW + (((4 * mm + t4) ^ n) << 4));
    for (int c = 0; c < C; ++c)
    {
        // ---- decode this wave's unit pair of chunk c into A operands; prefetch chunk c + 1; request the tile's tokens for chunk c
        // a quarter at a time between the decode stages (asynchronous: they arrive while the decode runs)
        uint32_t wb[6], wr[NW + 2];
        wb[0] = nb.x; wb[1] = nb.y; wb[2] = nb.z; wb[3] = nb.w;
#pragma unroll
        for (int i = 0; i < NW; ++i) wr[i] = nr[i];
        uint32_t dw = ndw;
        const uint32_t var = nvar;
        bool on = true;                                          // mask mode: is chunk c refined? (the same for the whole workgroup)
        if constexpr (masked)
            {   // residual records are compact over the refined chunks and fetched when needed
                const MaskedUnit m = masked_unit(mflags, L.strip, c, L.nstrips);
                on = __builtin_amdgcn_readfirstlane((int)m.on) != 0;
                if (on) { load_record<CODE>(wr, P.res, m.unit * 32 + (L.rec0 & 31), m.nrec); dw = P.dw[m.unit]; }
            }
        if (c + 1 < C)
        {
            nb = load_base<BK>(P, L.rec0 + (size_t)(c + 1) * 32, L.nrec);
            if constexpr (RES && !masked) { load_record<CODE>(nr, P.res, L.rec0 + (size_t)(c + 1) * 32, L.nrec); ndw = P.dw[L.unit0 + c + 1]; }
            if (P.var) nvar = P.var[L.unit0 + c + 1];
        }
        ext_base<BK>(wb, __shfl(wb[0], L.src));
        const uint32_t sgm = ((var >> L.g) & 1u) * 0x80008000u;
        half8_t aop[4][2];
        if (RES && (!masked || on))
        {
            if constexpr (RES)
            {
                prepare_record<CODE>(wr);
                ext_words<Rec<CODE>::BITS, Rec<CODE>::NW>(wr, __shfl(wr[0], L.src));
                const FoldK k = consts_fold(dw, sgm);
                static_for<4>([&](auto mm) {
                    constexpr int MM = decltype(mm)::value;
                    pf_stage_tokens<TG, MM>(A, K, row0, nrows, c, smem, warp, srow, scol);
                    aop[MM][0] = a_operand<RES, CODE, MM, 0, BK>(wb, wr, k);
                    aop[MM][1] = a_operand<RES, CODE, MM, 1, BK>(wb, wr, k);
                });
            }
        }
        else
        {
            const FoldK k = consts_l2(sgm);
            static_for<4>([&](auto mm) {
                constexpr int MM = decltype(mm)::value;
                pf_stage_tokens<TG, MM>(A, K, row0, nrows, c, smem, warp, srow, scol);
                aop[MM][0] = a_operand<false, 0, MM, 0, BK>(wb, wr, k);
                aop[MM][1] = a_operand<false, 0, MM, 1, BK>(wb, wr, k);
            });
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // this wavefront's share of the tile has landed
        __syncthreads();
        __builtin_amdgcn_s_setprio(3);                           // MFMA phase first: see below
        pf_mfmas<TG>(aop, smem, boff, acc);
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();                                         // every wavefront has read chunk c before chunk c + 1 overwrites it
    }
}

// grid (N / 128, ntiles), block 256 (4 wavefronts x 2 strips = 128 weight rows); dynamic LDS = 16 TG * PF_ROW bytes
// two workgroups per CU at every tile height (the tallest would otherwise need one register too many): while one decodes on
// the vector ALUs the other runs its MFMAs
// MASKED = false skips the tiles of experts in mask mode (table flags word set) or with a base window code other than 0,
// MASKED = true takes only those: the rarely used paths keep their extra registers out of the common kernel
template <int TG, bool MASKED>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) nq_pf_gemm_k(PfGemm a)
{
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63, warp = threadIdx.x >> 6;
    const int32_t* tile = a.tiles + 4 * blockIdx.y;
    const int e = tile[0], row0 = tile[1], nrows = tile[2], slot = tile[3] - 1;
    if (e < 0 || e >= a.E || nrows <= 0) return;
    const int64_t* ent = a.table + (size_t)e * TBL_W;
    const int lv = (int)ent[0];
    if (lv <= 0) return;                                         // rows of a level-0 expert are skipped downstream
    const int N = a.mode == 0 ? 2 * a.I : a.H, K = a.mode == 0 ? a.H : a.I, C = K / 128;
    const int sp = blockIdx.x * 4 + warp;                        // strip pair of this wavefront
    const _Float16* A = (a.mode == 0 && (int)(blockIdx.x * 128) >= a.I) ? a.A1 : a.A0;
    const int t4 = lane >> 4, ss = (lane >> 3) & 1, g = lane & 7, n = lane & 15;
    const Planes P = planes_of(ent, a.mode);
    if (((P.flags != nullptr && lv == 4) || P.bcode != 0) != MASKED)              // block-uniform: the other variant's tile
    {
        if (a.solo)
        {   // nobody will compute it (the host vouched for rows of one kind only): NaN, not whatever the scratch held
            const float nan = __builtin_nanf("");
            for (int i = threadIdx.x; i < nrows * 32; i += blockDim.x)
                *(float4_t*)(a.C + (size_t)(row0 + i / 32) * N + blockIdx.x * 128 + 4 * (i % 32)) = float4_t{nan, nan, nan, nan};
        }
        return;
    }
    LaneCtx L;
    L.unit0 = (size_t)(2 * sp + ss) * C; L.rec0 = L.unit0 * 32 + 4 * g + t4;
    L.nrec = (size_t)(N / 16) * C * 32;
    L.src = (lane + 16) & 63; L.g = g; L.xs = nullptr; L.xstep = 0;
    L.strip = (size_t)(2 * sp + ss); L.nstrips = (size_t)(N / 16); L.chunk0 = 0;
    float4_t acc[TG][2];
#pragma unroll
    for (int tg = 0; tg < TG; ++tg) { acc[tg][0] = float4_t{0.f, 0.f, 0.f, 0.f}; acc[tg][1] = float4_t{0.f, 0.f, 0.f, 0.f}; }
    if constexpr (!MASKED)
    {
        // a hot expert (several tiles): its weights were decoded once into the scratch by nq_pf_wdecode_k (block-uniform)
        const bool pre = a.Wop != nullptr && slot >= 0 && P.flags == nullptr;
        if (pre) pf_chunks_pre<TG>(a.Wop + wop_base(slot, a.mode, a.H, a.I) + (size_t)sp * C * 8 * 64, C, A, K, row0, nrows, smem, acc);
        else if (lv == 2) pf_chunks<TG, false, 0, false>(P, L, C, A, K, row0, nrows, smem, acc);
        else dispatch_code(P.code, [&](auto tag) { pf_chunks<TG, true, decltype(tag)::value, false>(P, L, C, A, K, row0, nrows, smem, acc); });
    }
    else
        dispatch_base(P.bcode, [&](auto bk) {
            constexpr int BK = decltype(bk)::value;
            if (lv == 2) pf_chunks<TG, false, 0, false, BK>(P, L, C, A, K, row0, nrows, smem, acc);
            else dispatch_code(P.code, [&](auto tag) { pf_chunks<TG, true, decltype(tag)::value, true, BK>(P, L, C, A, K, row0, nrows, smem, acc); });
        });
    // lane (t4, n) holds, for token 16 tg + n, weight rows 32 sp + 16 (t4 >> 1) + 4 (t4 & 1) + i (+ 8 for acc[..][1])
    const int wrow = 32 * sp + 16 * (t4 >> 1) + 4 * (t4 & 1);
#pragma unroll
    for (int tg = 0; tg < TG; ++tg)
    {
        const int tok = 16 * tg + n;
        if (tok < nrows)
        {
            float* c = a.C + (size_t)(row0 + tok) * N + wrow;
            *(float4_t*)c = acc[tg][0];
            *(float4_t*)(c + 8) = acc[tg][1];
        }
    }
}

int launch_pf_pre(const void* x, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg, void* xu, float* zg, int E, int H, int I,
                  const int32_t* tiles, int cap, int heights, hipStream_t st)
{
    if (!np) return 0;
    nq_pf_pre_k<<<np, 256, 0, st>>>((const _Float16*)x, pt, pe, table, (_Float16*)xg, (_Float16*)xu, zg, E, H, I, tiles, cap, heights);
    NQ_LAUNCH_CHECK("nq_pf_pre");
    return 0;
}
int launch_pf_mid(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h, const float* zg, float* zd, int E, int H, int I,
                  const int32_t* tiles, int cap, int heights, hipStream_t st)
{
    if (!np) return 0;
    nq_pf_mid_k<<<np, 256, 0, st>>>(acc_gu, pe, table, (_Float16*)h, zg, zd, E, H, I, tiles, cap, heights);
    NQ_LAUNCH_CHECK("nq_pf_mid");
    return 0;
}
int launch_pf_post(const float* y, const int32_t* pos, const int64_t* sel, const void* rw, int T, int topk, int row_lo, int nrows,
                   const int64_t* table, float* out, const float* zd, int E, int H, int I, hipStream_t st)
{
    if (!T || !nrows) return 0;
    nq_pf_post_k<<<T, 256, 0, st>>>(y, pos, sel, (const _Float16*)rw, topk, row_lo, nrows, table, out, zd, E, H, I);
    NQ_LAUNCH_CHECK("nq_pf_post");
    return 0;
}
int launch_pf_hits(const int32_t* counts, int32_t* hits, int E, hipStream_t st)
{
    nq_pf_hits_k<<<(E + 255) / 256, 256, 0, st>>>(counts, hits, E);
    NQ_LAUNCH_CHECK("nq_pf_hits");
    return 0;
}

template <int TG, bool MASKED>
static int launch_gemm_tg(const PfGemm& a, int ntiles, int N, hipStream_t st)
{
    const int shm = 16 * TG * PF_ROW;
    if (shm > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute((const void*)nq_pf_gemm_k<TG, MASKED>, hipFuncAttributeMaxDynamicSharedMemorySize, shm);
        if (e != hipSuccess) return set_error("nq_pf_gemm: LDS %d bytes: %s", shm, hipGetErrorString(e));
    }
    nq_pf_gemm_k<TG, MASKED><<<dim3(N / 128, ntiles), 256, shm, st>>>(a);
    NQ_LAUNCH_CHECK("nq_pf_gemm");
    return 0;
}

int launch_pf_gemm(const int64_t* table, const int32_t* tiles, int ntiles, int bm, int mode, const void* A0, const void* A1, float* C,
                   int E, int H, int I, const void* Wop, hipStream_t st)
{
    if (!ntiles) return 0;
    PfGemm a{table, tiles, (const _Float16*)A0, (const _Float16*)A1, C, mode & 1, E, H, I, (mode & 4) != 0, (const u32x4*)Wop};
    const int N = (mode & 1) == 0 ? 2 * I : H;
    const bool masked = (mode & 2) != 0;
    switch (bm)
    {
        case 16: return masked ? launch_gemm_tg<1, true>(a, ntiles, N, st) : launch_gemm_tg<1, false>(a, ntiles, N, st);
        case 32: return masked ? launch_gemm_tg<2, true>(a, ntiles, N, st) : launch_gemm_tg<2, false>(a, ntiles, N, st);
        case 64: return masked ? launch_gemm_tg<4, true>(a, ntiles, N, st) : launch_gemm_tg<4, false>(a, ntiles, N, st);
        case 128: return masked ? launch_gemm_tg<8, true>(a, ntiles, N, st) : launch_gemm_tg<8, false>(a, ntiles, N, st);
        case 256: return masked ? launch_gemm_tg<16, true>(a, ntiles, N, st) : launch_gemm_tg<16, false>(a, ntiles, N, st);
    }
    return set_error("nq_pf_gemm: tile height %d not in {16, 32, 64, 128, 256}", bm);
}

}  // namespace nq
