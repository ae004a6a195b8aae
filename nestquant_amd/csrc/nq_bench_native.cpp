// Torch-free driver of the C ABI (include/nq_moe_hip.h): builds one synthetic MoE layer with plain hipMalloc, runs the
// decode-path layer call eagerly and prints microseconds per call. It exists for two reasons: it is the smallest example
// of a host program binding the library without PyTorch, and it is a short program that rocprofv3 counter passes
// (--pmc FETCH_SIZE / WRITE_SIZE) can wrap; `--calib` adds one 256 MiB device copy as the known-size kernel that scales
// those counters.
//
//   nq_bench_native [--experts 64] [--batch 1] [--steps 32] [--calib] [--level L] [--prefill ROWS] [--hoist]
//
// --prefill ROWS times the decode-fused grouped GEMMs of the prefill path instead (nq_pf_gemm, gate|up then down): every
// expert gets ROWS pair rows (<= 256, one tile each); --level L puts every expert at level L.
//
// Planes are pseudo-random words (the decoder's cost does not depend on the values); levels cycle 2,2,2,3,4,2,2,4 so
// every step mixes levels; each step routes to 8 experts not used by the step before.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "../../include/nq_moe_hip.h"

#define HIPCHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)
#define NQCHK(x) do { if ((x) != 0) { fprintf(stderr, "%s: %s\n", #x, nq_last_error()); exit(1); } } while (0)

__global__ void fill_words(uint32_t* p, size_t n, uint32_t seed)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    {
        uint32_t x = (uint32_t)i * 2654435761u + seed; x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
        p[i] = x;
    }
}
__global__ void fill_block_words(uint32_t* p, size_t n, uint32_t seed)       // Mb in [120, 255], N = Mb / 2: always valid
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    {
        const uint32_t mb = 120u + ((uint32_t)i * 2654435761u + seed) % 136u;
        p[i] = mb | ((mb / 2u) << 8);
    }
}
__global__ void fill_half(uint16_t* p, size_t n, uint16_t v) { for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v; }
__global__ void copy_words(const uint4* __restrict__ a, uint4* __restrict__ b, size_t n) { for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) b[i] = a[i]; }

int main(int argc, char** argv)
{
    int E = 64, B = 1, steps = 32, calib = 0, level = 0, pf_rows = 0, hoist = 0;
    for (int i = 1; i < argc; ++i)
    {
        if (!strcmp(argv[i], "--experts") && i + 1 < argc) E = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--batch") && i + 1 < argc) B = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--steps") && i + 1 < argc) steps = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--calib")) calib = 1;
        else if (!strcmp(argv[i], "--hoist")) hoist = 1;
        else if (!strcmp(argv[i], "--level") && i + 1 < argc) level = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--prefill") && i + 1 < argc) pf_rows = atoi(argv[++i]);
        else { fprintf(stderr, "usage: %s [--experts E>=16] [--batch B<=8] [--steps K] [--calib] [--level 2|3|4] [--prefill ROWS<=256] [--hoist]\n", argv[0]); return 2; }
    }
    if ((level && level != 2 && level != 3 && level != 4) || pf_rows < 0 || pf_rows > 256) { fprintf(stderr, "need level in {2,3,4} and 0 <= ROWS <= 256\n"); return 2; }
    if (E < 16 || B < 1 || B > 8) { fprintf(stderr, "need E >= 16 and 1 <= B <= 8\n"); return 2; }
    const int H = 6144, I = 2048, topk = 8, S = B * topk;
    const size_t rec_gu = (size_t)(2 * I / 16) * (H / 128) * 32, rec_dn = (size_t)(H / 16) * (I / 128) * 32;
    const size_t units_gu = rec_gu / 32, units_dn = rec_dn / 32;
    static const int LV[8] = {2, 2, 2, 3, 4, 2, 2, 4};
    std::vector<int64_t> table((size_t)E * NQ_TBL_W, 0);
    uint16_t* signs; HIPCHK(hipMalloc(&signs, (size_t)(3 * H + 3 * I) * 2));
    fill_half<<<64, 256>>>(signs, 3 * H + 3 * I, 0x3C00);                    // all +1.0
    size_t plane_bytes = 0;
    for (int e = 0; e < E; ++e)
    {
        const int lv = level ? level : LV[e % 8];
        int64_t* r = &table[(size_t)e * NQ_TBL_W];
        r[0] = lv; r[9] = (int64_t)signs;
        const size_t recs[2] = {rec_gu, rec_dn}, units[2] = {units_gu, units_dn};
        for (int m = 0; m < 2; ++m)
        {
            uint32_t *base, *res = nullptr, *dw = nullptr;
            HIPCHK(hipMalloc(&base, recs[m] * 16)); fill_words<<<1024, 256>>>(base, recs[m] * 4, 17u * e + m);
            plane_bytes += recs[m] * 16;
            if (lv >= 3)
            {   // slot image: P3 sub-array, then P4 sub-array (8 bytes per record each), and one block word per unit
                HIPCHK(hipMalloc(&res, recs[m] * 16)); fill_words<<<1024, 256>>>(res, recs[m] * 4, 31u * e + m + 7);
                HIPCHK(hipMalloc(&dw, units[m] * 4)); fill_block_words<<<64, 256>>>(dw, units[m], e);
                plane_bytes += recs[m] * (lv == 3 ? 8 : 16) + units[m] * 4;
            }
            r[m == 0 ? 1 : 5] = (int64_t)base; r[m == 0 ? 2 : 6] = (int64_t)res; r[m == 0 ? 3 : 7] = (int64_t)dw;
            r[10 + m] = lv == 3 ? 10 : (lv == 4 ? 11 : 0);
        }
        NQCHK(nq_validate_row(r, H, I));
    }
    int64_t* d_table; HIPCHK(hipMalloc(&d_table, table.size() * 8));
    HIPCHK(hipMemcpy(d_table, table.data(), table.size() * 8, hipMemcpyHostToDevice));

    if (pf_rows)
    {
        const int np = E * pf_rows;
        int bm = 16; while (bm < pf_rows) bm *= 2;
        uint16_t *xg, *xu, *hh; float *cgu, *cdn; int32_t* tiles;
        HIPCHK(hipMalloc(&xg, (size_t)np * H * 2)); HIPCHK(hipMalloc(&xu, (size_t)np * H * 2)); HIPCHK(hipMalloc(&hh, (size_t)np * I * 2));
        HIPCHK(hipMalloc(&cgu, (size_t)np * 2 * I * 4)); HIPCHK(hipMalloc(&cdn, (size_t)np * H * 4));
        fill_half<<<1024, 256>>>(xg, (size_t)np * H, 0x2A66); fill_half<<<1024, 256>>>(xu, (size_t)np * H, 0x2A66); fill_half<<<1024, 256>>>(hh, (size_t)np * I, 0x2A66);
        std::vector<int32_t> ht((size_t)E * 4);
        for (int e = 0; e < E; ++e) { ht[4 * e] = e; ht[4 * e + 1] = e * pf_rows; ht[4 * e + 2] = pf_rows; ht[4 * e + 3] = 0; }
        HIPCHK(hipMalloc(&tiles, ht.size() * 4)); HIPCHK(hipMemcpy(tiles, ht.data(), ht.size() * 4, hipMemcpyHostToDevice));
        hipEvent_t e0, e1; HIPCHK(hipEventCreate(&e0)); HIPCHK(hipEventCreate(&e1));
        NQCHK(nq_pf_gemm(d_table, tiles, E, bm, 0, xg, xu, cgu, E, H, I, nullptr, nullptr)); NQCHK(nq_pf_gemm(d_table, tiles, E, bm, 1, hh, nullptr, cdn, E, H, I, nullptr, nullptr));
        HIPCHK(hipDeviceSynchronize());
        HIPCHK(hipEventRecord(e0, nullptr));
        for (int st = 0; st < steps; ++st)
        {
            NQCHK(nq_pf_gemm(d_table, tiles, E, bm, 0, xg, xu, cgu, E, H, I, nullptr, nullptr));
            NQCHK(nq_pf_gemm(d_table, tiles, E, bm, 1, hh, nullptr, cdn, E, H, I, nullptr, nullptr));
        }
        HIPCHK(hipEventRecord(e1, nullptr)); HIPCHK(hipEventSynchronize(e1));
        float ms; HIPCHK(hipEventElapsedTime(&ms, e0, e1));
        const double flop = 2.0 * np * 3.0 * H * I;
        printf("nq_bench_native prefill: E=%d tiles of %d rows (height %d), level %d: %.3f ms per gate|up + down pair, %.1f TFLOP/s, %.2f us per tile\n",
               E, pf_rows, bm, level, ms / steps, flop / (ms / steps * 1e-3) / 1e12, ms * 1e3 / steps / E);
        return 0;
    }

    const int cfg_gu[4] = {1, 4, 12, 0}, cfg_dn[4] = {1, 4, 4, 0};
    const int ny_gu = H / 128 / (cfg_gu[0] * cfg_gu[2]), ny_dn = I / 128 / (cfg_dn[0] * cfg_dn[2]);
    uint16_t *x, *rw, *h; int64_t* sel; float *out, *acc_gu, *acc_d, *zd; int32_t *cnt_gu, *cnt_d, *cnt_h;
    HIPCHK(hipMalloc(&x, (size_t)B * H * 2)); fill_half<<<64, 256>>>(x, (size_t)B * H, 0x2A66);   // 0.05
    HIPCHK(hipMalloc(&rw, (size_t)S * 2)); fill_half<<<1, 64>>>(rw, S, 0x3000);                    // 0.125
    HIPCHK(hipMalloc(&sel, (size_t)steps * S * 8));
    HIPCHK(hipMalloc(&h, (size_t)S * I * 2)); HIPCHK(hipMalloc(&out, (size_t)B * H * 4));
    HIPCHK(hipMalloc(&acc_gu, (size_t)ny_gu * S * 2 * I * 4)); HIPCHK(hipMalloc(&acc_d, (size_t)ny_dn * S * H * 4));
    HIPCHK(hipMalloc(&cnt_gu, (size_t)S * (I / 128) * 4)); HIPCHK(hipMalloc(&cnt_d, (size_t)(H / 128) * 4));
    HIPCHK(hipMalloc(&cnt_h, (size_t)S * (I / 128) * 4)); HIPCHK(hipMemset(cnt_h, 0, (size_t)S * (I / 128) * 4));
    HIPCHK(hipMalloc(&zd, (size_t)S * (I / 128) * 4 * sizeof(float)));
    void* route_ws; HIPCHK(hipMalloc(&route_ws, NQ_ROUTE_WS_BYTES));
    void* xrot; HIPCHK(hipMalloc(&xrot, (size_t)S * 2 * H * 2));
    HIPCHK(hipMemset(cnt_gu, 0, (size_t)S * (I / 128) * 4)); HIPCHK(hipMemset(cnt_d, 0, (size_t)(H / 128) * 4));
    std::vector<int64_t> hsel((size_t)steps * S);
    for (int st = 0; st < steps; ++st)                                        // distinct picks; a step never reuses the previous step's experts
        for (int b = 0; b < B; ++b)
            for (int k = 0; k < topk; ++k) hsel[((size_t)st * B + b) * topk + k] = ((int64_t)16 * st + 8 * b + k) % E;
    HIPCHK(hipMemcpy(sel, hsel.data(), hsel.size() * 8, hipMemcpyHostToDevice));
    HIPCHK(hipDeviceSynchronize());

    if (calib)
    {
        const size_t n = (size_t)256 << 20; uint4 *a, *b;
        HIPCHK(hipMalloc(&a, n)); HIPCHK(hipMalloc(&b, n)); HIPCHK(hipMemset(a, 1, n));
        copy_words<<<4096, 256>>>(a, b, n / 16);
        HIPCHK(hipDeviceSynchronize());
    }

    NqMoeArgs a; memset(&a, 0, sizeof a);
    a.x = x; a.rw = rw; a.table = d_table; a.out = out; a.acc_gu = acc_gu; a.h = h; a.acc_d = acc_d; a.cnt_gu = cnt_gu; a.cnt_d = cnt_d;
    a.acc_gu_elems = (int64_t)ny_gu * S * 2 * I; a.acc_d_elems = (int64_t)ny_dn * S * H; a.h_elems = (int64_t)S * I; a.out_elems = (int64_t)B * H;
    a.cnt_gu_elems = (int64_t)S * (I / 128); a.cnt_d_elems = H / 128; a.cnt_h = cnt_h; a.cnt_h_elems = (int64_t)S * (I / 128); a.zd = zd; a.zd_elems = (int64_t)S * (I / 128) * 4; a.route_ws = route_ws; a.route_ws_bytes = NQ_ROUTE_WS_BYTES; a.xrot = xrot; a.xrot_elems = (int64_t)S * 2 * H; a.common_rows = 1;   /* every row here has the K=2 base and a dense residual plane */
    a.B = B; a.topk = topk; a.E = E; a.H = H; a.I = I; a.which = 3; a.hoist_value_map = hoist;
    memcpy(a.cfg_gu, cfg_gu, sizeof cfg_gu); memcpy(a.cfg_dn, cfg_dn, sizeof cfg_dn);
    hipEvent_t e0, e1; HIPCHK(hipEventCreate(&e0)); HIPCHK(hipEventCreate(&e1));
    a.sel = sel; NQCHK(nq_moe_forward(&a, nullptr)); HIPCHK(hipDeviceSynchronize());            // warm-up
    HIPCHK(hipEventRecord(e0, nullptr));
    for (int st = 0; st < steps; ++st) { a.sel = sel + (size_t)st * S; NQCHK(nq_moe_forward(&a, nullptr)); }
    HIPCHK(hipEventRecord(e1, nullptr)); HIPCHK(hipEventSynchronize(e1));
    float ms; HIPCHK(hipEventElapsedTime(&ms, e0, e1));
    printf("nq_bench_native: E=%d B=%d steps=%d  %.2f us per layer call (eager launches, 3 kernels per call); resident planes %.1f MB\n",
           E, B, steps, ms * 1e3 / steps, plane_bytes / 1e6);
    return 0;
}
