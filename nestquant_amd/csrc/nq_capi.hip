// extern "C" surface of libnq_moe_hip.so (declarations and reference citations: include/nq_moe_hip.h).
// Argument checking happens here on the host; kernels assume the shapes these checks establish.
#include "../../include/nq_moe_hip.h"
#include "nq_decode.hpp"
#include "nq_host.hpp"
#include <string.h>

namespace nq {
char* error_buffer()
{
    static thread_local char buf[512] = {0};
    return buf;
}
static bool shape_ok(int H, int I) { return H > 0 && I > 0 && H % 128 == 0 && I % 128 == 0; }
// the kernels move 16 bytes per lane; rows are multiples of 256 bytes, so the base address decides
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
}  // namespace nq

using namespace nq;

extern "C" int nq_abi_version(void) { return NQ_ABI_VERSION; }
extern "C" const char* nq_last_error(void) { return error_buffer(); }

extern "C" int nq_codes(uint32_t out[4])
{
    NQ_REQUIRE(out, "nq_codes: null output");
    out[0] = out[1] = (1u << NCODES) - 1u;   // residual codes 0..12 in both kernels
    out[2] = out[3] = 3u;                     // base codes 0 (K = 2 ring base) and 1 (K = 1.75, sub-array layout)
    return 0;
}

extern "C" int nq_occ(int mode, int any_rows, int sb, int shm, int out[3])
{
    NQ_REQUIRE(out && (mode == 0 || mode == 1) && sb >= 1 && sb <= 16 && shm >= 0, "nq_occ: mode 0 / 1, 1..16 wavefronts per workgroup, an output array");
    return query_occ(mode, any_rows, sb, shm, out);
}

extern "C" int nq_validate_row(const int64_t* r, int H, int I)
{
    NQ_REQUIRE(r, "nq_validate_row: null row");
    NQ_REQUIRE(shape_ok(H, I), "nq_validate_row: H=%d I=%d must be positive multiples of 128", H, I);
    const int64_t lv = r[0];
    NQ_REQUIRE(lv == 0 || lv == 2 || lv == 3 || lv == 4, "table row: level %lld not in {0,2,3,4}", (long long)lv);
    if (lv == 0) return 0;
    NQ_REQUIRE(r[1] && r[5] && r[9], "table row: null base plane or sign vector");
    NQ_REQUIRE((r[4] == 0 && r[8] == 0) || lv == 2 || (lv == 4 && r[10] < CODE_L3 && r[11] < CODE_L3), "table row: mask mode (flags) goes with the wide residual plane of level 4 only");
    NQ_REQUIRE(r[14] ? (r[15] != 0 && r[16] >= 0 && r[16] <= 4 && r[17] >= 0 && r[17] <= 4 && r[16] + r[17] > 0) : (r[15] == 0 && r[16] == 0 && r[17] == 0),
               "table row: low-rank plane needs both buffers and ranks r_gu, r_dn in [0, 4] (got %lld, %lld)", (long long)r[16], (long long)r[17]);
    NQ_REQUIRE(r[18] == 0 || r[18] == 128 || (r[18] == 512 && I % 512 == 0), "table row: in_had_down %lld must be 0, 128, or 512 dividing I = %d", (long long)r[18], I);
    NQ_REQUIRE((r[19] & ~0x0101ll) == 0, "table row: base codes 0x%llx (gate|up | down << 8): only 0 (K=2) and 1 (K=1.75) are implemented", (long long)r[19]);
    if (lv >= 3)
    {
        NQ_REQUIRE(r[2] && r[3] && r[6] && r[7], "table row: level %lld needs residual planes and block words", (long long)lv);
        for (int m = 0; m < 2; ++m)
        {
            const int64_t c = r[10 + m];
            NQ_REQUIRE(c >= 0 && c < NCODES, "table row: residual code %lld out of range", (long long)c);
            NQ_REQUIRE(lv != 3 || c == CODE_L3, "table row: level 3 needs residual code %d (K=1 plane), got %lld", CODE_L3, (long long)c);
            NQ_REQUIRE(lv != 4 || c != CODE_L3, "table row: level 4 cannot use the level-3 code %d", CODE_L3);
        }
    }
    return 0;
}

extern "C" int nq_dequant(const int64_t* row, int proj, int level, int H, int I, void* out, void* stream)
{
    NQ_REQUIRE(row && out, "nq_dequant: null pointer");
    NQ_REQUIRE(proj == 0 || proj == 1, "nq_dequant: proj %d not in {0,1}", proj);
    NQ_REQUIRE(level == 0 || level == 2 || level == 3 || level == 4, "nq_dequant: level %d not in {0,2,3,4}", level);
    {   // a single projection only needs whole units: N % 16 == 0 and K % 128 == 0
        const int N = proj == 0 ? 2 * I : H, K = proj == 0 ? H : I;
        NQ_REQUIRE(H > 0 && I > 0 && N % 16 == 0 && K % 128 == 0, "nq_dequant: projection [%d][%d] is not whole 16x128 units", N, K);
    }
    return launch_dequant(row, proj, level, H, I, out, (hipStream_t)stream);
}

extern "C" int nq_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu, void* Wdn, int H, int I, void* stream)
{
    NQ_REQUIRE(G >= 0, "nq_pf_decode: G=%d", G);
    if (G == 0) return 0;
    NQ_REQUIRE(table && experts && Wgu && Wdn, "nq_pf_decode: null pointer");
    NQ_REQUIRE(shape_ok(H, I), "nq_pf_decode: H=%d I=%d must be positive multiples of 128", H, I);
    return launch_pf_decode(table, experts, G, Wgu, Wdn, H, I, (hipStream_t)stream);
}

extern "C" int nq_sal(const void* x, int x_dtype, int64_t x_row_stride, const void* w, int w_dtype, const void* ids, int ids_dtype,
                      int T, int H, int K, int E, double rsf, double* acc, double* host, void* stream)
{
    NQ_REQUIRE(T >= 0 && T <= 8 && K >= 1 && K <= 8, "nq_sal: T=%d K=%d (at most 8 tokens of at most 8 picks)", T, K);
    if (T == 0) return 0;
    NQ_REQUIRE(x && w && ids && acc && host, "nq_sal: null pointer");
    NQ_REQUIRE(H >= 1 && E >= 1 && x_row_stride >= H, "nq_sal: H=%d E=%d row stride %lld", H, E, (long long)x_row_stride);
    NQ_REQUIRE(x_dtype >= 0 && x_dtype <= 2 && w_dtype >= 0 && w_dtype <= 2 && ids_dtype >= 0 && ids_dtype <= 1,
               "nq_sal: dtype codes x=%d w=%d ids=%d", x_dtype, w_dtype, ids_dtype);
    return launch_sal(x, x_dtype, x_row_stride, w, w_dtype, ids, ids_dtype, T, H, K, E, (float)rsf, acc, host, (hipStream_t)stream);
}

// checks shared by the two decode entry points; own_ws: the caller brings the workspaces (nq_moe_forward), else they are
// carved from the library's built-in scratch (nq_moe_forward_static) and the workspace fields of *p are not looked at
static int moe_args(const char* who, const NqMoeArgs* p, bool own_ws, MoeArgs& a)
{
    NQ_REQUIRE(p, "%s: null args", who);
    NQ_REQUIRE(p->x && p->sel && p->rw && p->table && p->out, "%s: null pointer", who);
    NQ_REQUIRE(!own_ws || (p->acc_gu && p->h && p->acc_d && p->cnt_gu && p->cnt_d), "%s: null workspace pointer", who);
    NQ_REQUIRE(p->B >= 1 && p->B <= 8 && p->topk >= 1 && p->B * p->topk <= 64, "%s: B=%d topk=%d (B <= 8, B*topk <= 64)", who, p->B, p->topk);
    NQ_REQUIRE(p->E >= 1, "%s: E=%d", who, p->E);
    NQ_REQUIRE(shape_ok(p->H, p->I), "%s: H=%d I=%d must be positive multiples of 128", who, p->H, p->I);
    NQ_REQUIRE((p->which & ~15) == 0, "%s: which=%d", who, p->which);
    NQ_REQUIRE(!(p->which & 4) || own_ws, "%s: which bit 2 (routing of an earlier call) needs the caller's route_ws / xrot", who);
    NQ_REQUIRE(p->force_level == 0 || p->force_level == 2 || p->force_level == 3 || p->force_level == 4, "%s: force_level=%d", who, p->force_level);
    NQ_REQUIRE(p->x_dtype >= 0 && p->x_dtype <= 2 && p->rw_dtype >= 0 && p->rw_dtype <= 2 && p->sel_dtype >= 0 && p->sel_dtype <= 1 && p->out_dtype >= 0 && p->out_dtype <= 2,
               "%s: dtype codes x=%d sel=%d rw=%d out=%d", who, p->x_dtype, p->sel_dtype, p->rw_dtype, p->out_dtype);
    NQ_REQUIRE(aligned16(p->x) && aligned16(p->out), "%s: x and out must be 16-byte aligned", who);
    NQ_REQUIRE(!own_ws || (aligned16(p->acc_gu) && aligned16(p->acc_d) && aligned16(p->h)), "%s: acc_gu, acc_d and h must be 16-byte aligned", who);
    const int64_t S = (int64_t)p->B * p->topk;
    for (int mode = 0; mode < 2; ++mode)
    {
        const int32_t* cf = mode == 0 ? p->cfg_gu : p->cfg_dn;
        const int N = mode == 0 ? 2 * p->I : p->H, K = mode == 0 ? p->H : p->I, C = K / 128;
        NQ_REQUIRE(cf[0] >= 1 && cf[1] >= 1 && cf[2] >= 1 && cf[3] == 0, "bad cfg: {%d,%d,%d,%d} (cpw, sb, nst >= 1; persistent mode is not implemented)", cf[0], cf[1], cf[2], cf[3]);
        const int NC = cf[0] * cf[2], SB = cf[1];
        NQ_REQUIRE(C % NC == 0 && (SB == 1 || SB == 2 || SB == 4) && NC <= 48 && (N / 32) % SB == 0 && (mode == 1 || (p->I / 32) % SB == 0),
                   "bad cfg: k-slice %d chunks of %d, %d wavefronts per block for N=%d (sb must be 1, 2 or 4 and divide N / 32, for gate|up also I / 32)", NC, C, SB, N);
        const int64_t need = (int64_t)(C / NC) * S * N, have = mode == 0 ? p->acc_gu_elems : p->acc_d_elems;
        NQ_REQUIRE(!own_ws || have >= need, "workspace too small: %s holds %lld floats, needs %lld", mode == 0 ? "acc_gu" : "acc_d", (long long)have, (long long)need);
    }
    NQ_REQUIRE(p->out_elems >= (int64_t)p->B * p->H, "workspace too small: out");
    a = MoeArgs{};
    a.x = p->x; a.sel = p->sel; a.rw = p->rw; a.B = p->B; a.topk = p->topk;
    a.x_dtype = p->x_dtype; a.sel_dtype = p->sel_dtype; a.rw_dtype = p->rw_dtype; a.out_dtype = p->out_dtype;
    a.table = p->table; a.E = p->E; a.H = p->H; a.I = p->I;
    a.out = p->out; a.force_level = p->force_level; a.hits = p->hits;
    if (own_ws)
    {
        NQ_REQUIRE(p->h_elems >= S * p->I, "workspace too small: h");
        NQ_REQUIRE(p->cnt_gu_elems >= S * (p->I / 128) && p->cnt_d_elems >= p->H / 128, "workspace too small: cnt_gu or cnt_d");
        NQ_REQUIRE(p->cnt_h && p->cnt_h_elems >= S * (p->I / 128), "workspace too small: cnt_h");
        NQ_REQUIRE(p->zd && p->zd_elems >= S * (p->I / 128) * 4, "workspace too small: zd");
        a.part_gu = (float*)p->acc_gu; a.h = (_Float16*)p->h; a.part_d = (float*)p->acc_d;
        a.cnt_gu = p->cnt_gu; a.cnt_d = p->cnt_d; a.cnt_h = p->cnt_h; a.zd = (float*)p->zd;
        NQ_REQUIRE(p->route_ws && p->route_ws_bytes >= NQ_ROUTE_WS_BYTES && ((uintptr_t)p->route_ws & 63) == 0,
                   "workspace too small: route_ws needs %d bytes, 64-byte aligned", NQ_ROUTE_WS_BYTES);
        a.route = (RouteWs*)p->route_ws;
        NQ_REQUIRE(p->xrot && p->xrot_elems >= S * 2 * p->H && aligned16(p->xrot), "workspace too small: xrot needs B*topk * 2 * H halfs, 16-byte aligned");
        a.xrot = (_Float16*)p->xrot;
    }
    if (p->mb_table)
    {
        NQ_REQUIRE(p->mb_stage && p->mb_seq && p->mb_applied, "%s: mailbox needs stage, seq and applied", who);
        NQ_REQUIRE((const int64_t*)p->mb_table == p->table, "%s: the mailbox must be the one of the table the call reads", who);
        a.mb_table = p->mb_table; a.mb_stage = p->mb_stage; a.mb_seq = p->mb_seq; a.mb_applied = p->mb_applied; a.mb_applied_host = p->mb_applied_host;
    }
    NQ_REQUIRE(p->hoist_value_map == 0 || p->hoist_value_map == 1, "%s: hoist_value_map=%d (0 or 1)", who, p->hoist_value_map);
    a.hoist = p->hoist_value_map;
    NQ_REQUIRE(p->common_rows == 0 || p->common_rows == 1, "%s: common_rows=%d (0 or 1)", who, p->common_rows);
    a.common_rows = p->common_rows;
    NQ_REQUIRE(p->G == 0 || p->G == 4 || p->G == 2, "%s: G=%d (rings of 4 lanes, or 2)", who, p->G);
    a.G = p->G == 2 ? 2 : 4;
    return 0;
}

extern "C" int nq_moe_forward(const NqMoeArgs* p, void* stream)
{
    MoeArgs a;
    if (int rc = moe_args("nq_moe_forward", p, true, a)) return rc;
    return launch_moe(a, p->cfg_gu, p->cfg_dn, p->which, (hipStream_t)stream);
}

extern "C" int nq_moe_forward_static(const NqMoeArgs* p, void* stream)
{
    MoeArgs a;
    if (int rc = moe_args("nq_moe_forward_static", p, false, a)) return rc;
    return launch_moe_static(a, p->cfg_gu, p->cfg_dn, p->which, (hipStream_t)stream);
}

extern "C" int nq_mailbox(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E, void* stream)
{
    NQ_REQUIRE(table && stage && seq && applied, "nq_mailbox: null pointer");
    NQ_REQUIRE(E >= 1, "nq_mailbox: E=%d", E);
    return launch_mailbox(table, stage, seq, applied, applied_host, E, (hipStream_t)stream);
}

extern "C" int nq_pf_pre(const void* x, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg, void* xu,
                         float* zg, int E, int H, int I, void* stream)
{
    NQ_REQUIRE(np >= 0, "nq_pf_pre: np=%d", np);
    if (np == 0) return 0;
    NQ_REQUIRE(x && pt && pe && table && xg && xu, "nq_pf_pre: null pointer");
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_pre: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(x) && aligned16(xg) && aligned16(xu), "nq_pf_pre: x, xg and xu must be 16-byte aligned");
    return launch_pf_pre(x, pt, pe, np, table, xg, xu, zg, E, H, I, nullptr, 0, 0, (hipStream_t)stream);
}

extern "C" int nq_pf_pre_rows(const void* x, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg, void* xu,
                              float* zg, int E, int H, int I, const int32_t* tiles, int cap, int heights, void* stream)
{
    NQ_REQUIRE(np >= 0 && (heights & ~31) == 0, "nq_pf_pre_rows: np=%d, heights=0x%x (a mask of the five tile heights)", np, heights);
    if (np == 0 || heights == 0) return 0;
    NQ_REQUIRE(x && pt && pe && table && xg && xu && tiles, "nq_pf_pre_rows: null pointer");
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_pre_rows: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(x) && aligned16(xg) && aligned16(xu) && aligned16(tiles), "nq_pf_pre_rows: x, xg, xu and tiles must be 16-byte aligned");
    NQ_REQUIRE(cap >= E, "nq_pf_pre_rows: cap=%d below E=%d", cap, E);
    return launch_pf_pre(x, pt, pe, np, table, xg, xu, zg, E, H, I, tiles, cap, heights, (hipStream_t)stream);
}

extern "C" int nq_pf_gemm(const int64_t* table, const int32_t* tiles, int ntiles, int bm, int mode, const void* A0, const void* A1,
                          float* C, int E, int H, int I, const void* Wop, void* stream)
{
    NQ_REQUIRE(ntiles >= 0, "nq_pf_gemm: ntiles=%d", ntiles);
    if (ntiles == 0) return 0;
    NQ_REQUIRE(table && tiles && A0 && C, "nq_pf_gemm: null pointer");
    NQ_REQUIRE(mode >= 0 && mode <= 7, "nq_pf_gemm: mode %d not in 0..7", mode);
    NQ_REQUIRE((mode & 1) == 1 || A1, "nq_pf_gemm: gate|up needs both activation buffers");
    NQ_REQUIRE(ntiles <= 65535, "nq_pf_gemm: %d tiles exceed one launch (65535)", ntiles);
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_gemm: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(A0) && aligned16(A1) && aligned16(C) && aligned16(tiles), "nq_pf_gemm: tiles, activations and C must be 16-byte aligned");
    NQ_REQUIRE(aligned16(Wop), "nq_pf_gemm: the decoded-weight scratch must be 16-byte aligned");
    return launch_pf_gemm(table, tiles, ntiles, bm, mode, A0, A1, C, E, H, I, Wop, (hipStream_t)stream);
}

extern "C" int nq_pf_mid(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h, const float* zg, float* zd,
                         int E, int H, int I, void* stream)
{
    NQ_REQUIRE(np >= 0, "nq_pf_mid: np=%d", np);
    if (np == 0) return 0;
    NQ_REQUIRE(acc_gu && pe && table && h, "nq_pf_mid: null pointer");
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_mid: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(acc_gu) && aligned16(h), "nq_pf_mid: acc_gu and h must be 16-byte aligned");
    return launch_pf_mid(acc_gu, pe, np, table, h, zg, zd, E, H, I, nullptr, 0, 0, (hipStream_t)stream);
}

extern "C" int nq_pf_mid_rows(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h, const float* zg, float* zd,
                              int E, int H, int I, const int32_t* tiles, int cap, int heights, void* stream)
{
    NQ_REQUIRE(np >= 0 && (heights & ~31) == 0, "nq_pf_mid_rows: np=%d, heights=0x%x (a mask of the five tile heights)", np, heights);
    if (np == 0 || heights == 0) return 0;
    NQ_REQUIRE(acc_gu && pe && table && h && tiles, "nq_pf_mid_rows: null pointer");
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_mid_rows: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(acc_gu) && aligned16(h) && aligned16(tiles), "nq_pf_mid_rows: acc_gu, h and tiles must be 16-byte aligned");
    NQ_REQUIRE(cap >= E, "nq_pf_mid_rows: cap=%d below E=%d", cap, E);
    return launch_pf_mid(acc_gu, pe, np, table, h, zg, zd, E, H, I, tiles, cap, heights, (hipStream_t)stream);
}

extern "C" int nq_pf_post(const float* y, const int32_t* pos, const int64_t* sel, const void* rw, int T, int topk, int row_lo, int nrows,
                          const int64_t* table, float* out, const float* zd, int E, int H, int I, void* stream)
{
    NQ_REQUIRE(T >= 0 && nrows >= 0 && topk >= 1 && topk <= 64 && row_lo >= 0, "nq_pf_post: T=%d topk=%d (<= 64) row_lo=%d nrows=%d", T, topk, row_lo, nrows);
    if (T == 0 || nrows == 0) return 0;
    NQ_REQUIRE(y && pos && sel && rw && table && out, "nq_pf_post: null pointer");
    NQ_REQUIRE(E >= 1 && shape_ok(H, I), "nq_pf_post: E=%d H=%d I=%d (H, I positive multiples of 128)", E, H, I);
    NQ_REQUIRE(aligned16(y) && aligned16(out), "nq_pf_post: y and out must be 16-byte aligned");
    return launch_pf_post(y, pos, sel, rw, T, topk, row_lo, nrows, table, out, zd, E, H, I, (hipStream_t)stream);
}

extern "C" int nq_pf_wdecode(const int64_t* table, const int32_t* hot, int E, int mode, void* Wop, int64_t wop_bytes, int slots, int H, int I, void* stream)
{
    NQ_REQUIRE(table && hot && Wop, "nq_pf_wdecode: null pointer");
    NQ_REQUIRE(E >= 1 && E <= 65535 && (mode == 0 || mode == 1) && slots >= 1, "nq_pf_wdecode: E=%d (1..65535) mode=%d slots=%d", E, mode, slots);
    NQ_REQUIRE(shape_ok(H, I), "nq_pf_wdecode: H=%d I=%d (positive multiples of 128)", H, I);
    NQ_REQUIRE(aligned16(Wop) && wop_bytes >= (int64_t)slots * 3 * H * I * 2, "nq_pf_wdecode: the scratch needs %d slots of 3 * H * I halfs, 16-byte aligned", slots);
    return launch_pf_wdecode(table, hot, E, mode, Wop, H, I, (hipStream_t)stream);
}

extern "C" int nq_pf_plan(const int32_t* counts, int E, int row_lo, int nrows, int32_t* tiles, int cap, int32_t* hot, int hot_min, int hot_cap, void* stream)
{
    NQ_REQUIRE(counts && tiles, "nq_pf_plan: null pointer");
    NQ_REQUIRE(E >= 1 && E <= 4096 && row_lo >= 0 && nrows >= 0, "nq_pf_plan: E=%d (1..4096) row_lo=%d nrows=%d", E, row_lo, nrows);
    NQ_REQUIRE(aligned16(tiles), "nq_pf_plan: tiles must be 16-byte aligned");
    NQ_REQUIRE(cap >= E + nrows / 256 + 1, "nq_pf_plan: cap=%d, need at least E + nrows / 256 + 1 = %d", cap, E + nrows / 256 + 1);
    NQ_REQUIRE(!hot || (hot_min >= 1 && hot_cap >= 1), "nq_pf_plan: hot_min=%d hot_cap=%d (both at least 1 with a hot list)", hot_min, hot_cap);
    return launch_pf_plan(counts, E, row_lo, nrows, tiles, cap, hot, hot_min, hot_cap, (hipStream_t)stream);
}

extern "C" int nq_pf_hits(const int32_t* counts, int32_t* hits, int E, void* stream)
{
    NQ_REQUIRE(counts && E >= 1, "nq_pf_hits: null counts or E=%d", E);
    if (!hits) return 0;
    return launch_pf_hits(counts, hits, E, (hipStream_t)stream);
}
