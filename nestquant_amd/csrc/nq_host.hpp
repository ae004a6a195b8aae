// Host-side helpers shared by the translation units of libnq_moe_hip.so (internal; the public ABI is include/nq_moe_hip.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

namespace nq {

// last error text of the calling thread; every entry point returns 0 on success, non-zero after set_error()
char* error_buffer();
inline int set_error(const char* fmt, ...)
{
    va_list ap; va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return 1;
}
#define NQ_REQUIRE(cond, ...) do { if (!(cond)) return nq::set_error(__VA_ARGS__); } while (0)
#define NQ_LAUNCH_CHECK(what) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) return nq::set_error("%s: %s", what, hipGetErrorString(e_)); } while (0)

// arguments of one decode-path layer call (device pointers; see NqMoeArgs in include/nq_moe_hip.h)
struct RouteWs;                       // runs and picks of one call, written by the routing launch (nq_moe.hip)
struct MoeArgs
{
    const void* x; const void* sel; const void* rw; int B, topk;
    int x_dtype, sel_dtype, rw_dtype, out_dtype;   // NQ_DT_*: x / rw f16, bf16 or f32; sel i64 or i32; out f32, f16 or bf16
    const int64_t* table; int E, H, I;
    float* part_gu; _Float16* h; float* part_d; void* out;
    int force_level; int* hits;
    int* cnt_gu; int* cnt_d;          // arrival counters [S * I/128] and [H/128]: zero on entry, zero on exit
    float* zd;                        // low-rank plane: z_d partials [S][I/128][4], written by gate|up, read by down; may be null
    int* cnt_h;                       // arrival counters of the 512-column blocks (in_had_down = 512) [S * I/128]; may be null
    int G;                            // lanes per ring: 4, or 2 (the same planes read as rings of two records)
    int common_rows;                  // 1 = every row that can be picked has base window code 0 and no mask-mode flags; 0 = unknown
    int fuse;                         // both launches belong to this call: for runs whose row has neither a low-rank plane nor the
                                      // 512-wide rotation the down launch's staging does the gate|up finisher (set by launch_moe)
    RouteWs* route;                   // NQ_ROUTE_WS_BYTES of device memory: what the routing launch hands to the projection launches
    _Float16* xrot;                   // [B * topk][2][H] fp16: rotated activations of every active pick (gate, up), B-operand order
    int hoist;                        // NqMoeArgs::hoist_value_map: level-2 runs without a sign plane apply the value map to the sums
    int mb_apply;                     // this projection launch (the call's last) carries the block that applies the mailbox (set by launch_moe)
    int64_t* mb_table; const int64_t* mb_stage; const int32_t* mb_seq; int32_t* mb_applied; int32_t* mb_applied_host;
                                      // mailbox of the call (mb_table == nullptr: none): applied by the last projection launch, published by the next call's routing launch
};

// kernel launchers defined next to their kernels
int launch_moe(const MoeArgs& a, const int* cfg_gu, const int* cfg_dn, int which, hipStream_t st);
int launch_moe_static(MoeArgs a, const int* cfg_gu, const int* cfg_dn, int which, hipStream_t st);
int query_occ(int mode, int any_rows, int sb, int shm, int* out);
int launch_mailbox(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E, hipStream_t st);
int launch_dequant(const int64_t* row, int proj, int level, int H, int I, void* out, hipStream_t st);
int launch_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu, void* Wdn, int H, int I, hipStream_t st);
int launch_pf_pre(const void* x, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg, void* xu, float* zg, int E, int H, int I,
                  const int32_t* tiles, int cap, int heights, hipStream_t st);
int launch_pf_mid(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h, const float* zg, float* zd, int E, int H, int I,
                  const int32_t* tiles, int cap, int heights, hipStream_t st);
int launch_pf_post(const float* y, const int32_t* pos, const int64_t* sel, const void* rw, int T, int topk, int row_lo, int nrows,
                   const int64_t* table, float* out, const float* zd, int E, int H, int I, hipStream_t st);
int launch_sal(const void* x, int x_dtype, int64_t sx, const void* w, int w_dtype, const void* ids, int ids_dtype, int T, int H, int K,
               int E, float rsf, double* acc, double* host, hipStream_t st);
int launch_pf_plan(const int32_t* counts, int E, int row_lo, int nrows, int32_t* tiles, int cap, int32_t* hot, int hot_min, int hot_cap, hipStream_t st);
int launch_pf_wdecode(const int64_t* table, const int32_t* hot, int E, int mode, void* Wop, int H, int I, hipStream_t st);
int launch_pf_hits(const int32_t* counts, int32_t* hits, int E, hipStream_t st);
int launch_pf_gemm(const int64_t* table, const int32_t* tiles, int ntiles, int bm, int mode, const void* A0, const void* A1, float* C,
                   int E, int H, int I, const void* Wop, hipStream_t st);

}  // namespace nq
