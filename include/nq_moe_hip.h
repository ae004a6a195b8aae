/* libnq_moe_hip.so -- C ABI of the MI355X (gfx950) NestQuant routed-expert MoE hot path.
 *
 * Every pointer is a raw device address unless marked [host] or [host-mapped]; the library allocates nothing per call
 * and keeps no pointer after a call returns. All launches go to the stream passed in (a hipStream_t as void*, 0 = the
 * null stream). Entry points return 0 on success; otherwise non-zero and nq_last_error() describes the failure (the
 * reference raises TORCH_CHECK -> RuntimeError at the same points, sm120/nqmoe.cu:871-878,887,897).
 *
 * Table row = int64[NQ_TBL_W] per expert (reference sm120/moe.py:216-229, sm120/nqmoe.cu:26-45):
 *   [0] level 0/2/3/4   [1..4] gate|up: base, residual plane, block words, mask-mode flags (0 = none)   [5..8] down: same
 *   [9] fp16 sign/scale vector [H su_g | I sv_g | I sv_u | I su_d | H sv_o | H su_u]
 *   [10],[11] residual window code of gate|up, down (0..9 as the reference; 10 = nested K=1 plane P3; 11 = nested
 *   P3 || P4: uint2 sub-array of P3 followed by uint2 sub-array of P4)   [12],[13] sign-variant planes (0 = none)
 *   [14..17] low-rank plane: U/V buffers and ranks 0..4   [18] in_had_down 0 / 128 / 512   [19] base codes: 0 or 1 per projection
 */
#ifndef NQ_MOE_HIP_H
#define NQ_MOE_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define NQ_TBL_W 20
#define NQ_ABI_VERSION 3

/* library identification; no counterpart in the reference (its module is rebuilt per process by sm120/build.py:7-12) */
int nq_abi_version(void);
/* text of the calling thread's last failure (reference: the RuntimeError message of TORCH_CHECK) */
const char* nq_last_error(void);

/* Bit masks of the residual window codes compiled into {gate|up, down} of the decode kernels and the base codes
 * {gate|up, down}; replaces rk_codes() / bk_codes() (reference sm120/nqmoe.cu:938-940, sm120/moe.py:246-252). */
int nq_codes(uint32_t out[4]);

/* Occupancy of a decode kernel (mode 0 = gate|up, 1 = down; any_rows as NqMoeArgs.common_rows != 1) launched with sb
 * wavefronts per workgroup and shm bytes of dynamic LDS: out[0] = resident workgroups per CU, out[1] = registers per lane,
 * out[2] = spill bytes per lane. Replaces occ(mode, G, cpw, sb, shm) (reference sm120/nqmoe.cu:930-937, which packs the
 * three figures into one integer; G and cpw select no separate kernel here). Needs a GPU. */
int nq_occ(int mode, int any_rows, int sb, int shm, int out[3]);

/* Validate one table row held in HOST memory [host]: level, window codes, mask-mode flags (level 2, or level 4 with a wide
 * residual plane), low-rank plane (both buffers, ranks 0..4), in_had_down (0, 128, or 512 dividing I), and that the base
 * codes are 0 or 1 (the others are not implemented). Replaces the asserts of MoELayer.set (reference
 * sm120/moe.py:243-252); an unsupported field is an error, never silently ignored. */
int nq_validate_row(const int64_t* row_host, int H, int I);

/* Dense decode of one projection (proj 0 = gate|up [2I][H], 1 = down [H][I]) of the expert whose table row is at
 * `row` (device) into fp16 `out`. level 0 = use the row's level, else override. Replaces the NQ_WDUMP debug build +
 * set_wdump (reference sm120/nqmoe.cu:246-288,852-853) and is the bit-exactness probe of the decoder. */
int nq_dequant(const int64_t* row, int proj, int level, int H, int I, void* out_f16, void* stream);

/* Dense decode of G experts (device int32 ids) at their live table level into Wgu [G][2I][H] and Wdn [G][H][I] fp16;
 * level <= 0 decodes to zeros. Replaces pf_decode (reference sm120/nqmoe.cu:1013-1080,1247-1257). */
int nq_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu_f16, void* Wdn_f16, int H, int I,
                 void* stream);

/* One decode-path MoE layer call, B <= 8 tokens, B * topk <= 64 picks (reference moe_forward, sm120/nqmoe.cu:858-907).
 * cfg = {cpw, sb, nst, 0}: k-slice = cpw * nst chunks of 128 columns per block; sb = 1, 2 or 4 wavefronts per block (each
 * wavefront decodes two 16-row strips, so sb = 4 covers the reference's largest block of 128 rows); sb must divide N / 32 (and I / 32
 * for gate|up); the 4th entry
 * (persistent mode) must be 0. Workspaces: acc_gu / acc_d hold k-slice partial sums (plain stores, no float atomics):
 * acc_gu >= (H/128/(cpw*nst)) * B*topk * 2I floats, acc_d >= (I/128/(cpw*nst)) * B*topk * H floats, h >= B*topk * I
 * halfs; cnt_gu >= B*topk * I/128 and cnt_d >= H/128 int32 arrival counters, zero on entry and zero again on exit (the
 * reference's workspace contract, sm120/nqmoe.cu:855-857). Picks with rw == 0, level <= 0 or an expert id outside
 * [0, E) contribute nothing. which: bit 0 = gate|up launch, bit 1 = down launch; bit 2 = skip the call's first launch (routing
 * and rotation of the activations) because route_ws and xrot still hold what an earlier call with the same x, sel, rw and table
 * rows left there (what a benchmark of one projection launch alone uses); bit 3 = the two launches come as two calls but with the
 * arithmetic of one: the gate|up call (which = 1 | 8) leaves h to the down call (which = 2 | 4 | 8), which forms it from the gate|up
 * partial sums exactly as a which = 3 call does (same bits). Calls that share a routing (bits 2 / 3) must agree in B, topk, x, sel,
 * rw and cfg_gu's sb; the number of gate|up k-slices is taken from what the gate|up launch recorded in route_ws. hits: optional int32[E] pick counters
 * (device or host-mapped memory), incremented once per pick with rw != 0 (reference :784-787). */
/* Element types of the caller's tensors. The casts the reference's caller launches around the call (x.half(), ids.long(),
 * w.half(), out.to(x.dtype): sm120/serve/nq_vllm.py:522,560,573; fusing them is the open item of
 * threads/13-moe-layer-kernel/INTEGRATION.md:191-192) happen inside the kernels with the same roundings: x and rw pass
 * through fp16, the fp32 result is rounded once to the output type. */
enum { NQ_DT_F16 = 0, NQ_DT_BF16 = 1, NQ_DT_F32 = 2, NQ_DT_I64 = 0, NQ_DT_I32 = 1, NQ_DT_OUT_F32 = 0, NQ_DT_OUT_F16 = 1, NQ_DT_OUT_BF16 = 2 };

typedef struct NqMoeArgs
{
    const void* x;            /* [B][H], x_dtype */
    const void* sel;          /* [B][topk], sel_dtype */
    const void* rw;           /* [B][topk], rw_dtype */
    const int64_t* table;     /* int64 [E][NQ_TBL_W] */
    void* out;                /* [B][H], out_dtype */
    void* acc_gu;             /* fp32 workspace */
    void* h;                  /* fp16 [B*topk, I]: rotated SwiGLU output of every pick, input of the down launch. Written by the
                                 gate|up launch (which = 1, and runs whose row has a low-rank plane or in_had_down = 512) or,
                                 when both launches belong to the call (which = 3), by the down launch, which then forms it from
                                 the gate|up partial sums itself; same bits either way */
    void* acc_d;              /* fp32 workspace */
    int32_t* cnt_gu;          /* int32 workspace, zero on entry */
    int32_t* cnt_d;           /* int32 workspace, zero on entry */
    int32_t* hits;            /* optional, may be NULL */
    int64_t acc_gu_elems, acc_d_elems, h_elems, out_elems, cnt_gu_elems, cnt_d_elems;   /* capacities, checked */
    int32_t B, topk, E, H, I;
    int32_t cfg_gu[4], cfg_dn[4];
    int32_t force_level;      /* 0, or a level that overrides every active row's level (debug) */
    int32_t which;
    int32_t x_dtype;          /* NQ_DT_F16 (0), NQ_DT_BF16, NQ_DT_F32: element type of x */
    int32_t sel_dtype;        /* NQ_DT_I64 (0) or NQ_DT_I32 */
    int32_t rw_dtype;         /* NQ_DT_F16 (0), NQ_DT_BF16, NQ_DT_F32 */
    int32_t out_dtype;        /* NQ_DT_OUT_F32 (0), NQ_DT_OUT_F16, NQ_DT_OUT_BF16: element type of out */
    int32_t* cnt_h;           /* int32 [B*topk * I/128], zero on entry and on exit: arrival counters of the 512-column blocks
                                 of experts with in_had_down = 512 (reference cnt_h, sm120/nqmoe.cu:860) */
    int64_t cnt_h_elems;
    void* zd;                 /* fp32 [B*topk * I/128 * 4]: low-rank plane, z_d partials written by the gate|up launch and read by the
                                 down launch (reference zd, sm120/nqmoe.cu:860); needs no zeroing */
    int64_t zd_elems;
    int32_t common_rows;      /* 0 (the default): nothing is known about the rows, correct for every table. 1: the host vouches that
                                 every row that can be picked is of the common kind -- base window code 0 (table word 19) and no
                                 mask-mode flags (words 4 / 8) -- which selects a kernel without the other kinds' decode loops,
                                 a few percent faster; should a row of another kind be picked under it, its planes are not
                                 read and the tokens that picked it come out NaN. */
    int32_t G;                /* lanes per ring (reference moe_forward's G, sm120/nqmoe.cu:223-228,862): 0 or 4 = rings of four
                                 records (the format every artifact uses), 2 = the same planes read as rings of two records
                                 (the reference's test variant; not with sign-variant planes, not in prefill) */
    void* route_ws;           /* NQ_ROUTE_WS_BYTES of device memory, 64-byte aligned, contents irrelevant on entry: the call's first
                                 launch does the routing once (every workgroup for itself, one of them writes the result) -- picks -> runs of distinct experts with their table
                                 rows (reference route(), sm120/nqmoe.cu:379-449, which every block of the reference repeats) -- and
                                 leaves it here for the two projection launches */
    int64_t route_ws_bytes;
    void* xrot;               /* fp16 [B*topk][2][H], 16-byte aligned, contents irrelevant on entry: the first launch also rotates the
                                 activations of every active pick, once (x * su_g and x * su_u -> Hadamard-128 -> fp16; reference
                                 sm120/nqmoe.cu:506-519, which every block repeats for its k-slice), for the gate|up launch */
    int64_t xrot_elems;
    int64_t* mb_table;        /* optional mailbox of the call, without a launch of its own (the reference's caller launches nq_mailbox
                                 at the top of every layer step, sm120/serve/nq_vllm.py:546). Two halves, one observer each:
                                 (1) one extra workgroup of the call's LAST projection launch does table[e] <- stage[e] and
                                 mb_applied[e] <- mb_seq[e] for every e whose seq differs -- after this call's routing has read the
                                 table, so this call works from the rows as they were when it started and the next call from the
                                 new ones; (2) the routing launch of the NEXT call with this mailbox (or the next nq_mailbox) copies
                                 mb_applied to mb_applied_host. A row whose seq lands while call n runs is thus used and published
                                 from call n + 1 on, as with nq_mailbox at the top of call n + 1; applied_host[e] == seq[e] still
                                 means that no launch enqueued from then on reads the slot the replaced row named (reference
                                 threads/13-moe-layer-kernel/INTEGRATION.md:226-227). The last published state lags the table by one
                                 call: a caller that stops calling and wants it published launches nq_mailbox once.
                                 NULL = no mailbox in this call; otherwise == table */
    const int64_t* mb_stage;
    const int32_t* mb_seq;
    int32_t* mb_applied;
    int32_t* mb_applied_host; /* [host-mapped], may be NULL */
    int32_t hoist_value_map;  /* 0 (the default): every decoded weight is rounded to fp16 before it is multiplied, as the reference's kernel
                                 and its dense decoder do; results are within 5e-5 of the float64 layer over the exact fp16 weights.
                                 1: runs whose row has no sign plane and is of the common kind (common_rows = 1) multiply the integers
                                 1024 + S (level 2) or 1024 + F (levels 3, 4) and apply the value map to the sums -- once per k-slice
                                 at level 2, where A and B are global, per unit at levels 3 / 4 (the reference's "RM_P RAW" affine
                                 hoisting, threads/15-level4-decode/REPORT.md:40,42,66): one vector instruction fewer per weight pair,
                                 the weights are NOT rounded to fp16, and the layer output moves 4.6e-4 (relative l2, mean; 6.3e-4 at
                                 most over 64 routings of the full shape) from the exact form's -- inside the layer's 1e-3 tolerance,
                                 with little room to spare. nq_dequant is never affected. */
    int32_t reserved_;
} NqMoeArgs;
#define NQ_ROUTE_WS_BYTES 32768
int nq_moe_forward(const NqMoeArgs* args, void* stream);

/* nq_moe_forward for callers that cannot allocate device memory or keep workspaces of their own (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference, whose MoELayer
 * always owns its workspaces (sm120/moe.py:231-241). Same arguments, kernels and results as nq_moe_forward, except that the
 * workspace fields of *args (acc_gu, h, acc_d, cnt_gu, cnt_d, cnt_h, zd, route_ws, xrot and their capacities) are not looked at:
 * partial sums, h, z_d, the routing result and the arrival counters live in one array of NQ_STATIC_SCRATCH_BYTES that is part of the library's device
 * image (every GPU the library runs on holds its own copy until the process ends). The call allocates and frees nothing; it
 * clears the counters with a small kernel, then makes the two launches. A call whose shape and k-slices need more than the
 * array holds is refused with an error (full shape H=6144, I=2048, B*topk=64 picks with the default k-slices: about 8.9 MiB; with down k-slices of 4 chunks, as tuned for this shape: 9.8 MiB).
 * All calls on one GPU share the array: calls that overlap on one GPU (different streams) race; order them on one stream.
 * The first call on a device looks up the array's address (hipGetSymbolAddress) and so must not be made under stream
 * capture; later calls may be. */
#define NQ_STATIC_SCRATCH_BYTES (16u << 20)
int nq_moe_forward_static(const NqMoeArgs* args, void* stream);

/* table[e] <- stage[e] for every e with seq[e] != applied[e]; then applied[e] <- seq[e]; applied_host [host-mapped, optional]
 * receives every entry of applied (also those an earlier layer call's mailbox block applied without publishing them).
 * Replaces mailbox (reference sm120/nqmoe.cu:908-929). */
int nq_mailbox(int64_t* table, const int64_t* stage, const int32_t* seq, int32_t* applied, int32_t* applied_host, int E,
               void* stream);

/* Decode salience export: acc[e] += sum over the picks (t, k) with ids[t][k] == e of (rsf * w[t][k])^2 * sum_i x[t][i]^2, for
 * T <= 8 tokens of K <= 8 picks; acc fp64 [E] on the device, every touched entry also stored to host [host-mapped fp64 [E]].
 * x [T][H] with row stride x_row_stride elements, NQ_DT_F16 / NQ_DT_BF16 (or NQ_DT_F32, rounded through fp16); w [T][K]
 * likewise (rounded through fp16); ids NQ_DT_I64 / NQ_DT_I32. Picks with w == 0 or an id outside [0, E) are skipped. The
 * squared norm is an fp32 sum in this kernel's own order (one wavefront per token), the per-pick terms and the running sums
 * are fp64: values agree with the reference's to fp32 rounding of the norm, not bit for bit. Calls on one layer must be
 * stream-ordered (acc is updated without atomics). Replaces sal (reference sm120/nqsal.cu:19-78, called at
 * sm120/serve/nq_vllm.py:558,572). */
int nq_sal(const void* x, int x_dtype, int64_t x_row_stride, const void* w, int w_dtype, const void* ids, int ids_dtype, int T,
           int H, int K, int E, double rsf, double* acc, double* host, void* stream);

/* ---- prefill (more tokens than a decode call takes): pairs (token, expert) sorted by expert ------------------------------
 * pt / pe: int32[np] token and expert of each pair. Pairs whose expert is at level <= 0,
 * outside [0, E), or whose weight is 0 contribute nothing. Activation buffers xg, xu [np][H] and h [np][I] are fp16 with
 * every 128-column chunk stored in the MFMA B-operand column order (an internal layout shared by these entry points). */

/* xg / xu = fp16(Hadamard-128(x[pt] * su_g / su_u)); zg fp32 [np][4] (may be NULL when no expert has a low-rank plane):
 * zg[p] = x[pt[p]] V_gu^T of pair p's expert. Replaces pf_pre (reference sm120/nqmoe.cu:1082-1117,1258-1267). */
int nq_pf_pre(const void* x_f16, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg_f16,
              void* xu_f16, float* zg, int E, int H, int I, void* stream);

/* nq_pf_pre for the pair rows of some tile heights only: tiles / cap are the lists nq_pf_plan wrote for the same rows,
 * heights a bit mask (bit k = height 16 << k); a row is worked on when the tile that holds it has one of these heights, the
 * other rows of xg, xu and zg are left alone. With this and nq_pf_mid_rows the kernels of one tile height (pre, gate|up
 * GEMM, mid, down GEMM) form a chain of their own, so the heights can run on concurrent streams between nq_pf_plan and
 * nq_pf_post. The reference's pf_pre has no such restriction (its grouped GEMMs run one after the other,
 * sm120/moe.py:303-324). */
int nq_pf_pre_rows(const void* x_f16, const int32_t* pt, const int32_t* pe, int np, const int64_t* table, void* xg_f16,
                   void* xu_f16, float* zg, int E, int H, int I, const int32_t* tiles, int cap, int heights, void* stream);

/* Grouped GEMM with the weights decoded from the trellis planes inside the kernel (level and planes from the live table
 * row): for every tile t = tiles[t] = {expert, first pair row, rows, 0} (device int32[ntiles][4], rows <= bm,
 * bm in {16, 32, 64, 128, 256}):  C[row][n] = sum_k A[row][k] * W_expert[n][k]  with fp32 accumulation and output.
 * mode 0: gate|up, K = H, N = 2I, A0 = xg feeds weight rows [0, I), A1 = xu feeds rows [I, 2I), C = [np][2I];
 * mode 1: down, K = I, N = H, A0 = h, A1 ignored, C = [np][H]. mode | 2: the variant for experts in mask mode (flags word of
 * the table row set): it handles only their tiles, the plain variant only the others, so a layer with such experts makes
 * both calls; mode | 4: this is the only call for these tiles (the host knows every row to be of one kind), so a tile of the
 * other kind, which nothing would compute, gets NaN results instead of stale scratch. Replaces pf_decode + the Triton grouped GEMM / aten.mm
 * (reference sm120/pf_gemm.py:7-34, sm120/moe.py:303-324); decoded weights never touch HBM. */
int nq_pf_gemm(const int64_t* table, const int32_t* tiles, int ntiles, int bm, int mode, const void* A0_f16,
               const void* A1_f16, float* C, int E, int H, int I, const void* Wop, void* stream);

/* Decode the experts that nq_pf_plan marked hot (hot[e] = their slot, -1 = none; device int32 [E]) once per call: projection
 * `mode` (0 gate|up, 1 down) of each into slot hot[e] of the scratch Wop (slots x 3 * H * I fp16, 16-byte aligned), in the
 * order in which nq_pf_gemm holds weights in registers, so that every tile of such an expert (fourth word of the tile = slot + 1)
 * loads its operands instead of decoding the expert again. Experts at level <= 0, in mask mode or with a base code other than 0
 * are left out (their tiles decode in the GEMM as before). Pass the same Wop to nq_pf_gemm; NULL there = every tile decodes.
 * The reference decodes every expert of a group once too, but into dense [2I][H] / [H][I] matrices for a library GEMM
 * (pf_decode, sm120/nqmoe.cu:1013-1080,1247-1257; sm120/moe.py:303-324). */
int nq_pf_wdecode(const int64_t* table, const int32_t* hot, int E, int mode, void* Wop, int64_t wop_bytes, int slots, int H, int I,
                  void* stream);

/* h = fp16(Hadamard(silu(g) * u * su_d)), g = Hadamard(acc_gu[:, :I]) * sv_g, u = Hadamard(acc_gu[:, I:]) * sv_u; the last
 * Hadamard is 128 or 512 wide (table word 18). Low-rank plane: g / u += zg (U2 [+ U4 at level 4]) and zd[p] = (silu(g) * u)
 * V_dn^T, fp32 [np][4] (zg, zd may be NULL). Replaces pf_mid (reference sm120/nqmoe.cu:1119-1203,1268-1277). */
int nq_pf_mid(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h_f16, const float* zg, float* zd,
              int E, int H, int I, void* stream);

/* nq_pf_mid for the pair rows of some tile heights only (tiles, cap, heights as in nq_pf_pre_rows); the other rows of h and
 * zd are left alone. The reference's pf_mid has no such restriction. */
int nq_pf_mid_rows(const float* acc_gu, const int32_t* pe, int np, const int64_t* table, void* h_f16, const float* zg, float* zd,
                   int E, int H, int I, const int32_t* tiles, int cap, int heights, void* stream);

/* For every token t < T: out[t] += sum over its picks k whose pair row pos[t][k] lies in [row_lo, row_lo + nrows) of
 * rw[t][k] * sv_o (.) Hadamard(y[pos[t][k] - row_lo]). pos int32 [T][topk] = row of pair (t, k) in the expert-sorted
 * order; sel int64 [T][topk]; rw fp16 [T][topk]; y fp32 [nrows][H]; out fp32 [T][H], zeroed by the caller before the
 * first row chunk; zd fp32 [nrows][4] from nq_pf_mid adds the low-rank term zd (U2_d [+ U4_d]) per pick (may be NULL).
 * Gathered per token: no atomics, fixed summation order. Replaces pf_post (reference sm120/nqmoe.cu:1205-1240,1278-1287,
 * which adds with float atomics). */
int nq_pf_post(const float* y, const int32_t* pos, const int64_t* sel, const void* rw_f16, int T, int topk, int row_lo,
               int nrows, const int64_t* table, float* out, const float* zd, int E, int H, int I, void* stream);

/* Tile lists of one chunk of pair rows, built on the device. counts int32 [E] = pairs per expert over the whole call (pairs
 * sorted by expert); the chunk holds the pair rows [row_lo, row_lo + nrows). tiles: int32 [5][cap][4], list k for tile height
 * 16 << k, cap >= E + nrows / 256 + 1. An expert's rows inside the chunk are cut into 256-row tiles (indices E.. of list 4);
 * the remainder goes to index e of the list of the smallest height that holds it; every other entry gets expert -1, which
 * nq_pf_gemm skips. Launch nq_pf_gemm on list k with ntiles = E (k < 4) or cap (k = 4). hot (device int32 [E], may be NULL):
 * experts with at least hot_min rows in the chunk get a slot 0 .. hot_cap - 1 of the decoded-weight scratch, in expert order as
 * far as the slots reach: hot[e] = slot or -1, and the fourth word of each of their tiles = slot + 1 (0 otherwise); see
 * nq_pf_wdecode. Replaces the host loop over the
 * expert counts of the reference's prefill (sm120/moe.py:296-302) and the host synchronisation that feeds it. */
int nq_pf_plan(const int32_t* counts, int E, int row_lo, int nrows, int32_t* tiles, int cap, int32_t* hot, int hot_min, int hot_cap,
               void* stream);

/* hits[e] += counts[e] (hits may be host-mapped). Replaces pf_hits (reference sm120/nqmoe.cu:1241-1245,1288-1293). */
int nq_pf_hits(const int32_t* counts, int32_t* hits, int E, void* stream);

/* ---- Refinement-record upgrade engine (host threads + one side stream; replaces the class Engine of the reference's
 * streaming/nqstream.cu:51-277 and its Python surface, :8-26). One engine per record file (one rank) and GPU. Unlike the
 * entry points above, an engine owns memory for its lifetime: n_host pinned host entries of rec_bytes each (bounce
 * buffers of the reads and a least-recently-used cache of records), pinned staging of rows and sequence numbers, an
 * optional pinned RAM tier, one non-blocking stream of default priority, qd (+ qd_alt) reader threads and one director
 * thread. It launches no kernel: its device work is hipMemcpyAsync host -> device. ---- */
typedef struct NqStream NqStream;

/* one finished op, as the tuples of the reference's Engine.poll() (streaming/nqstream.cu:110-113): hit = the record came
 * from the host cache or the RAM tier; a failed read has t_read < 0 (the negated errno, or -1 for a short read) and
 * t_e2e = -1 and has written neither row nor seq; a cancelled op has cancelled = 1 and both times = -1e9 */
typedef struct NqStreamDone { int64_t tag; int32_t hit; int32_t cancelled; double t_read; double t_e2e; } NqStreamDone;

/* counters of Engine.stats() (streaming/nqstream.cu:114-128); drive_direct = the file was opened with O_DIRECT (0 = the
 * file system refused it and reads are buffered); failed = a HIP call of the engine failed (nq_last_error has its text) */
typedef struct NqStreamStats
{
    int64_t upgrades, posts, host_hits, bytes_read, fault_injected, queued, reading, copying;
    int64_t drives, n_host, drive_qd[2], drive_inflight[2], drive_reads[2], drive_bytes[2], drive_direct[2];
    double drive_read_s[2];
    int64_t tier_state, tier_recs, tier_hits, tier_bytes, cancelled, waiting, failed;
    double now;
    int64_t uploads, upload_bytes;
} NqStreamStats;

/* Open the record file `path` [host] (records of rec_bytes each, rec_bytes % 4096 == 0) for device `device`; alt_path
 * (NULL or "" = none) is an identical copy on a second drive with its own queue depth qd_alt (0 = qd): each read goes to
 * the drive with fewer reads in flight. n_host >= qd + qd_alt. The environment variables NQ_FAULT_READ_MS and
 * NQ_FAULT_FAIL_PPM set the fault injection of nq_stream_set_fault at open. NULL on failure (nq_last_error).
 * Reference: Engine(path, rec_bytes, n_host, qd, device, alt_path, qd_alt), streaming/nqstream.cu:72-93. */
NqStream* nq_stream_open(const char* path, const char* alt_path, int64_t rec_bytes, int n_host, int qd, int qd_alt, int device);

/* Queue an upgrade and return: record `rec` of the file -> device address slot (rec_bytes), then row_host [host]
 * int64[NQ_TBL_W] -> stage_row (device), then seq -> seq_ptr (device int32), in this order on the engine's stream.
 * Reference: Engine.upgrade, streaming/nqstream.cu:97-100. */
int nq_stream_upgrade(NqStream* s, int64_t tag, int64_t rec, void* slot, void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq);

/* Queue a row-only op (a downgrade): row, then seq. Reference: Engine.post, streaming/nqstream.cu:101-104. */
int nq_stream_post(NqStream* s, int64_t tag, void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq);

/* Queue an upload from the caller's pinned host memory and return: nspans (1..NQ_STREAM_MAX_SPANS) copies src_host[i] ->
 * dst[i] (device) of nbytes[i], then the row, then seq, in this order on the engine's stream. The source must stay valid
 * and unchanged until nq_stream_poll reports the op. This is the promotion of a resident-in-RAM expert (several spans: the
 * planes a nested level adds); an engine opened with path NULL or "" serves only uploads and row-only ops and owns no
 * host entries. The reference has no such call: its serving engine reads every record from the file or its RAM tier
 * (streaming/nqstream.cu:183-191); its level-switch script copies from pinned tensors with torch
 * (sm120/levelswitch_mbox.py:33-65), which this replaces. */
#define NQ_STREAM_MAX_SPANS 8
int nq_stream_upload(NqStream* s, int64_t tag, int nspans, const void* const* src_host, void* const* dst, const int64_t* nbytes,
                     void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq);

/* Best effort: an op that has started neither a read nor a device write is dropped and reported by nq_stream_poll as
 * cancelled; one that has started completes normally. Reference: Engine.cancel, streaming/nqstream.cu:95,200-210. */
int nq_stream_cancel(NqStream* s, int64_t tag);

/* Move up to max finished ops into out [host]; returns their number. The device writes of a reported op are complete, so
 * the next nq_mailbox may apply its row. Reference: Engine.poll, streaming/nqstream.cu:110-113. */
int nq_stream_poll(NqStream* s, NqStreamDone* out, int max);

/* Pinned RAM tier: read the n records recs [host] once, in the caller's thread, into one pinned buffer; an upgrade of
 * one of them then skips the drive. Returns n, or -1. nq_stream_tier_drop releases the tier once no copy reads from it.
 * Reference: Engine.tier_load / tier_drop, streaming/nqstream.cu:130-155,218-220. */
int64_t nq_stream_tier_load(NqStream* s, const int64_t* recs, int64_t n);
int nq_stream_tier_drop(NqStream* s);

/* Fault injection for tests of the failure paths: read_ms = minimum spacing between the starts of drive reads (a slow
 * drive), fail_ppm = share of completed reads reported as failed (a failing drive). Reference: the environment
 * variables NQ_FAULT_READ_MS / NQ_FAULT_FAIL_PPM read by the constructor, streaming/nqstream.cu:68-70,92-93,264-269. */
int nq_stream_set_fault(NqStream* s, double read_ms, int64_t fail_ppm);

int nq_stream_stats(NqStream* s, NqStreamStats* out);

/* Stop the threads, wait for the stream, free everything; ops not yet finished are dropped without a report.
 * Reference: Engine.close, streaming/nqstream.cu:83-93. */
void nq_stream_close(NqStream* s);

#ifdef __cplusplus
}
#endif
#endif
