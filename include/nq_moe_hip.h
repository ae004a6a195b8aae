/* libnq_moe_hip.so -- C ABI of the MI355X (gfx950) NestQuant routed-expert MoE hot path.
 *
 * Every pointer is a raw device address unless marked [host] or [host-mapped]; the library allocates nothing per call
 * and keeps no pointer after a call returns. All launches go to the stream passed in (a hipStream_t as void*, 0 = the
 * null stream). Entry points return 0 on success; otherwise non-zero and nq_last_error() describes the failure (the
 * reference raises TORCH_CHECK -> RuntimeError at the same points, sm120/nqmoe.cu:871-878,887,897).
 *
 * Table row = int64[NQ_TBL_W] per expert (reference sm120/moe.py:216-229, sm120/nqmoe.cu:26-45):
 *   [0] level 0/2/3/4   [1..4] gate|up: base, residual plane, block words, flags(must be 0)   [5..8] down: same
 *   [9] fp16 sign/scale vector [H su_g | I sv_g | I sv_u | I su_d | H sv_o | H su_u]
 *   [10],[11] residual window code of gate|up, down (0..9 as the reference; 10 = nested K=1 plane P3; 11 = nested
 *   P3 || P4: uint2 sub-array of P3 followed by uint2 sub-array of P4)   [12],[13] sign-variant planes (0 = none)
 *   [14..17] low-rank plane (must be 0)   [18] in_had_down (must be 0 or 128)   [19] base codes (must be 0)
 */
#ifndef NQ_MOE_HIP_H
#define NQ_MOE_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define NQ_TBL_W 20
#define NQ_ABI_VERSION 1

/* library identification; no counterpart in the reference (its module is rebuilt per process by sm120/build.py:7-12) */
int nq_abi_version(void);
/* text of the calling thread's last failure (reference: the RuntimeError message of TORCH_CHECK) */
const char* nq_last_error(void);

/* Bit masks of the residual window codes compiled into {gate|up, down} of the decode kernels and the base codes
 * {gate|up, down}; replaces rk_codes() / bk_codes() (reference sm120/nqmoe.cu:938-940, sm120/moe.py:246-252). */
int nq_codes(uint32_t out[4]);

/* Validate one table row held in HOST memory [host]: level, window codes, and that every field this library does not
 * implement (flags, low-rank plane, in_had_down > 128, base codes) is zero. Replaces the asserts of MoELayer.set
 * (reference sm120/moe.py:243-252); an unsupported field is an error, never silently ignored. */
int nq_validate_row(const int64_t* row_host, int H, int I);

/* Dense decode of one projection (proj 0 = gate|up [2I][H], 1 = down [H][I]) of the expert whose table row is at
 * `row` (device) into fp16 `out`. level 0 = use the row's level, else override. Replaces the NQ_WDUMP debug build +
 * set_wdump (reference sm120/nqmoe.cu:246-288,852-853) and is the bit-exactness probe of the decoder. */
int nq_dequant(const int64_t* row, int proj, int level, int H, int I, void* out_f16, void* stream);

/* Dense decode of G experts (device int32 ids) at their live table level into Wgu [G][2I][H] and Wdn [G][H][I] fp16;
 * level <= 0 decodes to zeros. Replaces pf_decode (reference sm120/nqmoe.cu:1013-1080,1247-1257). */
int nq_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu_f16, void* Wdn_f16, int H, int I,
                 void* stream);

#ifdef __cplusplus
}
#endif
#endif
