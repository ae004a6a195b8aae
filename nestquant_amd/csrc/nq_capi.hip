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
}  // namespace nq

using namespace nq;

extern "C" int nq_abi_version(void) { return NQ_ABI_VERSION; }
extern "C" const char* nq_last_error(void) { return error_buffer(); }

extern "C" int nq_codes(uint32_t out[4])
{
    NQ_REQUIRE(out, "nq_codes: null output");
    out[0] = out[1] = (1u << NCODES) - 1u;   // residual codes 0..11 in both kernels
    out[2] = out[3] = 1u;                     // base code 0 (K = 2 ring base) only
    return 0;
}

extern "C" int nq_validate_row(const int64_t* r, int H, int I)
{
    NQ_REQUIRE(r, "nq_validate_row: null row");
    NQ_REQUIRE(shape_ok(H, I), "nq_validate_row: H=%d I=%d must be positive multiples of 128", H, I);
    const int64_t lv = r[0];
    NQ_REQUIRE(lv == 0 || lv == 2 || lv == 3 || lv == 4, "table row: level %lld not in {0,2,3,4}", (long long)lv);
    if (lv == 0) return 0;
    NQ_REQUIRE(r[1] && r[5] && r[9], "table row: null base plane or sign vector");
    NQ_REQUIRE(r[4] == 0 && r[8] == 0, "table row: mask mode (flags) is not implemented");
    NQ_REQUIRE(r[14] == 0 && r[15] == 0 && r[16] == 0 && r[17] == 0, "table row: low-rank plane is not implemented");
    NQ_REQUIRE(r[18] == 0 || r[18] == 128, "table row: in_had_down %lld is not implemented (128 only)", (long long)r[18]);
    NQ_REQUIRE(r[19] == 0, "table row: base code %lld is not implemented (K=2 ring base only)", (long long)r[19]);
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
