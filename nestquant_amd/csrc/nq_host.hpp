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

// kernel launchers defined next to their kernels
int launch_dequant(const int64_t* row, int proj, int level, int H, int I, void* out, hipStream_t st);
int launch_pf_decode(const int64_t* table, const int32_t* experts, int G, void* Wgu, void* Wdn, int H, int I, hipStream_t st);

}  // namespace nq
