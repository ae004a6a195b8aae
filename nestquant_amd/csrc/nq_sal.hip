// Decode salience export: sal[e] += sum over the picks (t, k) of expert e of (rsf * w[t][k])^2 * |x[t]|^2, a running fp64 sum per
// expert on the device, every touched entry mirrored to host-mapped memory (what the level scheduler's predictor reads next to
// the routing hit counters; reference sm120/nqsal.cu:19-78, called at sm120/serve/nq_vllm.py:558,572). At most 8 tokens of 8
// picks per call, no host synchronisation, static pointers, so the call can sit in a captured decode step.
//
// Built for 64-wide wavefronts: one workgroup of eight wavefronts, wavefront t owns token t. Its lanes walk the row in 16-byte
// steps (eight fp16 / bf16 values, or four fp32 values rounded through fp16) with two independent fp32 accumulators, the 64
// lane sums meet in a butterfly of lane exchanges, and nothing but the eight norms crosses wavefronts (through LDS). The picks
// are then the lanes of wavefront 0: a ballot loop groups the picks of one expert, their fp64 terms are added in pick order
// and the group's first lane updates the accumulator once (calls on one layer are stream-ordered, so no atomics). The squared
// norm is an fp32 sum (about 1e-6 relative at H = 6144); weights pass through fp16 as the caller's cast would leave them.
#include "nq_host.hpp"

namespace nq {

struct SalArgs
{
    const void* x; int64_t sx; const void* w; const void* ids;
    int T, H, K, E; int x_dtype, w_dtype, ids_dtype;       // x / w: 0 f16, 1 bf16, 2 f32 (rounded through fp16); ids: 0 i64, 1 i32
    float rsf; double* acc; double* host;
};

__device__ __forceinline__ float sal_bf16(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
__device__ __forceinline__ float sal_elem(const void* p, int64_t i, int dt)
{
    if (dt == 0) return (float)((const _Float16*)p)[i];
    if (dt == 1) return sal_bf16(((const uint16_t*)p)[i]);
    return (float)(_Float16)((const float*)p)[i];
}
// squares of the two 16-bit values of a word, added to s
__device__ __forceinline__ float sal_sq2(uint32_t u, int dt, float s)
{
    const float lo = dt == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)u) : sal_bf16(u & 0xFFFFu);
    const float hi = dt == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16)) : sal_bf16(u >> 16);
    return __builtin_fmaf(hi, hi, __builtin_fmaf(lo, lo, s));
}

__global__ void __launch_bounds__(512) nq_sal_k(SalArgs a)
{
    __shared__ float norm2[8];
    const int lane = threadIdx.x & 63, t = threadIdx.x >> 6;
    if (t < a.T)
    {
        const int esz = a.x_dtype == 2 ? 4 : 2;
        const char* row = (const char*)a.x + (int64_t)t * a.sx * esz;
        const int per = 16 / esz;                                  // values per 16-byte step
        float s0 = 0.f, s1 = 0.f;
        int done = 0;
        if (((uintptr_t)row & 15) == 0)
        {
            const int nv = a.H / per;
            for (int i = lane; i < nv; i += 128)
            {
                const uint4 u = ((const uint4*)row)[i];
                const bool two = i + 64 < nv;
                const uint4 v = two ? ((const uint4*)row)[i + 64] : uint4{0u, 0u, 0u, 0u};       // zero bits are 0.0 in all three types
                if (a.x_dtype == 2)
                {
                    const float f[8] = {__builtin_bit_cast(float, u.x), __builtin_bit_cast(float, u.y), __builtin_bit_cast(float, u.z), __builtin_bit_cast(float, u.w),
                                        __builtin_bit_cast(float, v.x), __builtin_bit_cast(float, v.y), __builtin_bit_cast(float, v.z), __builtin_bit_cast(float, v.w)};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        const float p = (float)(_Float16)f[j], q = (float)(_Float16)f[4 + j];
                        s0 = __builtin_fmaf(p, p, s0); s1 = __builtin_fmaf(q, q, s1);
                    }
                }
                else
                {
                    s0 = sal_sq2(u.x, a.x_dtype, s0); s0 = sal_sq2(u.y, a.x_dtype, s0); s0 = sal_sq2(u.z, a.x_dtype, s0); s0 = sal_sq2(u.w, a.x_dtype, s0);
                    s1 = sal_sq2(v.x, a.x_dtype, s1); s1 = sal_sq2(v.y, a.x_dtype, s1); s1 = sal_sq2(v.z, a.x_dtype, s1); s1 = sal_sq2(v.w, a.x_dtype, s1);
                }
            }
            done = nv * per;
        }
        for (int i = done + lane; i < a.H; i += 64) { const float f = sal_elem(row, i, a.x_dtype); s0 = __builtin_fmaf(f, f, s0); }   // rest, or a row off 16-byte alignment
        float s = s0 + s1;
#pragma unroll
        for (int m = 32; m; m >>= 1) s += __shfl_xor(s, m);
        if (lane == 0) norm2[t] = s;
    }
    __syncthreads();
    if (t != 0) return;
    const int n = a.T * a.K;                                        // <= 64: one pick per lane
    long long e = -1; double term = 0.0;
    if (lane < n)
    {
        const float wf = (float)(_Float16)sal_elem(a.w, lane, a.w_dtype);
        e = a.ids_dtype == 0 ? (long long)((const int64_t*)a.ids)[lane] : (long long)((const int32_t*)a.ids)[lane];
        if (wf == 0.f || e < 0 || e >= a.E) e = -1;                 // weight 0 or an id outside the table: skipped, as the hit counters do
        const double ww = (double)(wf * a.rsf);
        term = ww * ww * (double)norm2[lane / a.K];
    }
    unsigned long long rem = __ballot(e >= 0);
    while (rem)
    {
        const int first = __ffsll((long long)rem) - 1;
        const long long ev = __shfl(e, first);
        const unsigned long long same = __ballot(e == ev);
        double tot = 0.0;
        for (unsigned long long m = same; m; m &= m - 1) tot += __shfl(term, __ffsll((long long)m) - 1);     // in pick order
        if (lane == first) { const double v = a.acc[ev] + tot; a.acc[ev] = v; a.host[ev] = v; }
        rem &= ~same;
    }
}

int launch_sal(const void* x, int x_dtype, int64_t sx, const void* w, int w_dtype, const void* ids, int ids_dtype, int T, int H, int K,
               int E, float rsf, double* acc, double* host, hipStream_t st)
{
    SalArgs a{x, sx, w, ids, T, H, K, E, x_dtype, w_dtype, ids_dtype, rsf, acc, host};
    nq_sal_k<<<1, 512, 0, st>>>(a);
    NQ_LAUNCH_CHECK("nq_sal");
    return 0;
}

}  // namespace nq
