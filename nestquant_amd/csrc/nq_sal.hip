// Decode salience export: sal[e] += sum over the picks (t, k) of expert e of (rsf * w[t][k])^2 * |x[t]|^2, a running fp64 sum per
// expert on the device, every touched entry mirrored to host-mapped memory (what the level scheduler's predictor reads next to
// the routing hit counters). One workgroup per call, at most 8 tokens x 8 picks, no host synchronisation, static pointers.
//
// The fp32 arithmetic follows the reference kernel's order (sm120/nqsal.cu:20-60) so that the exported numbers are the same
// bits: 256 threads, thread tid takes elements 8 i .. 8 i + 7 for i = tid, tid + 256, ... (or single elements i = tid, tid + 256,
// ... when H is not a multiple of 8 or the row is not 16-byte aligned), fused multiply-adds in that order, a butterfly over
// groups of 32 threads (offsets 16, 8, 4, 2, 1), then the eight group sums added in order. A wavefront holds two such groups;
// the butterfly offsets stay below 32, so each half reduces on its own.
#include "nq_host.hpp"

namespace nq {

struct SalArgs
{
    const void* x; int64_t sx; const void* w; const void* ids;
    int T, H, K, E; int x_dtype, w_dtype, ids_dtype;       // x / w: 0 f16, 1 bf16, 2 f32 (rounded through fp16); ids: 0 i64, 1 i32
    float rsf; double* acc; double* host;
};

__device__ __forceinline__ float bf16_bits_to_f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
__device__ __forceinline__ float elem_f(const void* p, int64_t i, int dt)
{
    if (dt == 0) return (float)((const _Float16*)p)[i];
    if (dt == 1) return bf16_bits_to_f(((const uint16_t*)p)[i]);
    return (float)(_Float16)((const float*)p)[i];
}

__global__ void __launch_bounds__(256) nq_sal_k(SalArgs a)
{
    __shared__ float red[8][8];                  // [token][group of 32 threads]
    __shared__ float xn[8];
    __shared__ int se[64];
    __shared__ double sv[64];
    const int tid = threadIdx.x, sub = tid & 31, grp = tid >> 5;
    const int esz = a.x_dtype == 2 ? 4 : 2;
    for (int t = 0; t < a.T; ++t)
    {
        const char* row = (const char*)a.x + (int64_t)t * a.sx * esz;
        float s = 0.f;
        // an fp32 row stands for the contiguous fp16 copy a caller would make of it, which is always aligned
        const bool by8 = (a.H & 7) == 0 && (a.x_dtype == 2 || ((uintptr_t)row & 15) == 0);
        if (by8 && a.x_dtype != 2)
        {
            for (int i = tid; i < a.H / 8; i += 256)
            {
                const uint4 u = ((const uint4*)row)[i];
                const uint32_t q[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 8; ++j)
                {
                    const uint16_t b = (uint16_t)(q[j >> 1] >> (16 * (j & 1)));
                    const float f = a.x_dtype == 0 ? (float)__builtin_bit_cast(_Float16, b) : bf16_bits_to_f(b);
                    s = __builtin_fmaf(f, f, s);
                }
            }
        }
        else if (by8)
        {
            for (int i = tid; i < a.H / 8; i += 256)
#pragma unroll
                for (int j = 0; j < 8; ++j) { const float f = elem_f(row, (int64_t)i * 8 + j, 2); s = __builtin_fmaf(f, f, s); }
        }
        else
            for (int i = tid; i < a.H; i += 256) { const float f = elem_f(row, i, a.x_dtype); s = __builtin_fmaf(f, f, s); }
#pragma unroll
        for (int o = 16; o; o >>= 1) s += __shfl_xor(s, o);
        if (sub == 0) red[t][grp] = s;
    }
    __syncthreads();
    if (tid < a.T) { float s = 0.f; for (int j = 0; j < 8; ++j) s += red[tid][j]; xn[tid] = s; }
    __syncthreads();
    const int n = a.T * a.K;
    if (tid < n)
    {
        float ww = (float)(_Float16)elem_f(a.w, tid, a.w_dtype);
        const int64_t e = a.ids_dtype == 0 ? ((const int64_t*)a.ids)[tid] : (int64_t)((const int32_t*)a.ids)[tid];
        se[tid] = (ww != 0.f && e >= 0 && e < a.E) ? (int)e : -1;        // weight 0 or an id outside the table: skipped, as the hit counters do
        ww *= a.rsf;
        sv[tid] = (double)(ww * ww * xn[tid / a.K]);
    }
    __syncthreads();
    if (tid < n && se[tid] >= 0)
    {
        // the first pick of an expert adds all of that expert's picks, in pick order, and writes once
        const int e = se[tid]; double tot = 0.0; bool first = true;
        for (int j = 0; j < n; ++j)
            if (se[j] == e) { if (j < tid) { first = false; break; } tot += sv[j]; }
        if (first) { const double v = a.acc[e] + tot; a.acc[e] = v; a.host[e] = v; }
    }
}

int launch_sal(const void* x, int x_dtype, int64_t sx, const void* w, int w_dtype, const void* ids, int ids_dtype, int T, int H, int K,
               int E, float rsf, double* acc, double* host, hipStream_t st)
{
    SalArgs a{x, sx, w, ids, T, H, K, E, x_dtype, w_dtype, ids_dtype, rsf, acc, host};
    nq_sal_k<<<1, 256, 0, st>>>(a);
    NQ_LAUNCH_CHECK("nq_sal");
    return 0;
}

}  // namespace nq
