// Issue-rate probes for gfx950 (MI355X): how fast a SIMD issues the vector instructions the trellis decoder is made of.
// A stand-alone program (no library, no inputs); `python -m nestquant_amd.build` builds it as nestquant_amd/nq_issue_probe.
// The kernels are loops of inline asm on a few registers; results are written only so that nothing is optimised away.
//   part 1  one opcode, eight independent chains, 1 / 2 / 4 wavefronts per SIMD
//   part 2  the decoder's dependent chain (funnel shift, hash, two dot products, permute, packed FMA): one chain, and four
//           chains side by side
//   part 3  the level-2 decode of four weights with the hash as 16-bit multiply-add pair and as and/shift + 32-bit multiply
//   part 4  MFMAs of one wavefront and vector instructions of another wavefront on the same SIMD
// Times are ns per wavefront instruction per SIMD (256 workgroups, one per CU).
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#define CHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define REP8(OP) OP(0) OP(1) OP(2) OP(3) OP(4) OP(5) OP(6) OP(7)
#define I0(i) "v_mov_b32_e32 %" #i ", %8\n"
#define I1(i) "v_lshrrev_b32_e32 %" #i ", 3, %" #i "\n"
#define I2(i) "v_add_u32_e32 %" #i ", %8, %" #i "\n"
#define I3(i) "v_xor_b32_e64 %" #i ", %" #i ", %8\n"
#define I4(i) "v_mul_lo_u16_e32 %" #i ", %8, %" #i "\n"
#define I5(i) "v_fma_f32 %" #i ", %" #i ", %8, %9\n"
#define I6(i) "v_mad_u32_u16 %" #i ", %" #i ", %8, 0\n"
#define I7(i) "v_pk_mad_u16 %" #i ", %" #i ", %8, %9\n"
#define I8(i) "v_dot4_u32_u8 %" #i ", %" #i ", %8, %9\n"
#define I9(i) "v_sad_u8 %" #i ", %" #i ", 0, %9\n"
#define I10(i) "v_perm_b32 %" #i ", %" #i ", %8, %9\n"
#define I11(i) "v_pk_fma_f16 %" #i ", %" #i ", %8, %9\n"
#define I12(i) "v_alignbit_b32 %" #i ", %" #i ", %8, 6\n"
#define I13(i) "v_mul_lo_u32 %" #i ", %" #i ", %8\n"
#define I14(i) "v_bfe_u32 %" #i ", %" #i ", 3, 16\n"
#define I15(i) "v_mul_u32_u24_e32 %" #i ", %8, %" #i "\n"
#define I16(i) "v_mad_u16 %" #i ", %" #i ", %8, %9\n"
template <int OP>
__global__ void one_opcode(uint32_t* out, int iters)
{
    uint32_t r0 = threadIdx.x * 2654435761u, r1 = r0 ^ 0x1234567u, r2 = r0 + 77u, r3 = r0 * 3u, r4 = r0 + 5, r5 = r0 + 6, r6 = r0 + 7, r7 = r0 + 8;
    uint32_t a = 0x00010001u + threadIdx.x, b = 0x3c003c00u + threadIdx.x;
    for (int i = 0; i < iters; ++i)
    {
#define BODY(M) asm volatile(REP8(M) REP8(M) REP8(M) REP8(M) : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7) : "v"(a), "v"(b));
#define CASE(n) else if constexpr (OP == n) BODY(I##n)
        if constexpr (OP == 0) BODY(I0) CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(9) CASE(10) CASE(11) CASE(12) CASE(13) CASE(14) CASE(15) CASE(16)
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = r0 ^ r1 ^ r2 ^ r3 ^ r4 ^ r5 ^ r6 ^ r7;
}

// the decoder's chain on register r with temporaries t, u (7 vector instructions)
#define STEP(r, t, u) \
    "v_alignbit_b32 " t ", " r ", " r ", 6\n v_mad_u32_u16 " u ", " t ", %[klo], 0\n s_nop 0\n" \
    "v_pk_mad_u16 " t ", " t ", %[khi], " u " op_sel:[0,0,0] op_sel_hi:[0,1,1]\n s_nop 0\n" \
    "v_dot4_u32_u8 " u ", " t ", %[m], %[c]\n v_dot4_u32_u8 " u ", " t ", %[n], " u "\n s_nop 2\n" \
    "v_perm_b32 " t ", " u ", " u ", %[sel]\n v_pk_fma_f16 " r ", " t ", %[a], %[b]\n"
#define STAGE4(op, d, s, rest) op " %[" d "0], %[" s "0]" rest "\n" op " %[" d "1], %[" s "1]" rest "\n" op " %[" d "2], %[" s "2]" rest "\n" op " %[" d "3], %[" s "3]" rest "\n"
template <int ILP>
__global__ void chain(uint32_t* out, int iters)
{
    uint32_t r0 = threadIdx.x * 2654435761u, r1 = r0 ^ 0x1234567u, r2 = r0 + 77u, r3 = r0 * 3u;
    uint32_t t0, t1, t2, t3, u0, u1, u2, u3;
    const uint32_t klo = 0xD12D, khi = 0x83DC83DC, c = 0x640080, sel = 0x06050201;
    uint32_t m = 0x05050505 + threadIdx.x, n = 0x03030303, a = 0x3c003c00, b = 0x38003800;
    for (int i = 0; i < iters; ++i)
    {
        if constexpr (ILP == 1)
            asm volatile(STEP("%[r0]", "%[t0]", "%[u0]") STEP("%[r0]", "%[t0]", "%[u0]") STEP("%[r0]", "%[t0]", "%[u0]") STEP("%[r0]", "%[t0]", "%[u0]")
                         : [r0] "+v"(r0), [t0] "=&v"(t0), [u0] "=&v"(u0)
                         : [klo] "s"(klo), [khi] "s"(khi), [m] "v"(m), [n] "v"(n), [c] "s"(c), [sel] "s"(sel), [a] "v"(a), [b] "v"(b));
        else
            asm volatile(
                "v_alignbit_b32 %[t0], %[r0], %[r0], 6\n v_alignbit_b32 %[t1], %[r1], %[r1], 6\n v_alignbit_b32 %[t2], %[r2], %[r2], 6\n v_alignbit_b32 %[t3], %[r3], %[r3], 6\n"
                STAGE4("v_mad_u32_u16", "u", "t", ", %[klo], 0")
                "v_pk_mad_u16 %[t0], %[t0], %[khi], %[u0] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n v_pk_mad_u16 %[t1], %[t1], %[khi], %[u1] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n"
                "v_pk_mad_u16 %[t2], %[t2], %[khi], %[u2] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n v_pk_mad_u16 %[t3], %[t3], %[khi], %[u3] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n"
                STAGE4("v_dot4_u32_u8", "u", "t", ", %[m], %[c]")
                "v_dot4_u32_u8 %[u0], %[t0], %[n], %[u0]\n v_dot4_u32_u8 %[u1], %[t1], %[n], %[u1]\n v_dot4_u32_u8 %[u2], %[t2], %[n], %[u2]\n v_dot4_u32_u8 %[u3], %[t3], %[n], %[u3]\n"
                "v_perm_b32 %[t0], %[u0], %[u0], %[sel]\n v_perm_b32 %[t1], %[u1], %[u1], %[sel]\n v_perm_b32 %[t2], %[u2], %[u2], %[sel]\n v_perm_b32 %[t3], %[u3], %[u3], %[sel]\n"
                STAGE4("v_pk_fma_f16", "r", "t", ", %[a], %[b]")
                : [r0] "+v"(r0), [t0] "=&v"(t0), [u0] "=&v"(u0), [r1] "+v"(r1), [t1] "=&v"(t1), [u1] "=&v"(u1),
                  [r2] "+v"(r2), [t2] "=&v"(t2), [u2] "=&v"(u2), [r3] "+v"(r3), [t3] "=&v"(t3), [u3] "=&v"(u3)
                : [klo] "s"(klo), [khi] "s"(khi), [m] "v"(m), [n] "v"(n), [c] "s"(c), [sel] "s"(sel), [a] "v"(a), [b] "v"(b));
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = r0 ^ r1 ^ r2 ^ r3;
}

// level-2 decode of four weights (two register-sharing pairs); V = 0: hash as v_mad_u32_u16 + v_pk_mad_u16, V = 1: and / shift + v_mul_lo_u32
template <int V>
__global__ void decode4(uint32_t* out, int iters)
{
    uint32_t w0 = threadIdx.x * 2654435761u, w1 = w0 ^ 0x1234567u, acc = 0;
    const uint32_t klo = 0xD12D, khi = 0x83DC0000u, hc = 0x83DCD12Du, c64 = 0x64006400u;
    uint32_t A = 0x1eee1eeeu + (threadIdx.x >> 9), B = 0xc931c931u;
    uint32_t r0, r1, y0, y1, y2, y3, x0, x1, x2, x3, t0, t1, u0, u1;
#define TAIL "v_sad_u8 %[t0], %[x0], 0, %[c64]\n v_sad_u8 %[t1], %[x2], 0, %[c64]\n v_sad_hi_u8 %[t0], %[x1], 0, %[t0]\n v_sad_hi_u8 %[t1], %[x3], 0, %[t1]\n" \
             "v_pk_fma_f16 %[u0], %[t0], %[A], %[B]\n v_pk_fma_f16 %[u1], %[t1], %[A], %[B]\n v_xor_b32 %[acc], %[acc], %[u0]\n v_xor_b32 %[w0], %[w0], %[u1]\n"
#define OUTS [r0] "=&v"(r0), [r1] "=&v"(r1), [y0] "=&v"(y0), [y1] "=&v"(y1), [y2] "=&v"(y2), [y3] "=&v"(y3), [x0] "=&v"(x0), [x1] "=&v"(x1), [x2] "=&v"(x2), \
             [x3] "=&v"(x3), [t0] "=&v"(t0), [t1] "=&v"(t1), [u0] "=&v"(u0), [u1] "=&v"(u1), [acc] "+v"(acc), [w0] "+v"(w0)
    for (int i = 0; i < iters; ++i)
    {
        if constexpr (V == 0)
            asm volatile("v_alignbit_b32 %[r0], %[w1], %[w0], 6\n v_alignbit_b32 %[r1], %[w1], %[w0], 10\n"
                         "v_mad_u32_u16 %[y0], %[r0], %[klo], 0\n v_mad_u32_u16 %[y1], %[r0], %[klo], 0 op_sel:[1,0,0,0]\n"
                         "v_mad_u32_u16 %[y2], %[r1], %[klo], 0\n v_mad_u32_u16 %[y3], %[r1], %[klo], 0 op_sel:[1,0,0,0]\n"
                         "v_pk_mad_u16 %[x0], %[r0], %[khi], %[y0] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n v_pk_mad_u16 %[x1], %[r0], %[khi], %[y1] op_sel:[1,0,0] op_sel_hi:[1,1,1]\n"
                         "v_pk_mad_u16 %[x2], %[r1], %[khi], %[y2] op_sel:[0,0,0] op_sel_hi:[0,1,1]\n v_pk_mad_u16 %[x3], %[r1], %[khi], %[y3] op_sel:[1,0,0] op_sel_hi:[1,1,1]\n" TAIL
                         : OUTS : [w1] "v"(w1), [klo] "s"(klo), [khi] "s"(khi), [c64] "s"(c64), [A] "v"(A), [B] "v"(B));
        else
            asm volatile("v_alignbit_b32 %[r0], %[w1], %[w0], 6\n v_alignbit_b32 %[r1], %[w1], %[w0], 10\n"
                         "v_and_b32 %[y0], 0xffff, %[r0]\n v_lshrrev_b32 %[y1], 16, %[r0]\n v_and_b32 %[y2], 0xffff, %[r1]\n v_lshrrev_b32 %[y3], 16, %[r1]\n"
                         "v_mul_lo_u32 %[x0], %[y0], %[hc]\n v_mul_lo_u32 %[x1], %[y1], %[hc]\n v_mul_lo_u32 %[x2], %[y2], %[hc]\n v_mul_lo_u32 %[x3], %[y3], %[hc]\n" TAIL
                         : OUTS : [w1] "v"(w1), [hc] "s"(hc), [c64] "s"(c64), [A] "v"(A), [B] "v"(B));
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = acc ^ w0;
}

// mode bit 0: wavefronts 0..3 (one per SIMD) run 8 independent MFMAs per iteration; bit 1: wavefronts 4..7 run 16 vector instructions
__global__ void __launch_bounds__(512) mfma_and_valu(float* out, int iters, int mode)
{
    const int warp = threadIdx.x >> 6;
    if (warp < 4)
    {
        if (!(mode & 1)) return;
        half8_t a, b;
        for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(i * 0.5f); }
        float4_t c[8] = {};
        for (int i = 0; i < iters; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c[j], 0, 0, 0);
        for (int j = 1; j < 8; ++j) c[0] += c[j];
        out[blockIdx.x * 512 + threadIdx.x] = c[0][0] + c[0][1] + c[0][2] + c[0][3];
    }
    else
    {
        if (!(mode & 2)) return;
        uint32_t r0 = threadIdx.x * 2654435761u, r1 = r0 ^ 0x1234567u, r2 = r0 + 77u, r3 = r0 * 3u, r4 = r0 + 5, r5 = r0 + 6, r6 = r0 + 7, r7 = r0 + 8;
        uint32_t a = 0x00010001u + threadIdx.x, b = 0x00030005u;
        for (int i = 0; i < iters; ++i)
            asm volatile(REP8(I7) REP8(I7) : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7) : "v"(a), "v"(b));
        out[blockIdx.x * 512 + threadIdx.x] = (float)(r0 ^ r1 ^ r2 ^ r3 ^ r4 ^ r5 ^ r6 ^ r7);
    }
}

static uint32_t* g_out;
static hipEvent_t g_e0, g_e1;
template <class F> static int timed(F launch, int iters, float* ms)
{
    launch(100);
    CHK(hipEventRecord(g_e0));
    launch(iters);
    CHK(hipEventRecord(g_e1));
    CHK(hipDeviceSynchronize());
    CHK(hipEventElapsedTime(ms, g_e0, g_e1));
    return 0;
}
template <int OP> static int opcode(const char* name)
{
    const int iters = 20000;
    printf("  %-22s", name);
    for (int w : {1, 2, 4})
    {
        float ms;
        if (timed([&](int n) { one_opcode<OP><<<256, 256 * w>>>(g_out, n); }, iters, &ms)) return 1;
        printf("  %d per SIMD: %.2f", w, ms * 1e6 / ((double)w * iters * 32));
    }
    printf("\n");
    return 0;
}
int main()
{
    CHK(hipMalloc(&g_out, 4 * 1024 * 256)); CHK(hipEventCreate(&g_e0)); CHK(hipEventCreate(&g_e1));
    printf("part 1: one opcode, eight independent chains; ns per wavefront instruction per SIMD at 1 / 2 / 4 wavefronts per SIMD\n");
    if (opcode<0>("v_mov_b32") || opcode<1>("v_lshrrev_b32") || opcode<2>("v_add_u32") || opcode<3>("v_xor_b32 (e64)") || opcode<4>("v_mul_lo_u16") || opcode<5>("v_fma_f32")
        || opcode<6>("v_mad_u32_u16") || opcode<7>("v_pk_mad_u16") || opcode<8>("v_dot4_u32_u8") || opcode<9>("v_sad_u8") || opcode<10>("v_perm_b32") || opcode<11>("v_pk_fma_f16")
        || opcode<12>("v_alignbit_b32") || opcode<13>("v_mul_lo_u32") || opcode<14>("v_bfe_u32") || opcode<15>("v_mul_u32_u24") || opcode<16>("v_mad_u16")) return 1;
    printf("part 2: the decoder's chain of seven dependent instructions; ns per instruction per SIMD\n");
    for (int w : {1, 2, 4})
    {
        float m1, m4;
        const int iters = 20000;
        if (timed([&](int n) { chain<1><<<256, 256 * w>>>(g_out, n); }, iters, &m1) || timed([&](int n) { chain<4><<<256, 256 * w>>>(g_out, n); }, iters, &m4)) return 1;
        printf("  %d per SIMD: one chain %.2f, four chains side by side %.2f\n", w, m1 * 1e6 / ((double)w * iters * 28), m4 * 1e6 / ((double)w * iters * 28));
    }
    printf("part 3: level-2 decode of four weights (18 instructions), 4 wavefronts per SIMD; ns per four weights per SIMD\n");
    {
        float m0, m1;
        const int iters = 200000;
        if (timed([&](int n) { decode4<0><<<256, 1024>>>(g_out, n); }, iters, &m0) || timed([&](int n) { decode4<1><<<256, 1024>>>(g_out, n); }, iters, &m1)) return 1;
        printf("  hash = v_mad_u32_u16 + v_pk_mad_u16: %.2f   hash = and / shift + v_mul_lo_u32: %.2f\n", m0 * 1e6 / (4.0 * iters), m1 * 1e6 / (4.0 * iters));
    }
    printf("part 4: 8 MFMAs (16x16x32 f16) per iteration on one wavefront, 16 vector instructions per iteration on another, same SIMD; ns per iteration\n");
    for (int mode = 1; mode <= 3; ++mode)
    {
        float ms;
        const int iters = 100000;
        if (timed([&](int n) { mfma_and_valu<<<256, 512>>>((float*)g_out, n, mode); }, iters, &ms)) return 1;
        printf("  %s: %.1f\n", mode == 1 ? "MFMAs alone" : mode == 2 ? "vector instructions alone" : "both", ms * 1e6 / iters);
    }
    return 0;
}
