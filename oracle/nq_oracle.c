/* CPU oracle in C for the NestQuant nested-trellis decoder.  TEST INFRASTRUCTURE ONLY: linked by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg, never by the product library.
 *
 * A second, independent restatement (the first is oracle/nq_oracle.py) of
 *   window patterns / step offsets   reference sm120/ref15_spec.py:43-46, sm120/moe.py:10-20
 *   lane records and ring wrap       reference sm120/ref15_spec.py:49-61,132-137, sm120/moe.py:111-127
 *   mul1 hash, byte sum, Q2          reference sm120/ref15_spec.py:64-76
 *   RM_P fold and its constants      reference sm120/ref15_spec.py:79-90, sm120/moe.py:128-134 (fp32 subtraction)
 *   sub-array plane layout           reference sm120/moe.py:36-66
 *   unit geometry                    reference sm120/ref15_spec.py:118-125
 * written with scalar loops and 64-bit shifts (no vector tricks), parallel over units with OpenMP. Pinned by
 * tests/test_oracle_c.py against the numpy oracle and the golden fixtures of the reference's own decoder.
 */
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

static const int PAT_KA[13]   = {2, 1, 2, 2, 3, 1, 1, 2, 1, 2, 1, 2, 2};
static const int PAT_MASK[13] = {0x0000, 0xEEEE, 0xAAAA, 0x8888, 0x0000, 0xAAAA, 0xFFFE, 0x9248, 0xFEFE, 0xD5AA, 0x0000, 0x0000, 0x0000};

static int popc(int m) { int c = 0; while (m) { c += m & 1; m >>= 1; } return c; }
int nqo_rbits(int code) { return 4 * (16 * PAT_KA[code] + popc(PAT_MASK[code])); }
int nqo_step_off(int p, int code)
{
    const int ka = PAT_KA[code], mask = PAT_MASK[code];
    int s = (p >> 4) * (16 * ka + popc(mask));
    for (int i = 0; i < (p & 15); ++i) s += ka + ((mask >> i) & 1);
    return s;
}

/* fp32 -> fp16 bits, round to nearest even, with subnormals; fp16 bits -> fp32 */
static uint16_t f32_to_f16(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | (x > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);             /* rounds to infinity */
    if (x < 0x33000001u) return (uint16_t)sign;                          /* below half the smallest subnormal */
    int e = (int)(x >> 23) - 127;
    uint32_t m = (x & 0x7FFFFFu) | 0x800000u;                            /* 24-bit significand */
    int shift = e >= -14 ? 13 : 13 + (-14 - e);                          /* bits dropped */
    uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    if (e >= -14) return (uint16_t)(sign | ((uint32_t)((e + 15) << 10) + (q - 0x400u)));   /* carry moves into the exponent */
    return (uint16_t)(sign | q);                                          /* subnormal (q == 0x400 becomes the smallest normal) */
}
static float f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3FFu;
    uint32_t x;
    if (e == 0)
    {
        if (m == 0) x = sign;
        else { int k = 0; uint32_t mm = m; while (!(mm & 0x400u)) { mm <<= 1; ++k; } x = sign | ((uint32_t)(113 - k) << 23) | ((mm & 0x3FFu) << 13); }
    }
    else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112u) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
}
uint16_t nqo_f32_to_f16(float f) { return f32_to_f16(f); }
float nqo_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

static int hash_sum(uint32_t st)
{
    const uint32_t x = st * 0x83DCD12Du;
    return (int)((x & 255u) + ((x >> 8) & 255u) + ((x >> 16) & 255u) + (x >> 24));
}
int nqo_hash_sum(uint32_t st) { return hash_sum(st & 0xFFFFu); }

/* 16-bit window at bit offset `off` of a little-endian word array */
static uint32_t window(const uint32_t* w, int off)
{
    const int i = off >> 5, s = off & 31;
    const uint64_t both = (uint64_t)w[i] | ((uint64_t)w[i + 1] << 32);
    return (uint32_t)(both >> s) & 0xFFFFu;
}

/* value = fp16(a * h + c) with one rounding; the exact sum has at most 24 significant bits, so double -> float is exact */
static uint16_t fma_f16(uint16_t a, double h, uint16_t c, int negate)
{
    double v = (double)f16_to_f32(a) * h + (double)f16_to_f32(c);
    if (negate) v = -v;
    return f32_to_f16((float)v);
}

void nqo_fold_consts(int Mb, int N, uint16_t* Ah, uint16_t* Ch)
{
    const volatile float rcp = 1.0f / (float)Mb;                         /* volatile: one IEEE operation per line */
    const volatile float a = 1.732421875f * rcp;
    *Ah = f32_to_f16(a);
    const volatile float t0 = (float)N * rcp;
    const volatile float t1 = t0 * -3.453125f;
    const volatile float t2 = t1 + -3.453125f;
    const volatile float t3 = 1024.0f * f16_to_f32(*Ah);
    const volatile float t4 = t2 - t3;
    *Ch = f32_to_f16(t4);
}

/* unpack the sub-array layout (uint4 x n4 | uint2 | uint | ushort | bit-packed tail) into words[nrec][NW];
 * split == 1: 128-bit records stored as uint2 | uint2 (plane P3's records, then plane P4's); split == 2: the same storage, the
 * record being the two 64-bit records interleaved bit by bit (bit 2 i from P3, bit 2 i + 1 from P4) */
void nqo_unpack(const uint8_t* buf, long nrec, int code, int split, uint32_t* words)
{
    const int bits = nqo_rbits(code), nw = (bits + 31) / 32;
    memset(words, 0, (size_t)nrec * nw * 4);
    if (split)
    {
        const uint32_t* a = (const uint32_t*)buf; const uint32_t* b = a + nrec * 2;
        for (long r = 0; r < nrec; ++r)
        {
            if (split == 1) { words[r * 4] = a[2 * r]; words[r * 4 + 1] = a[2 * r + 1]; words[r * 4 + 2] = b[2 * r]; words[r * 4 + 3] = b[2 * r + 1]; continue; }
            const uint64_t p3 = (uint64_t)a[2 * r] | ((uint64_t)a[2 * r + 1] << 32), p4 = (uint64_t)b[2 * r] | ((uint64_t)b[2 * r + 1] << 32);
            for (int i = 0; i < 64; ++i)
            {
                words[r * 4 + (2 * i) / 32] |= (uint32_t)((p3 >> i) & 1u) << ((2 * i) & 31);
                words[r * 4 + (2 * i + 1) / 32] |= (uint32_t)((p4 >> i) & 1u) << ((2 * i + 1) & 31);
            }
        }
        return;
    }
    const int n4 = bits / 128, r1 = bits % 128, n2 = r1 / 64, r2 = r1 % 64, n1 = r2 / 32, nh = (r2 % 32) / 16, T = bits % 16;
    const uint8_t* p = buf; int k = 0;
    if (n4) { for (long r = 0; r < nrec; ++r) memcpy(words + r * nw, p + r * 16 * n4, 16 * n4); p += nrec * 16 * n4; k = 4 * n4; }
    if (n2) { for (long r = 0; r < nrec; ++r) memcpy(words + r * nw + k, p + r * 8, 8); p += nrec * 8; k += 2; }
    if (n1) { for (long r = 0; r < nrec; ++r) memcpy(words + r * nw + k, p + r * 4, 4); p += nrec * 4; k += 1; }
    if (nh) { for (long r = 0; r < nrec; ++r) { uint16_t v; memcpy(&v, p + r * 2, 2); words[r * nw + k] = v; } p += nrec * 2; }
    if (T)
    {
        const int a = bits - T;
        for (long r = 0; r < nrec; ++r)
            for (int i = 0; i < T; ++i)
            {
                const long b = r * T + i;
                const uint32_t bit = (p[b >> 3] >> (b & 7)) & 1u;
                words[r * nw + (a + i) / 32] |= bit << ((a + i) & 31);
            }
    }
}

/* Dense decode of one projection [N][K] -> fp16 bits, row-major.
 * base [nrec][4]; level 2: res/dw ignored. level >= 3: res [nrec][NW] unpacked words of `code`, dw [units] = Mb | N << 8.
 * var: optional uint8 per unit, bit g negates ring g. */
void nqo_decode_proj(const uint32_t* base, const uint32_t* res, int code, const uint32_t* dw, const uint8_t* var,
                     int N, int K, int level, uint16_t* out)
{
    const int S = N / 16, C = K / 128;
    const int rb = level >= 3 ? nqo_rbits(code) : 0, nw = (rb + 31) / 32;
    int offb[64], offr[64];
    for (int j = 0; j < 64; ++j) { offb[j] = nqo_step_off(j, 0); offr[j] = level >= 3 ? nqo_step_off(j, code) : 0; }
#pragma omp parallel for schedule(static)
    for (long u = 0; u < (long)S * C; ++u)
    {
        const int strip = (int)(u / C), chunk = (int)(u % C);
        uint16_t Ah = 0x1EEE, Ch = 0xC931; int Mb = 0, Nn = 0;
        if (level >= 3) { Mb = (int)(dw[u] & 255u); Nn = (int)((dw[u] >> 8) & 255u); nqo_fold_consts(Mb, Nn, &Ah, &Ch); }
        for (int lane = 0; lane < 32; ++lane)
        {
            const int g = lane >> 2, t4 = lane & 3, nb = 4 * g + ((t4 + 1) & 3);   /* next lane of the ring */
            const long rec = u * 32 + lane, recn = u * 32 + nb;
            uint32_t wb[8] = {0}, wr[10] = {0};
            memcpy(wb, base + rec * 4, 16); wb[4] = base[recn * 4];
            if (level >= 3)
            {
                memcpy(wr, res + rec * nw, (size_t)nw * 4);
                const uint32_t first = res[recn * nw]; const int t = rb & 31;
                if (t == 0) wr[nw] = first;
                else { wr[nw - 1] = (wr[nw - 1] & ((1u << t) - 1u)) | (first << t); wr[nw] = first >> (32 - t); }
            }
            const int neg = var ? (var[u] >> g) & 1 : 0;
            for (int j = 0; j < 64; ++j)
            {
                const int sb = hash_sum(window(wb, offb[j]));
                double h;
                if (level >= 3)
                {
                    const int sr = hash_sum(window(wr, offr[j]));
                    h = 1024.0 + (double)((Mb * sb + Nn * sr + 128) >> 8);
                }
                else h = 1024.0 + (double)sb;
                const int pp = j >> 1, e = j & 1, t = pp >> 2, r = pp & 3;
                const int row = 16 * strip + g + 8 * (r & 1), col = 128 * chunk + 16 * t + 2 * t4 + 8 * (r >> 1) + e;
                out[(size_t)row * K + col] = fma_f16(Ah, h, Ch, neg);
            }
        }
    }
}

/* y[n] = sum_k W[n][k] (fp16 bits) * x[k] in fp32, parallel over rows: the matvec of the CPU baseline */
void nqo_matvec_f16(const uint16_t* W, const float* x, int N, int K, float* y)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
    {
        float acc = 0.f;
        const uint16_t* w = W + (size_t)n * K;
        for (int k = 0; k < K; ++k) acc += f16_to_f32(w[k]) * x[k];
        y[n] = acc;
    }
}
