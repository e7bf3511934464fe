/*
 * oxk_oracle.c — CPU restatement of oxidize-c's quantized-matvec arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels.  See
 * oxk_oracle.h for what each function restates and how it was pinned.
 *
 * Build: gcc -std=c11 -O2 -ffp-contract=off -fopenmp (float contraction must
 * stay off: the reference evaluates `dw*dq*(float)pos - dmin*dq*(float)mn`
 * as four roundings plus one for the running sum, oxidize-c/Makefile:21).
 */
#include "oxk_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ─── scalar helpers ──────────────────────────────────────────────────── */

static inline uint16_t rd_u16(const uint8_t *p)
{
    return (uint16_t)(p[0] | ((unsigned)p[1] << 8));
}

static inline uint32_t rd_u32(const uint8_t *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) |
           ((uint32_t)p[3] << 24);
}

static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Exact binary16 -> binary32 (oxk.c:26-56): zero, subnormal (renormalised),
 * normal, inf/nan.  Written as "value = mant * 2^(e-25)" for subnormals so it
 * does not share the reference's shift loop. */
float oxo_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 31u;
    const uint32_t m = h & 0x3FFu;
    if (e == 31u) return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e != 0u)  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    if (m == 0u)  return bits_f32(sign);
    /* subnormal: m * 2^-24, exactly representable in binary32 */
    const float mag = (float)m * 5.9604644775390625e-8f;
    uint32_t u;
    memcpy(&u, &mag, 4);
    return bits_f32(u | sign);
}

/* binary32 -> binary16 bits with the reference's round-half-UP rule
 * (flash_attention.c:149-185): drop the low mantissa bits, add one when the
 * highest dropped bit is set; carries may bump the exponent up to inf;
 * values below 2^-25 flush to signed zero. */
uint16_t oxo_f32_to_f16_bits(float v)
{
    uint32_t u;
    memcpy(&u, &v, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const int32_t e32 = (int32_t)((u >> 23) & 0xFFu);
    const uint32_t man = u & 0x7FFFFFu;

    if (e32 == 255) {
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        uint16_t payload = (uint16_t)(man >> 13);
        if (payload == 0) payload = 1;
        return (uint16_t)(sign | 0x7C00u | payload);
    }
    const int32_t e16 = e32 - 112;
    if (e16 >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e16 >= 1) {
        uint32_t out = ((uint32_t)e16 << 10) | (man >> 13);
        if (man & 0x1000u) {
            /* +1 on the 10-bit field; a carry out of it clears the field and
             * increments the exponent, which is what plain addition does. */
            out += 1u;
            if (out >= 0x7C00u) return (uint16_t)(sign | 0x7C00u);
        }
        return (uint16_t)(sign | out);
    }
    if (e16 < -10) return sign;
    const uint32_t full = man | 0x800000u;
    const uint32_t sh = (uint32_t)(14 - e16);
    uint32_t out = full >> sh;
    if ((full >> (sh - 1u)) & 1u) out += 1u;
    return (uint16_t)(sign | out);
}

void oxo_scale_min_k4(unsigned j, const uint8_t s[12], uint8_t *sc, uint8_t *mn)
{
    if (j < 4u) {
        *sc = (uint8_t)(s[j] & 0x3Fu);
        *mn = (uint8_t)(s[j + 4u] & 0x3Fu);
        return;
    }
    const unsigned lo = s[j + 4u];
    *sc = (uint8_t)((lo & 15u) | ((s[j - 4u] >> 6) << 4));
    *mn = (uint8_t)((lo >> 4) | ((s[j] >> 6) << 4));
}

/* All eight (scale, min) pairs at once through the three-word mask form
 * (the form the GPU kernels use; equality with oxo_scale_min_k4 over random
 * inputs is part of the oracle's self-test). */
static void scale_min_all(const uint8_t s[12], uint8_t sc[8], uint8_t mn[8])
{
    const uint32_t u0 = rd_u32(s), u1 = rd_u32(s + 4), u2 = rd_u32(s + 8);
    const uint32_t sc_lo = u0 & 0x3F3F3F3Fu;
    const uint32_t mn_lo = u1 & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (u2 & 0x0F0F0F0Fu) | ((u0 >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((u2 >> 4) & 0x0F0F0F0Fu) | ((u1 >> 2) & 0x30303030u);
    for (int k = 0; k < 4; k++) {
        sc[k]     = (uint8_t)(sc_lo >> (8 * k));
        sc[k + 4] = (uint8_t)(sc_hi >> (8 * k));
        mn[k]     = (uint8_t)(mn_lo >> (8 * k));
        mn[k + 4] = (uint8_t)(mn_hi >> (8 * k));
    }
}

/* ─── activation quantisers ───────────────────────────────────────────── */

static inline float absmax(const float *x, size_t n)
{
    float m = 0.0f;
    for (size_t i = 0; i < n; i++) {
        const float a = fabsf(x[i]);
        if (a > m) m = a;
    }
    return m;
}

/* matvec.c:147-150 and :303-306, literally.  For a product that is not finite (a non-finite input, or a
 * block so small that 1/d overflows: largest magnitude below 3.7e-37) the value depends on the host's
 * float -> integer conversion and differs between the reference's own scalar and AVX-512 quantisers;
 * such inputs are outside what the parity tests compare. */
static inline int8_t quant1(float x, float inv)
{
    int v = (int)lrintf(x * inv);
    if (v > 127) v = 127;
    if (v < -128) v = -128;
    return (int8_t)v;
}

void oxo_quantize_q8_k(const float *x, size_t n, uint8_t *out)
{
    for (size_t b = 0; b < n / OXO_QK_K; b++) {
        const float *src = x + b * OXO_QK_K;
        uint8_t *dst = out + b * OXO_Q8_K_BYTES;
        const float d = absmax(src, OXO_QK_K) / 127.0f;
        const float inv = (d != 0.0f) ? 1.0f / d : 0.0f;
        memcpy(dst, &d, 4);
        int8_t *q = (int8_t *)(dst + 4);
        for (size_t g = 0; g < 16; g++) {
            int32_t acc = 0;
            for (size_t i = 16 * g; i < 16 * g + 16; i++) {
                q[i] = quant1(src[i], inv);
                acc += q[i];
            }
            const int16_t s = (int16_t)acc;
            memcpy(dst + 260 + 2 * g, &s, 2);
        }
    }
}

void oxo_quantize_q8_0(const float *x, size_t n, uint8_t *out)
{
    for (size_t b = 0; b < n / OXO_QK8_0; b++) {
        const float *src = x + b * OXO_QK8_0;
        uint8_t *dst = out + b * OXO_Q8_0_BYTES;
        const float d = absmax(src, OXO_QK8_0) / 127.0f;
        const float inv = (d != 0.0f) ? 1.0f / d : 0.0f;
        const uint16_t h = oxo_f32_to_f16_bits(d);
        dst[0] = (uint8_t)(h & 0xFFu);
        dst[1] = (uint8_t)(h >> 8);
        for (size_t i = 0; i < OXO_QK8_0; i++)
            dst[2 + i] = (uint8_t)quant1(src[i], inv);
    }
}

/* ─── block dots ──────────────────────────────────────────────────────── */

float oxo_dot_q4_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *sub, int32_t *posmin)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q4_K_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        const float dmin = oxo_f16_to_f32(rd_u16(w + 2));
        float dq;
        memcpy(&dq, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);
        const uint8_t *nib = w + 16;

        uint8_t sc[8], mn[8];
        scale_min_all(w + 4, sc, mn);

        /* sub-block j = elements [32j, 32j+32): even j are the low nibbles of
         * the 32 bytes nib[16j ..], odd j the high nibbles of the same bytes */
        int32_t S[8];
        for (int j = 0; j < 8; j++) {
            const uint8_t *src = nib + 32 * (j >> 1);
            const int shift = (j & 1) * 4;
            int32_t acc = 0;
            for (int l = 0; l < 32; l++)
                acc += (int32_t)((src[l] >> shift) & 15) * (int32_t)q[32 * j + l];
            S[j] = acc;
        }
        int32_t pos = 0, mins = 0;
        for (int j = 0; j < 8; j++) {
            int16_t b0, b1;
            memcpy(&b0, a + 260 + 4 * j, 2);
            memcpy(&b1, a + 262 + 4 * j, 2);
            pos += (int32_t)sc[j] * S[j];
            mins += (int32_t)mn[j] * ((int32_t)b0 + (int32_t)b1);
        }
        if (sub) memcpy(sub + 8 * b, S, sizeof S);
        if (posmin) { posmin[2 * b] = pos; posmin[2 * b + 1] = mins; }

        const float t_pos = dw * dq;
        const float t_min = dmin * dq;
        const float up = t_pos * (float)pos;
        const float dn = t_min * (float)mins;
        sum += up - dn;
    }
    return sum;
}

float oxo_dot_q5_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *sub, int32_t *posmin)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q5_K_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        const float dmin = oxo_f16_to_f32(rd_u16(w + 2));
        float dq;
        memcpy(&dq, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);
        const uint8_t *hbits = w + 16;      /* 32 bytes: bit j of byte l is the fifth bit of element 32j + l */
        const uint8_t *nib = w + 48;

        uint8_t sc[8], mn[8];
        scale_min_all(w + 4, sc, mn);

        /* sub-block j = elements [32j, 32j+32): the nibble comes from where
         * Q4_K keeps it, the fifth bit of element 32j + l is bit j of hbits[l] */
        int32_t S[8];
        for (int j = 0; j < 8; j++) {
            const uint8_t *src = nib + 32 * (j >> 1);
            const int shift = (j & 1) * 4;
            int32_t acc = 0;
            for (int l = 0; l < 32; l++) {
                const int32_t code = (int32_t)((src[l] >> shift) & 15) +
                                     (int32_t)(((hbits[l] >> j) & 1) << 4);
                acc += code * (int32_t)q[32 * j + l];
            }
            S[j] = acc;
        }
        int32_t pos = 0, mins = 0;
        for (int j = 0; j < 8; j++) {
            int16_t b0, b1;
            memcpy(&b0, a + 260 + 4 * j, 2);
            memcpy(&b1, a + 262 + 4 * j, 2);
            pos += (int32_t)sc[j] * S[j];
            mins += (int32_t)mn[j] * ((int32_t)b0 + (int32_t)b1);
        }
        if (sub) memcpy(sub + 8 * b, S, sizeof S);
        if (posmin) { posmin[2 * b] = pos; posmin[2 * b + 1] = mins; }

        const float t_pos = dw * dq;
        const float t_min = dmin * dq;
        const float up = t_pos * (float)pos;
        const float dn = t_min * (float)mins;
        sum += up - dn;
    }
    return sum;
}

float oxo_dot_q6_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *grp)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q6_K_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const int8_t *sc = (const int8_t *)(w + 192);
        const float dw = oxo_f16_to_f32(rd_u16(w + 208));
        float dq;
        memcpy(&dq, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);

        /* element e of the block: half n = e/128, quarter k = (e%128)/32,
         * l = e%32; low 4 bits from ql[64n + 32(k&1) + l] (low nibble for
         * k<2, high nibble otherwise), top 2 bits from qh[32n + l] >> 2k. */
        int32_t G[16];
        for (int g = 0; g < 16; g++) {
            int32_t acc = 0;
            for (int i = 0; i < 16; i++) {
                const int e = 16 * g + i;
                const int n = e >> 7, k = (e >> 5) & 3, l = e & 31;
                const unsigned lo = w[64 * n + 32 * (k & 1) + l];
                const unsigned hi = w[128 + 32 * n + l];
                const int code = (int)((k < 2 ? (lo & 15u) : (lo >> 4)) |
                                       (((hi >> (2 * k)) & 3u) << 4));
                acc += code * (int32_t)q[e];
            }
            G[g] = acc;
        }
        int32_t pos = 0, off = 0;
        for (int g = 0; g < 16; g++) {
            int16_t bs;
            memcpy(&bs, a + 260 + 2 * g, 2);
            pos += (int32_t)sc[g] * G[g];
            off += (int32_t)sc[g] * (int32_t)bs;
        }
        if (grp) memcpy(grp + 16 * b, G, sizeof G);
        const float t = dw * dq;
        sum += t * (float)(pos - 32 * off);
    }
    return sum;
}

/* Q2_K and Q3_K walk their 2-bit codes alike: element e = 128*outer +
 * 32*inner + l (l < 32) is bits [2*inner, 2*inner + 2) of qs[32*outer + l];
 * Q3_K adds bit (4*outer + inner) of hmask[l] as the code's third bit
 * (src/compute/oxk.c:512-590). */
static unsigned q23_code(const uint8_t *qs, const uint8_t *hmask, unsigned e)
{
    const unsigned outer = e >> 7, inner = (e >> 5) & 3u, l = e & 31u;
    unsigned c = (qs[32u * outer + l] >> (2u * inner)) & 3u;
    if (hmask) c |= ((hmask[l] >> (4u * outer + inner)) & 1u) << 2;
    return c;
}

/* the sixteen 6-bit scales of a Q3_K block, minus 32 (src/compute/oxk.c:556-573) */
static void q3k_scales(const uint8_t *p, int8_t sc[16])
{
    uint32_t a[4];
    for (unsigned i = 0; i < 3; i++)
        a[i] = (uint32_t)p[4 * i] | ((uint32_t)p[4 * i + 1] << 8) | ((uint32_t)p[4 * i + 2] << 16) |
               ((uint32_t)p[4 * i + 3] << 24);
    const uint32_t t = a[2];
    a[2] = ((a[0] >> 4) & 0x0F0F0F0Fu) | (((t >> 4) & 0x03030303u) << 4);
    a[3] = ((a[1] >> 4) & 0x0F0F0F0Fu) | (((t >> 6) & 0x03030303u) << 4);
    a[0] = (a[0] & 0x0F0F0F0Fu) | ((t & 0x03030303u) << 4);
    a[1] = (a[1] & 0x0F0F0F0Fu) | (((t >> 2) & 0x03030303u) << 4);
    for (unsigned i = 0; i < 4; i++)
        for (unsigned j = 0; j < 4; j++)
            sc[4 * i + j] = (int8_t)(int32_t)(((a[i] >> (8 * j)) & 0xFFu) - 32u);
}

float oxo_dot_q2_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *grp)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q2_K_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w + 80));
        const float dmin = oxo_f16_to_f32(rd_u16(w + 82));
        float dq;
        memcpy(&dq, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);
        int32_t pos = 0, min_acc = 0;
        for (unsigned g = 0; g < 16; g++) {
            int32_t acc = 0;
            for (unsigned i = 0; i < 16; i++)
                acc += (int32_t)q23_code(w + 16, NULL, 16 * g + i) * (int32_t)q[16 * g + i];
            int16_t bs;
            memcpy(&bs, a + 260 + 2 * g, 2);
            pos += (int32_t)(w[g] & 15u) * acc;
            min_acc += (int32_t)(w[g] >> 4) * (int32_t)bs;
            if (grp) grp[16 * b + g] = acc;
        }
        sum += dq * (dw * (float)pos - dmin * (float)min_acc);
    }
    return sum;
}

float oxo_dot_q3_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *grp)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q3_K_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w + 108));
        float dq;
        memcpy(&dq, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);
        int8_t sc[16];
        q3k_scales(w + 96, sc);
        int32_t pos = 0, off = 0;
        for (unsigned g = 0; g < 16; g++) {
            int32_t acc = 0;
            for (unsigned i = 0; i < 16; i++)
                acc += (int32_t)q23_code(w + 32, w, 16 * g + i) * (int32_t)q[16 * g + i];
            int16_t bs;
            memcpy(&bs, a + 260 + 2 * g, 2);
            pos += (int32_t)sc[g] * acc;
            off += (int32_t)sc[g] * (int32_t)bs;
            if (grp) grp[16 * b + g] = acc;
        }
        sum += dw * dq * (float)(pos - 4 * off);
    }
    return sum;
}

float oxo_dot_q8_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *isum)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_Q8_0_BYTES;
        const uint8_t *a = act + b * OXO_Q8_0_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        const float dq = oxo_f16_to_f32(rd_u16(a));
        int32_t acc = 0;
        for (int i = 0; i < 32; i++)
            acc += (int32_t)(int8_t)w[2 + i] * (int32_t)(int8_t)a[2 + i];
        if (isum) isum[b] = acc;
        const float t = dw * dq;
        sum += t * (float)acc;
    }
    return sum;
}

/* The 32-value formats.  `isum` (optional) receives one int32 per block: the
 * offset-corrected integer dot for Q4_0 / Q5_0, the plain code dot for Q4_1 /
 * Q5_1 (whose second integer is the sum of the activation values). */
static float dot_legacy(int five_bit, int has_min, const uint8_t *row, size_t blocks,
                        const uint8_t *act, int32_t *isum)
{
    const size_t bytes = 18u + (has_min ? 2u : 0u) + (five_bit ? 4u : 0u);
    const size_t qh_at = has_min ? 4u : 2u, qs_at = bytes - 16u;
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * bytes;
        const uint8_t *a = act + b * OXO_Q8_0_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        const float mw = has_min ? oxo_f16_to_f32(rd_u16(w + 2)) : 0.0f;
        const float dq = oxo_f16_to_f32(rd_u16(a));
        const int8_t *q = (const int8_t *)(a + 2);
        uint32_t qh = 0;
        if (five_bit) memcpy(&qh, w + qh_at, 4);
        int32_t dotp = 0, qsum = 0;
        for (int j = 0; j < 16; j++) {
            /* low nibble of byte j = element j, high nibble = element j + 16 */
            const int32_t x0 = (int32_t)(w[qs_at + j] & 15u) | (int32_t)(((qh >> j) & 1u) << 4);
            const int32_t x1 = (int32_t)(w[qs_at + j] >> 4) | (int32_t)(((qh >> (j + 16)) & 1u) << 4);
            dotp += x0 * (int32_t)q[j] + x1 * (int32_t)q[j + 16];
            qsum += (int32_t)q[j] + (int32_t)q[j + 16];
        }
        if (has_min) {
            if (isum) isum[b] = dotp;
            const float t = dw * dq;
            const float tm = mw * dq;
            const float up = t * (float)dotp;
            const float off = tm * (float)qsum;
            sum += up + off;
        } else {
            const int32_t v = dotp - (five_bit ? 16 : 8) * qsum;
            if (isum) isum[b] = v;
            const float t = dw * dq;
            sum += t * (float)v;
        }
    }
    return sum;
}

/* the 3-bit code of element i: bits [3i, 3i+3) of the 12 packed bytes, least
 * significant bit first (src/compute/oxk.c:206-218) */
static unsigned al5_xs_code(const uint8_t *packed, unsigned i)
{
    unsigned v = 0;
    for (unsigned bb = 0; bb < 3; bb++) {
        const unsigned bit = 3u * i + bb;
        v |= ((packed[bit >> 3] >> (bit & 7u)) & 1u) << bb;
    }
    return v;
}

float oxo_dot_al5_xs_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_AL5_XS_BYTES;
        const uint8_t *a = act + b * OXO_Q8_0_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        const float dq = oxo_f16_to_f32(rd_u16(a));
        const int8_t *q = (const int8_t *)(a + 2);
        int32_t acc = 0;
        for (unsigned i = 0; i < 32; i++)
            acc += ((int32_t)al5_xs_code(w + 2, i) - 4) * (int32_t)q[i];
        if (isum) isum[b] = acc;
        const float t = dw * dq;
        sum += t * (float)acc;
    }
    return sum;
}

float oxo_dot_q4_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum)
{
    return dot_legacy(0, 0, row, blocks, act, isum);
}
float oxo_dot_q4_1_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum)
{
    return dot_legacy(0, 1, row, blocks, act, isum);
}
float oxo_dot_q5_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum)
{
    return dot_legacy(1, 0, row, blocks, act, isum);
}
float oxo_dot_q5_1_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum)
{
    return dot_legacy(1, 1, row, blocks, act, isum);
}

/* ─── the codebook formats ────────────────────────────────────────────── */

#include "iq_grids.inc"     /* OXH_IQ3S_GRID, OXH_IQ1XXXS_GRID: data shared with the kernels */

float oxo_dot_iq3_s_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *lanes)
{
    float acc[8] = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f };
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_IQ3_S_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        float dq;
        memcpy(&dq, a, 4);
        const float d = oxo_f16_to_f32(rd_u16(w)) * dq;
        const int8_t *q = (const int8_t *)(a + 4);
        int32_t lane[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
        for (unsigned sb = 0; sb < 8; sb++) {
            const uint8_t *codes = w + 2 + 8 * sb, *signs = w + 74 + 4 * sb;
            const unsigned ninth = w[66 + sb];
            const unsigned nib = (w[106 + sb / 2] >> (4 * (sb & 1))) & 15u;
            const int32_t ls = 2 * (int32_t)nib + 1;
            /* value e of the sub-block: byte e%4 of the grid entry of code e/4; sign bit e%8 of byte e/8 */
            for (unsigned e = 0; e < 32; e++) {
                const unsigned c = e / 4;
                const unsigned code = codes[c] | (((ninth >> c) & 1u) << 8);
                const int32_t mag = (int32_t)((OXH_IQ3S_GRID[code] >> (8 * (e % 4))) & 0xFFu);
                const int32_t wv = ((signs[e / 8] >> (e % 8)) & 1u) ? -mag : mag;
                lane[e / 4] += ls * wv * (int32_t)q[32 * sb + e];
            }
        }
        if (lanes) memcpy(lanes + 8 * b, lane, sizeof lane);
        for (int j = 0; j < 8; j++) acc[j] = acc[j] + d * (float)lane[j];
    }
    const float s0 = acc[0] + acc[4], s1 = acc[1] + acc[5], s2 = acc[2] + acc[6], s3 = acc[3] + acc[7];
    return (s0 + s2) + (s1 + s3);
}

float oxo_dot_iq1_xxxs_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *sums)
{
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *w = row + b * OXO_IQ1_XXXS_BYTES;
        const uint8_t *a = act + b * OXO_Q8_K_BYTES;
        const float dw = oxo_f16_to_f32(rd_u16(w));
        float da;
        memcpy(&da, a, 4);
        const int8_t *q = (const int8_t *)(a + 4);
        int32_t main_sum = 0, delta_sum = 0;
        for (unsigned g = 0; g < 8; g++) {          /* groups of 32 values */
            const unsigned nib = (w[34 + g / 2] >> (4 * (g & 1))) & 15u;
            const int32_t scale = 2 * (int32_t)(nib & 7u) + 1;
            int32_t dot = 0, total = 0;
            for (unsigned e = 0; e < 32; e++) {
                const uint64_t entry = OXH_IQ1XXXS_GRID[w[2 + 4 * g + e / 8]];
                dot += (int32_t)(int8_t)(entry >> (8 * (e % 8))) * (int32_t)q[32 * g + e];
            }
            for (unsigned h = 0; h < 2; h++) {
                int16_t bs;
                memcpy(&bs, a + 260 + 2 * (2 * g + h), 2);
                total += bs;
            }
            main_sum += scale * dot;
            delta_sum += scale * ((nib & 8u) ? -1 : 1) * total;
        }
        if (sums) { sums[2 * b] = main_sum; sums[2 * b + 1] = delta_sum; }
        sum += dw * da * ((float)main_sum + 0.125f * (float)delta_sum);
    }
    return sum;
}

/* ─── eligibility ─────────────────────────────────────────────────────── */

static size_t block_bytes(uint32_t qtype)
{
    switch (qtype) {
    case OXO_AL5:
    case OXO_Q4_0:   return 18u;
    case OXO_Q4_1:   return 20u;
    case OXO_AL6:
    case OXO_Q5_0:   return 22u;
    case OXO_Q5_1:   return 24u;
    case OXO_AL8:
    case OXO_Q8_0:   return OXO_Q8_0_BYTES;
    case OXO_AL5_XS: return OXO_AL5_XS_BYTES;
    case OXO_Q4_K_S:
    case OXO_Q4_K_M: return OXO_Q4_K_BYTES;
    case OXO_Q5_K_S:
    case OXO_Q5_K_M: return OXO_Q5_K_BYTES;
    case OXO_Q6_K:   return OXO_Q6_K_BYTES;
    case OXO_Q2_K:   return OXO_Q2_K_BYTES;
    case OXO_Q3_K_S:
    case OXO_Q3_K_M:
    case OXO_Q3_K_L: return OXO_Q3_K_BYTES;
    case OXO_IQ3_S:  return OXO_IQ3_S_BYTES;
    case OXO_IQ1_XXXS: return OXO_IQ1_XXXS_BYTES;
    default:         return 0;
    }
}

int oxo_act_kind(uint32_t qtype, size_t cols)
{
    switch (qtype) {
    case OXO_Q4_0:
    case OXO_AL5:
    case OXO_Q4_1:
    case OXO_Q5_0:
    case OXO_AL6:
    case OXO_Q5_1:
    case OXO_Q8_0:
    case OXO_AL8:
    case OXO_AL5_XS: return (cols % OXO_QK8_0 == 0) ? 1 : 0;
    case OXO_Q2_K:
    case OXO_Q3_K_S:
    case OXO_Q3_K_M:
    case OXO_Q3_K_L:
    case OXO_Q4_K_S:
    case OXO_Q4_K_M:
    case OXO_Q5_K_S:
    case OXO_Q5_K_M:
    case OXO_Q6_K:
    case OXO_IQ1_XXXS:
    case OXO_IQ3_S:  return (cols % OXO_QK_K == 0) ? 2 : 0;
    default:         return 0;
    }
}

static size_t n_blocks(int kind, size_t cols)
{
    return kind == 2 ? cols / OXO_QK_K : cols / OXO_QK8_0;
}

int oxo_stride_ok(uint32_t qtype, size_t cols, size_t row_bytes)
{
    const int kind = oxo_act_kind(qtype, cols);
    if (!kind) return 0;
    return row_bytes == n_blocks(kind, cols) * block_bytes(qtype);
}

static float row_dot(uint32_t qtype, const uint8_t *row, size_t blocks,
                     const uint8_t *act)
{
    switch (qtype) {
    /* AL5 / AL6 / AL8: the Q4_0 / Q5_0 / Q8_0 dots (src/compute/matvec.c:323-329) */
    case OXO_AL5:
    case OXO_Q4_0:   return oxo_dot_q4_0_q8_0(row, blocks, act, NULL);
    case OXO_Q4_1:   return oxo_dot_q4_1_q8_0(row, blocks, act, NULL);
    case OXO_AL6:
    case OXO_Q5_0:   return oxo_dot_q5_0_q8_0(row, blocks, act, NULL);
    case OXO_Q5_1:   return oxo_dot_q5_1_q8_0(row, blocks, act, NULL);
    case OXO_AL8:
    case OXO_Q8_0:   return oxo_dot_q8_0_q8_0(row, blocks, act, NULL);
    case OXO_AL5_XS: return oxo_dot_al5_xs_q8_0(row, blocks, act, NULL);
    case OXO_Q6_K:   return oxo_dot_q6_k_q8_k(row, blocks, act, NULL);
    case OXO_IQ3_S:  return oxo_dot_iq3_s_q8_k(row, blocks, act, NULL);
    case OXO_IQ1_XXXS: return oxo_dot_iq1_xxxs_q8_k(row, blocks, act, NULL);
    case OXO_Q2_K:   return oxo_dot_q2_k_q8_k(row, blocks, act, NULL);
    case OXO_Q3_K_S:
    case OXO_Q3_K_M:
    case OXO_Q3_K_L: return oxo_dot_q3_k_q8_k(row, blocks, act, NULL);
    case OXO_Q5_K_S:
    case OXO_Q5_K_M: return oxo_dot_q5_k_q8_k(row, blocks, act, NULL, NULL);
    default:         return oxo_dot_q4_k_q8_k(row, blocks, act, NULL, NULL);
    }
}

static void quantize(int kind, const float *x, size_t cols, uint8_t *out)
{
    if (kind == 2) oxo_quantize_q8_k(x, cols, out);
    else           oxo_quantize_q8_0(x, cols, out);
}

static size_t act_bytes_for(int kind, size_t cols)
{
    return n_blocks(kind, cols) * (kind == 2 ? OXO_Q8_K_BYTES : OXO_Q8_0_BYTES);
}

/* ─── entry points ────────────────────────────────────────────────────── */

int oxo_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp)
{
    const int kind = oxo_act_kind(qtype, cols);
    if (!kind || !oxo_stride_ok(qtype, cols, row_bytes) || temp == NULL)
        return 1;
    uint8_t *act = (uint8_t *)temp;
    quantize(kind, input, cols, act);
    const size_t blocks = n_blocks(kind, cols);
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; r++)
        output[r] = row_dot(qtype, data + (size_t)r * row_bytes, blocks, act);
    return 0;
}

int oxo_matvec_quantized_fused(const uint32_t *qtypes,
                               const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input,
                               float *const *outs, float *temp)
{
    /* The reference shares one activation quantisation when every matrix has
     * the same eligible type and otherwise calls the single entry point per
     * matrix; either way each output row is the same dot. */
    int rc = 0;
    for (size_t k = 0; k < n_outs; k++)
        rc |= oxo_matvec_quantized(qtypes[k], datas[k], rows[k], cols,
                                   row_bytes[k], input, outs[k], temp);
    return rc;
}

int oxo_matvec_quantized_multi_input(const uint32_t *qtypes,
                                     const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs,
                                     float *const *outs, float *temp)
{
    int rc = 0;
    for (size_t k = 0; k < n_outs; k++)
        rc |= oxo_matvec_quantized(qtypes[k], datas[k], rows[k], cols,
                                   row_bytes[k], inputs[k], outs[k], temp);
    return rc;
}

size_t oxo_matvec_batch_scratch_bytes(size_t max_cols)
{
    const size_t q8k = (max_cols / OXO_QK_K) * OXO_Q8_K_BYTES;
    const size_t nb0 = max_cols / OXO_QK8_0;
    /* Q8_0 activation plus the f32 scale tail one reference kernel appends:
     * blocks*34 rounded up to 4, then 4 bytes per block. */
    const size_t q80x = ((nb0 * OXO_Q8_0_BYTES + 3u) & ~(size_t)3u) + nb0 * 4u;
    const size_t one = q8k > q80x ? q8k : q80x;
    const size_t tile = (size_t)4u << 20;
    return one > tile ? one : tile;
}

int oxo_matvec_quantized_batch(uint32_t qtype, const uint8_t *data,
                               size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec,
                               uint8_t *act_scratch, size_t act_bytes)
{
    if (n_vec == 0 || rows == 0) return 0;
    const int kind = oxo_act_kind(qtype, cols);
    if (!kind || !oxo_stride_ok(qtype, cols, row_bytes)) return 1;
    const size_t ab = act_bytes_for(kind, cols);
    if (act_scratch == NULL || ab == 0 || act_bytes < ab) return 1;
    const size_t blocks = n_blocks(kind, cols);
    size_t tile = act_bytes / ab;
    if (tile > n_vec) tile = n_vec;
    for (size_t base = 0; base < n_vec; base += tile) {
        const size_t m = n_vec - base < tile ? n_vec - base : tile;
        for (size_t v = 0; v < m; v++)
            quantize(kind, inputs + (base + v) * in_stride, cols,
                     act_scratch + v * ab);
#pragma omp parallel for schedule(static)
        for (long r = 0; r < (long)rows; r++) {
            const uint8_t *row = data + (size_t)r * row_bytes;
            for (size_t v = 0; v < m; v++)
                outputs[(base + v) * out_stride + (size_t)r] =
                    row_dot(qtype, row, blocks, act_scratch + v * ab);
        }
    }
    return 0;
}

/* ─── MoE routing ─────────────────────────────────────────────────────── */

void oxo_moe_route(const float *logits, size_t n_tok, size_t n_expert,
                   size_t k, int renorm, int32_t *ids, float *weights)
{
    float *p = (float *)malloc(n_expert * sizeof(float));
    uint32_t *order = (uint32_t *)malloc(n_expert * sizeof(uint32_t));
    if (!p || !order) { free(p); free(order); return; }
    for (size_t t = 0; t < n_tok; t++) {
        const float *lg = logits + t * n_expert;
        float top = lg[0];
        for (size_t e = 1; e < n_expert; e++) if (lg[e] > top) top = lg[e];
        double z = 0.0;
        for (size_t e = 0; e < n_expert; e++) {
            p[e] = expf(lg[e] - top);
            z += (double)p[e];
        }
        if (z > 0.0) {
            const float inv = (float)(1.0 / z);
            for (size_t e = 0; e < n_expert; e++) p[e] *= inv;
        }
        /* partial selection sort on an index list, swapping as it goes */
        for (size_t e = 0; e < n_expert; e++) order[e] = (uint32_t)e;
        for (size_t i = 0; i < k; i++) {
            size_t best = i;
            for (size_t c = i + 1; c < n_expert; c++)
                if (p[order[c]] > p[order[best]]) best = c;
            const uint32_t tmp = order[i];
            order[i] = order[best];
            order[best] = tmp;
            ids[t * k + i] = (int32_t)order[i];
        }
        double norm = 1.0;
        if (renorm) {
            norm = 0.0;
            for (size_t i = 0; i < k; i++) norm += (double)p[ids[t * k + i]];
            if (norm <= 0.0) norm = 1.0;
        }
        for (size_t i = 0; i < k; i++)
            weights[t * k + i] = 1.0f * (float)(p[ids[t * k + i]] / norm);
    }
    free(p);
    free(order);
}

/* ─── float steps in front of the quantiser ───────────────────────────── */

void oxo_rms_norm_f32(const float *x, const float *weight, float *out, size_t n,
                      float eps)
{
    float ss = 0.0f;
    for (size_t i = 0; i < n; i++) ss += x[i] * x[i];
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (size_t i = 0; i < n; i++) out[i] = x[i] * inv * weight[i];
}

void oxo_swiglu_f32(const float *gate, const float *up, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        const float g = gate[i];
        const float sig = 1.0f / (1.0f + expf(-g));
        out[i] = g * sig * up[i];
    }
}

/* ─── dequantisation (layout cross-check only) ────────────────────────── */

/* src/compute/quant_tables.h:13-16 */
static const int8_t iq4_values[16] = { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 };

size_t oxo_dequant_path_row_bytes(uint32_t qtype, size_t cols)
{
    if (cols == 0) return 0;
    if (qtype == OXO_IQ4_NL) return cols % 32u ? 0 : cols / 32u * 18u;
    if (qtype == OXO_IQ4_XS) return cols % 256u ? 0 : cols / 256u * 136u;
    return 0;
}

/* src/compute/quantization.c:1401-1421 (IQ4_NL), :1429-1459 (IQ4_XS) */
static void dequant_iq4(uint32_t qtype, const uint8_t *row, size_t cols, float *out)
{
    if (qtype == OXO_IQ4_NL) {
        for (size_t b = 0; b < cols / 32u; b++) {
            const uint8_t *w = row + b * 18u;
            const float d = oxo_f16_to_f32(rd_u16(w));
            for (unsigned j = 0; j < 16; j++) {
                out[32 * b + j] = d * (float)iq4_values[w[2 + j] & 15u];
                out[32 * b + j + 16] = d * (float)iq4_values[w[2 + j] >> 4];
            }
        }
        return;
    }
    for (size_t b = 0; b < cols / 256u; b++) {
        const uint8_t *w = row + b * 136u;
        const float d = oxo_f16_to_f32(rd_u16(w));
        const uint32_t high = rd_u16(w + 2);
        for (unsigned ib = 0; ib < 8; ib++) {
            const int32_t lo4 = (w[4 + ib / 2] >> (4 * (ib % 2))) & 15;
            const int32_t hi2 = (int32_t)((high >> (2 * ib)) & 3u) << 4;
            const float dl = d * (float)((lo4 | hi2) - 32);
            for (unsigned j = 0; j < 16; j++) {
                const uint8_t q = w[8 + 16 * ib + j];
                out[256 * b + 32 * ib + j] = dl * (float)iq4_values[q & 15u];
                out[256 * b + 32 * ib + j + 16] = dl * (float)iq4_values[q >> 4];
            }
        }
    }
}

int oxo_matvec_dequant(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                       const float *x, double *out, double *mag)
{
    const size_t rb = oxo_dequant_path_row_bytes(qtype, cols);
    if (rb == 0 || row_bytes != rb) return 1;
    float *tmp = (float *)malloc(cols * sizeof *tmp);
    if (!tmp) return 2;
    for (size_t r = 0; r < rows; r++) {
        dequant_iq4(qtype, data + r * row_bytes, cols, tmp);
        double s = 0.0, m = 0.0;
        for (size_t i = 0; i < cols; i++) {
            const double t = (double)tmp[i] * (double)x[i];
            s += t;
            m += t < 0 ? -t : t;
        }
        out[r] = s;
        if (mag) mag[r] = m;
    }
    free(tmp);
    return 0;
}

int oxo_dequant_row(uint32_t qtype, const uint8_t *row, size_t cols, float *out)
{
    if (qtype == OXO_IQ4_NL || qtype == OXO_IQ4_XS) {
        if (oxo_dequant_path_row_bytes(qtype, cols) == 0) return 1;
        dequant_iq4(qtype, row, cols, out);
        return 0;
    }
    if (qtype == OXO_AL5) qtype = OXO_Q4_0;     /* src/compute/quantization.c:781-800 */
    if (qtype == OXO_AL6) qtype = OXO_Q5_0;
    if (qtype == OXO_AL8) qtype = OXO_Q8_0;
    const int kind = oxo_act_kind(qtype, cols);
    if (!kind) return 1;
    const size_t blocks = n_blocks(kind, cols);
    for (size_t b = 0; b < blocks; b++) {
        if (qtype == OXO_Q4_0 || qtype == OXO_Q4_1 || qtype == OXO_Q5_0 || qtype == OXO_Q5_1) {
            /* src/compute/quantization.c:386-474: value i is the low nibble of
             * byte i, value i + 16 the high nibble; fifth bit e of the 32-bit
             * word belongs to value e */
            const int has_m = qtype == OXO_Q4_1 || qtype == OXO_Q5_1;
            const int has_h = qtype == OXO_Q5_0 || qtype == OXO_Q5_1;
            const uint8_t *w = row + b * block_bytes(qtype);
            const float d = oxo_f16_to_f32(rd_u16(w));
            const float m = has_m ? oxo_f16_to_f32(rd_u16(w + 2)) : 0.0f;
            const uint8_t *qh = w + (has_m ? 4 : 2);
            const uint8_t *qs = qh + (has_h ? 4 : 0);
            const uint32_t bits = has_h ? ((uint32_t)qh[0] | ((uint32_t)qh[1] << 8) |
                                           ((uint32_t)qh[2] << 16) | ((uint32_t)qh[3] << 24)) : 0u;
            for (unsigned e = 0; e < 32; e++) {
                const unsigned nib = e < 16 ? (qs[e] & 15u) : (unsigned)(qs[e - 16] >> 4);
                const unsigned code = nib | (((bits >> e) & 1u) << 4);
                if (has_m) out[32 * b + e] = (float)code * d + m;
                else       out[32 * b + e] = (float)((int)code - (has_h ? 16 : 8)) * d;
            }
        } else if (qtype == OXO_AL5_XS) {
            /* src/compute/quantization.c:802-832 */
            const uint8_t *w = row + b * OXO_AL5_XS_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w));
            for (unsigned i = 0; i < 32; i++)
                out[32 * b + i] = (float)((int32_t)al5_xs_code(w + 2, i) - 4) * d;
        } else if (qtype == OXO_Q2_K) {
            /* src/compute/quantization.c:521-561 */
            const uint8_t *w = row + b * OXO_Q2_K_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w + 80));
            const float mn = oxo_f16_to_f32(rd_u16(w + 82));
            for (unsigned e = 0; e < 256; e++) {
                const float dl = d * (float)(w[e >> 4] & 15u);
                const float ml = mn * (float)(w[e >> 4] >> 4);
                out[256 * b + e] = dl * (float)q23_code(w + 16, NULL, e) - ml;
            }
        } else if (qtype == OXO_Q3_K_S || qtype == OXO_Q3_K_M || qtype == OXO_Q3_K_L) {
            /* src/compute/quantization.c:563-630 */
            const uint8_t *w = row + b * OXO_Q3_K_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w + 108));
            int8_t sc[16];
            q3k_scales(w + 96, sc);
            for (unsigned e = 0; e < 256; e++) {
                const float dl = d * (float)sc[e >> 4];
                out[256 * b + e] = dl * (float)((int)q23_code(w + 32, w, e) - 4);
            }
        } else if (qtype == OXO_Q8_0) {
            const uint8_t *w = row + b * OXO_Q8_0_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w));
            for (int i = 0; i < 32; i++)
                out[32 * b + i] = (float)(int8_t)w[2 + i] * d;
        } else if (qtype == OXO_Q6_K) {
            const uint8_t *w = row + b * OXO_Q6_K_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w + 208));
            const int8_t *sc = (const int8_t *)(w + 192);
            for (int e = 0; e < 256; e++) {
                const int n = e >> 7, k = (e >> 5) & 3, l = e & 31;
                const unsigned lo = w[64 * n + 32 * (k & 1) + l];
                const unsigned hi = w[128 + 32 * n + l];
                const int code = (int)((k < 2 ? (lo & 15u) : (lo >> 4)) |
                                       (((hi >> (2 * k)) & 3u) << 4)) - 32;
                out[256 * b + e] = d * (float)sc[e >> 4] * (float)code;
            }
        } else if (qtype == OXO_Q5_K_S || qtype == OXO_Q5_K_M) {
            const uint8_t *w = row + b * OXO_Q5_K_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w));
            const float dmin = oxo_f16_to_f32(rd_u16(w + 2));
            uint8_t sc[8], mn[8];
            for (unsigned j = 0; j < 8; j++)
                oxo_scale_min_k4(j, w + 4, &sc[j], &mn[j]);
            for (int e = 0; e < 256; e++) {
                const int j = e >> 5, l = e & 31;
                const unsigned byte = w[48 + 32 * (j >> 1) + l];
                const unsigned code = ((j & 1) ? (byte >> 4) : (byte & 15u)) +
                                      (((w[16 + l] >> j) & 1u) ? 16u : 0u);
                const float ds = d * (float)sc[j];
                const float ms = dmin * (float)mn[j];
                out[256 * b + e] = ds * (float)code - ms;
            }
        } else {
            const uint8_t *w = row + b * OXO_Q4_K_BYTES;
            const float d = oxo_f16_to_f32(rd_u16(w));
            const float dmin = oxo_f16_to_f32(rd_u16(w + 2));
            uint8_t sc[8], mn[8];
            for (unsigned j = 0; j < 8; j++)
                oxo_scale_min_k4(j, w + 4, &sc[j], &mn[j]);
            for (int e = 0; e < 256; e++) {
                const int j = e >> 5, l = e & 31;
                const unsigned byte = w[16 + 32 * (j >> 1) + l];
                const unsigned code = (j & 1) ? (byte >> 4) : (byte & 15u);
                const float ds = d * (float)sc[j];
                const float ms = dmin * (float)mn[j];
                out[256 * b + e] = ds * (float)code - ms;
            }
        }
    }
    return 0;
}

/* ─── MoE feed-forward ────────────────────────────────────────────────── */

int oxo_moe_ffn(uint32_t qtype_gate_up, uint32_t qtype_down, const uint8_t *w_gate,
                const uint8_t *w_up, const uint8_t *w_down, size_t n_expert, size_t k,
                size_t hidden, size_t ffn, int renorm, const float *logits,
                const float *x, size_t n_tok, float *out)
{
    const size_t rb_gu = n_blocks(oxo_act_kind(qtype_gate_up, hidden), hidden) * block_bytes(qtype_gate_up);
    const size_t rb_dn = n_blocks(oxo_act_kind(qtype_down, ffn), ffn) * block_bytes(qtype_down);
    int32_t *ids = (int32_t *)malloc(n_tok * k * sizeof(int32_t));
    float *wts = (float *)malloc(n_tok * k * sizeof(float));
    float *gate = (float *)malloc(ffn * sizeof(float));
    float *up = (float *)malloc(ffn * sizeof(float));
    float *down = (float *)malloc(hidden * sizeof(float));
    float *temp = (float *)malloc(((hidden > ffn ? hidden : ffn) / 256u + 1u) * 296u);
    int rc = 1;
    if (!ids || !wts || !gate || !up || !down || !temp) goto done;
    oxo_moe_route(logits, n_tok, n_expert, k, renorm, ids, wts);
    memset(out, 0, n_tok * hidden * sizeof(float));
    rc = 0;
    /* experts in ascending order, each over its tokens in token order: what
     * the counting sort plus the per-expert pass amount to */
    for (size_t e = 0; e < n_expert && !rc; e++)
        for (size_t t = 0; t < n_tok && !rc; t++)
            for (size_t j = 0; j < k; j++) {
                if ((size_t)ids[t * k + j] != e) continue;
                const float *xt = x + t * hidden;
                rc |= oxo_matvec_quantized(qtype_gate_up, w_gate + e * ffn * rb_gu, ffn, hidden, rb_gu, xt, gate, temp);
                rc |= oxo_matvec_quantized(qtype_gate_up, w_up + e * ffn * rb_gu, ffn, hidden, rb_gu, xt, up, temp);
                oxo_swiglu_f32(gate, up, gate, ffn);
                rc |= oxo_matvec_quantized(qtype_down, w_down + e * hidden * rb_dn, hidden, ffn, rb_dn, gate, down, temp);
                const float w = wts[t * k + j];
                float *dst = out + t * hidden;
                for (size_t i = 0; i < hidden; i++) dst[i] += w * down[i];
            }
done:
    free(ids); free(wts); free(gate); free(up); free(down); free(temp);
    return rc;
}
