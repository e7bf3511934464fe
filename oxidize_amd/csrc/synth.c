/*
 * synth.c — seeded synthetic tensors for the quantized-matvec benchmarks and
 * tests: raw Q4_K / Q5_K / Q6_K / Q8_0 weight blocks and f32 activations.
 *
 * Everything is integer arithmetic plus exactly-representable float steps, so
 * the same (seed, stream, index) yields the same bits on every machine and at
 * any thread count; no libm is involved.
 *
 *   uniform bits : splitmix64 seeded per block from (seed, stream, block)
 *   N(0,1)       : Irwin-Hall, sum of twelve 16-bit uniforms, centred, / 2^16
 *   f16 scales   : |N(0,sigma)| rounded to binary16 (round-to-nearest-even)
 *
 * Block contents follow the layouts the kernels consume (GGUF):
 *   Q4_K 144 B: f16 d, f16 dmin, 12 B packed 6-bit scales/mins, 128 B nibbles
 *   Q5_K 176 B: f16 d, f16 dmin, 12 B packed 6-bit scales/mins, 32 B fifth-bit
 *               plane, 128 B nibbles
 *   Q6_K 210 B: 128 B ql, 64 B qh, 16 int8 scales, f16 d
 *   Q8_0  34 B: f16 d, 32 int8
 *   Q4_0 18 B / Q4_1 20 B / Q5_0 22 B / Q5_1 24 B: f16 d [, f16 m][, 32 fifth
 *               bits], 16 B nibbles
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

typedef struct { uint64_t s; } Rng;

static inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint64_t next64(Rng *r)
{
    r->s += 0x9E3779B97F4A7C15ull;
    return mix64(r->s);
}

static inline Rng rng_for(uint64_t seed, uint64_t stream, uint64_t index)
{
    Rng r;
    r.s = mix64(seed ^ mix64(stream * 0xD1B54A32D192ED03ull + 0x8CB92BA72F3D8DD7ull))
          + index * 0xA0761D6478BD642Full;
    r.s = mix64(r.s);
    return r;
}

/* N(0,1) approximation with support (-6, 6); exact in binary32. */
static inline float normal(Rng *r)
{
    uint32_t acc = 0;
    for (int k = 0; k < 3; k++) {
        const uint64_t u = next64(r);
        acc += (uint32_t)(u & 0xFFFF) + (uint32_t)((u >> 16) & 0xFFFF) +
               (uint32_t)((u >> 32) & 0xFFFF) + (uint32_t)(u >> 48);
    }
    return (float)((int32_t)acc - 393210) * (1.0f / 65536.0f);
}

/* binary32 -> binary16, round to nearest even, for finite non-negative
 * inputs below 65504 (all this file produces). */
static inline uint16_t f16_rne(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t e = (u >> 23) & 0xFF;
    uint32_t m = u & 0x7FFFFF;
    if (e < 103) return 0;                       /* < 2^-24 / 2 */
    if (e < 113) {                               /* subnormal half */
        m |= 0x800000;
        const uint32_t sh = 126 - e;             /* 14..23 */
        uint32_t q = m >> sh;
        const uint32_t rem = m & ((1u << sh) - 1u);
        const uint32_t half = 1u << (sh - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)q;
    }
    uint32_t q = ((e - 112) << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFF;
    if (rem > 0x1000 || (rem == 0x1000 && (q & 1u))) q++;
    return (uint16_t)q;
}

static inline uint16_t half_abs_normal(Rng *r, float sigma)
{
    float z = normal(r) * sigma;
    if (z < 0.0f) z = -z;
    return f16_rne(z);
}

static inline void put16(uint8_t *p, uint16_t v)
{
    p[0] = (uint8_t)(v & 0xFF);
    p[1] = (uint8_t)(v >> 8);
}

/* rows*blocks_per_row Q4_K blocks.  d, dmin ~ |N(0,sigma)|; eight 6-bit scales
 * and eight 6-bit mins uniform in [0,63]; nibbles uniform. */
void oxs_fill_q4_k(uint8_t *dst, size_t n_blocks, uint64_t seed,
                   uint64_t stream, float sigma)
{
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * 144u;
        put16(blk, half_abs_normal(&r, sigma));
        put16(blk + 2, half_abs_normal(&r, sigma));
        uint8_t sc[8], mn[8];
        uint64_t u = next64(&r), v = next64(&r);
        for (int j = 0; j < 8; j++) {
            sc[j] = (uint8_t)((u >> (6 * j)) & 63u);
            mn[j] = (uint8_t)((v >> (6 * j)) & 63u);
        }
        uint8_t *s = blk + 4;
        for (int j = 0; j < 4; j++) {
            s[j]     = (uint8_t)(sc[j] | ((sc[j + 4] >> 4) << 6));
            s[j + 4] = (uint8_t)(mn[j] | ((mn[j + 4] >> 4) << 6));
            s[j + 8] = (uint8_t)((sc[j + 4] & 15u) | ((mn[j + 4] & 15u) << 4));
        }
        for (int i = 0; i < 16; i++) {
            const uint64_t w = next64(&r);
            memcpy(blk + 16 + 8 * i, &w, 8);
        }
    }
}

/* Q5_K blocks: the Q4_K header, then 32 bytes of fifth bits and 128 bytes of
 * nibbles, all uniform (codes uniform in [0,31]). */
void oxs_fill_q5_k(uint8_t *dst, size_t n_blocks, uint64_t seed,
                   uint64_t stream, float sigma)
{
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * 176u;
        put16(blk, half_abs_normal(&r, sigma));
        put16(blk + 2, half_abs_normal(&r, sigma));
        uint8_t sc[8], mn[8];
        uint64_t u = next64(&r), v = next64(&r);
        for (int j = 0; j < 8; j++) {
            sc[j] = (uint8_t)((u >> (6 * j)) & 63u);
            mn[j] = (uint8_t)((v >> (6 * j)) & 63u);
        }
        uint8_t *s = blk + 4;
        for (int j = 0; j < 4; j++) {
            s[j]     = (uint8_t)(sc[j] | ((sc[j + 4] >> 4) << 6));
            s[j + 4] = (uint8_t)(mn[j] | ((mn[j + 4] >> 4) << 6));
            s[j + 8] = (uint8_t)((sc[j + 4] & 15u) | ((mn[j + 4] & 15u) << 4));
        }
        for (int i = 0; i < 20; i++) {
            const uint64_t w = next64(&r);
            memcpy(blk + 16 + 8 * i, &w, 8);
        }
    }
}

/* Q6_K blocks: codes uniform in [0,63] (ql/qh bytes uniform), int8 scales
 * uniform in [-32,31], d ~ |N(0,sigma)|. */
void oxs_fill_q6_k(uint8_t *dst, size_t n_blocks, uint64_t seed,
                   uint64_t stream, float sigma)
{
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * 210u;
        for (int i = 0; i < 24; i++) {
            const uint64_t w = next64(&r);
            memcpy(blk + 8 * i, &w, 8);
        }
        const uint64_t a = next64(&r), c = next64(&r);
        for (int g = 0; g < 8; g++) {
            blk[192 + g] = (uint8_t)(int8_t)((int)((a >> (8 * g)) & 63u) - 32);
            blk[200 + g] = (uint8_t)(int8_t)((int)((c >> (8 * g)) & 63u) - 32);
        }
        put16(blk + 208, half_abs_normal(&r, sigma));
    }
}

/* Q2_K (84 B: 16 scale|min bytes, 64 code bytes, f16 d, f16 dmin) and Q3_K
 * (110 B: 32 third-bit bytes, 64 code bytes, 12 scale bytes, f16 d): every
 * payload byte uniform, the f16 scales ~ |N(0,sigma)|. */
void oxs_fill_q23_k(uint8_t *dst, size_t n_blocks, uint64_t seed, uint64_t stream, float sigma,
                    int is_q3)
{
    const size_t bytes = is_q3 ? 110u : 84u;
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * bytes;
        uint8_t raw[112];
        for (int i = 0; i < 14; i++) {
            const uint64_t w = next64(&r);
            memcpy(raw + 8 * i, &w, 8);
        }
        memcpy(blk, raw, bytes);
        if (is_q3) {
            put16(blk + 108, half_abs_normal(&r, sigma));
        } else {
            put16(blk + 80, half_abs_normal(&r, sigma));
            put16(blk + 82, half_abs_normal(&r, sigma));
        }
    }
}

/* Q8_0 blocks: int8 uniform in [-127,127], d ~ |N(0,sigma)|. */
void oxs_fill_q8_0(uint8_t *dst, size_t n_blocks, uint64_t seed,
                   uint64_t stream, float sigma)
{
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * 34u;
        put16(blk, half_abs_normal(&r, sigma));
        for (int i = 0; i < 32; i += 4) {
            const uint64_t w = next64(&r);
            for (int k = 0; k < 4; k++)
                blk[2 + i + k] =
                    (uint8_t)(int8_t)((int)(((w >> (16 * k)) & 0xFFFFu) % 255u) - 127);
        }
    }
}

/* The 32-value formats Q4_0 (18 B), Q4_1 (20 B), Q5_0 (22 B), Q5_1 (24 B):
 * f16 d (and f16 m when has_min) ~ |N(0,sigma)|, every other byte uniform. */
void oxs_fill_legacy(uint8_t *dst, size_t n_blocks, uint64_t seed, uint64_t stream,
                     float sigma, uint32_t block_bytes, int has_min)
{
#pragma omp parallel for schedule(static)
    for (long b = 0; b < (long)n_blocks; b++) {
        Rng r = rng_for(seed, stream, (uint64_t)b);
        uint8_t *blk = dst + (size_t)b * block_bytes;
        put16(blk, half_abs_normal(&r, sigma));
        uint32_t at = 2;
        if (has_min) { put16(blk + 2, half_abs_normal(&r, sigma)); at = 4; }
        uint64_t w = 0;
        for (uint32_t i = at, k = 0; i < block_bytes; i++, k++) {
            if ((k & 7u) == 0u) w = next64(&r);
            blk[i] = (uint8_t)(w >> (8u * (k & 7u)));
        }
    }
}

/* n f32 values ~ N(0,1) * scale.  Indexed in chunks of 256 so the result does
 * not depend on the thread count. */
void oxs_fill_normal_f32(float *dst, size_t n, uint64_t seed, uint64_t stream,
                         float scale)
{
    const size_t chunks = (n + 255u) / 256u;
#pragma omp parallel for schedule(static)
    for (long c = 0; c < (long)chunks; c++) {
        Rng r = rng_for(seed, stream, (uint64_t)c);
        const size_t lo = (size_t)c * 256u;
        const size_t hi = lo + 256u < n ? lo + 256u : n;
        for (size_t i = lo; i < hi; i++) dst[i] = normal(&r) * scale;
    }
}
