/*
 * oxh_kernels.hip — gfx950 kernels and the thin device-resident C ABI of
 * liboxhip (layer 2 of include/oxhip.h).
 *
 * Arithmetic contract (all paths relative to the reference checkout):
 *   Q8_K / Q8_0 activation bytes  oxidize-c/src/compute/matvec.c:276-316, :130-155
 *   f32 -> f16 (round half up)    oxidize-c/src/compute/flash_attention.c:149-185
 *   Q4_K x Q8_K block dot         oxidize-c/src/compute/oxk.c:243-297
 *   Q6_K x Q8_K block dot         oxidize-c/src/compute/oxk.c:913-964
 *   Q8_0 x Q8_0 block dot         oxidize-c/src/compute/oxk.c:224-241
 *
 * All integer sums are exact, so they may be formed in any order.  The f32
 * part keeps the reference's order: one term per block, rounded exactly as
 * `dw*dq*(float)pos - dmin*dq*(float)min_acc`, then a strictly sequential sum
 * over the blocks of a row starting from 0.0f.  Float contraction is disabled
 * for this file (build flag -ffp-contract=off and the pragma below).
 *
 * Wave64 only.  Build: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off
 *   -Xclang -target-feature -Xclang -packed-fp32-ops
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "oxhip.h"
#include "oxh_internal.h"

#pragma clang fp contract(off)

/* ─── error plumbing ──────────────────────────────────────────────────── */

static thread_local char g_err[512] = "";

extern "C" const char *oxh_last_error(void) { return g_err; }

extern "C" void oxh_set_error(const char *fmt, const char *a, const char *b)
{
    snprintf(g_err, sizeof g_err, fmt, a ? a : "", b ? b : "");
}

static int hip_fail(hipError_t e, const char *what)
{
    snprintf(g_err, sizeof g_err, "HIP error in %s: %s", what, hipGetErrorString(e));
    return OXH_ERR_HIP;
}

#define HIP_TRY(call)                                                          \
    do {                                                                       \
        hipError_t e_ = (call);                                                \
        if (e_ != hipSuccess) return hip_fail(e_, #call);                      \
    } while (0)

static int arg_fail(const char *what)
{
    snprintf(g_err, sizeof g_err, "invalid argument: %s", what);
    return OXH_ERR_ARG;
}

/* ─── small device helpers ────────────────────────────────────────────── */

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

/* 16-byte vector with only 2-byte alignment: Q6_K (210 B) and Q8_0 (34 B)
 * blocks start on even addresses.  gfx9+ under HSA runs with unaligned
 * global access enabled, and the compiler emits one global_load_dwordx4. */
struct __attribute__((packed, aligned(2))) U32x4u2 { uint32_t x, y, z, w; };
struct __attribute__((packed, aligned(2))) U32u2 { uint32_t v; };

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c)
{
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

/* Sum over the four lanes of a quad; every lane receives the total. */
__device__ __forceinline__ int quad_sum(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false); /* lanes ^1 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false); /* lanes ^2 */
    return v;
}

/* Exact binary16 -> binary32 including subnormals (integer-only so it does
 * not depend on the wave's denormal mode). */
__device__ __forceinline__ float half_bits_to_float(uint32_t h)
{
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 31u;
    const uint32_t m = h & 0x3FFu;
    uint32_t bits;
    if (e == 31u) {
        bits = sign | 0x7F800000u | (m << 13);
    } else if (e != 0u) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        bits = sign;
    } else {
        const uint32_t lz = (uint32_t)__clz((int)m) - 21u;   /* shifts to bit 10 */
        bits = sign | ((113u - lz) << 23) | (((m << lz) & 0x3FFu) << 13);
    }
    return __uint_as_float(bits);
}

/* binary32 -> binary16 bits, round-half-UP on the dropped bits
 * (flash_attention.c:149-185). */
__device__ __forceinline__ uint32_t float_to_half_bits_half_up(float v)
{
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e32 = (int)((u >> 23) & 0xFFu);
    const uint32_t man = u & 0x7FFFFFu;
    if (e32 == 255) {
        if (man == 0u) return sign | 0x7C00u;
        uint32_t payload = man >> 13;
        if (payload == 0u) payload = 1u;
        return sign | 0x7C00u | payload;
    }
    const int e16 = e32 - 112;
    if (e16 >= 31) return sign | 0x7C00u;
    if (e16 >= 1) {
        uint32_t out = ((uint32_t)e16 << 10) | (man >> 13);
        if (man & 0x1000u) {
            out += 1u;
            if (out >= 0x7C00u) return sign | 0x7C00u;
        }
        return sign | out;
    }
    if (e16 < -10) return sign;
    const uint32_t full = man | 0x800000u;
    const uint32_t sh = (uint32_t)(14 - e16);
    uint32_t out = full >> sh;
    if ((full >> (sh - 1u)) & 1u) out += 1u;
    return sign | out;
}

__device__ __forceinline__ int quantize_one(float x, float inv)
{
    /* lrintf under round-to-nearest-even == v_rndne_f32 + convert */
    int v = (int)rintf(x * inv);
    v = v > 127 ? 127 : v;
    v = v < -128 ? -128 : v;
    return v;
}

/* ─── activation quantisers ───────────────────────────────────────────── */

/* One wave per 256-value block; lane l owns values 4l..4l+3. */
__global__ __launch_bounds__(256) void
k_quantize_q8_k(const float *__restrict__ x, size_t in_stride, uint32_t blocks_per_vec,
                uint32_t total_blocks, uint8_t *__restrict__ act)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t gb = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (gb >= total_blocks) return;
    const uint32_t vec = gb / blocks_per_vec;
    const uint32_t blk = gb - vec * blocks_per_vec;
    const float *src = x + (size_t)vec * in_stride + (size_t)blk * 256u + 4u * lane;
    const float v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];

    /* max |x| over the block; NaNs never win a '>' comparison in the
     * reference's scan, fmaxf drops them the same way */
    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));

    const float d = amax / 127.0f;
    const float inv = (d != 0.0f) ? 1.0f / d : 0.0f;
    const int q0 = quantize_one(v0, inv), q1 = quantize_one(v1, inv);
    const int q2 = quantize_one(v2, inv), q3 = quantize_one(v3, inv);

    uint8_t *dst = act + (size_t)gb * OXH_Q8_K_BYTES;
    const uint32_t packed = (uint32_t)(q0 & 255) | ((uint32_t)(q1 & 255) << 8) |
                            ((uint32_t)(q2 & 255) << 16) | ((uint32_t)(q3 & 255) << 24);
    reinterpret_cast<uint32_t *>(dst + 4)[lane] = packed;
    if (lane == 0) *reinterpret_cast<float *>(dst) = d;

    const int s = quad_sum(q0 + q1 + q2 + q3);   /* 16 values = one bsum group */
    if ((lane & 3u) == 0u)
        reinterpret_cast<int16_t *>(dst + 260)[lane >> 2] = (int16_t)s;
}

/* One wave per 8 blocks of 32 values; lane l owns values 4l..4l+3 of the
 * 256-value span, i.e. 8 lanes per block. */
__global__ __launch_bounds__(256) void
k_quantize_q8_0(const float *__restrict__ x, size_t in_stride, uint32_t blocks_per_vec,
                uint32_t n_vec, uint8_t *__restrict__ act)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t spans_per_vec = (blocks_per_vec + 7u) / 8u;
    const uint32_t gs = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (gs >= spans_per_vec * n_vec) return;
    const uint32_t vec = gs / spans_per_vec;
    const uint32_t span = gs - vec * spans_per_vec;
    const uint32_t blk = span * 8u + (lane >> 3);
    const bool live = blk < blocks_per_vec;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
    if (live) {
        const float *src = x + (size_t)vec * in_stride + (size_t)blk * 32u + 4u * (lane & 7u);
        v0 = src[0]; v1 = src[1]; v2 = src[2]; v3 = src[3];
    }
    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
#pragma unroll
    for (int m = 4; m >= 1; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    const float d = amax / 127.0f;
    const float inv = (d != 0.0f) ? 1.0f / d : 0.0f;
    const int q0 = quantize_one(v0, inv), q1 = quantize_one(v1, inv);
    const int q2 = quantize_one(v2, inv), q3 = quantize_one(v3, inv);
    if (!live) return;
    uint8_t *dst = act + ((size_t)vec * blocks_per_vec + blk) * OXH_Q8_0_BYTES;
    /* the block starts on an even address only: 16-bit stores */
    uint16_t *q16 = reinterpret_cast<uint16_t *>(dst + 2 + 4u * (lane & 7u));
    q16[0] = (uint16_t)((q0 & 255) | ((q1 & 255) << 8));
    q16[1] = (uint16_t)((q2 & 255) | ((q3 & 255) << 8));
    if ((lane & 7u) == 0u)
        *reinterpret_cast<uint16_t *>(dst) = (uint16_t)float_to_half_bits_half_up(d);
}

/* ─── decode GEMV ─────────────────────────────────────────────────────── */

#define OXH_MAX_SEGS 32
#define OXH_GEMV_WAVES 4          /* waves per workgroup */
#define OXH_MAX_NV 8

/* Bytes of LDS one staged Q8_K activation takes: 256 B of values, 16 B of
 * sub-block sums and 4 B of scale per block, rounded up so the next
 * activation's 16-byte vectors stay aligned. */
__host__ __device__ static inline uint32_t q8k_lds_bytes(uint32_t blocks)
{
    return (blocks * (256u + 16u + 4u) + 15u) & ~15u;
}

/* Q6_K pairing: 256 B of values, 16 x int32 pre-scaled group sums, scale. */
__host__ __device__ static inline uint32_t q8k6_lds_bytes(uint32_t blocks)
{
    return (blocks * (256u + 64u + 4u) + 15u) & ~15u;
}

/* Q8_0 activation: 32 B of values and the decoded f32 scale per block. */
__host__ __device__ static inline uint32_t q80_lds_bytes(uint32_t blocks)
{
    return (blocks * (32u + 4u) + 15u) & ~15u;
}

struct SegTable {
    const uint8_t *w[OXH_MAX_SEGS];
    float *out[OXH_MAX_SEGS];
    uint32_t rows[OXH_MAX_SEGS];
    uint32_t act_first[OXH_MAX_SEGS];
    uint32_t wg_begin[OXH_MAX_SEGS + 1];   /* first workgroup of each segment */
    uint32_t n;
};

struct GemvParams {
    uint32_t blocks;        /* weight blocks per row                        */
    uint32_t magic;         /* ceil(2^32 / blocks), for g / blocks          */
    uint32_t rows_per_wave; /* RW                                           */
    uint32_t n_vec;         /* activations per segment (1..8)               */
    uint32_t act_bytes;     /* bytes of one quantised activation            */
    uint32_t out_stride;    /* floats between output vectors                */
    uint32_t term_stride;   /* blocks + 1 (LDS row pitch of the term table) */
    int32_t *dump;          /* debug: sub-block sums, or NULL               */
};

/* LDS layout for the Q8_K-activation kernels (per workgroup), in this order:
 *   per activation v: q  [4][blocks*4] x 16 B   values of (block, 64-span s),
 *                        quarter i, at ((i*blocks*4) + block*4 + s)
 *                     bs [blocks*4]   x 4 B    Q4_K: B_{2s} | B_{2s+1}<<16
 *                     dq [blocks]     x 4 B
 *   terms: [waves][n_vec][rows_per_wave][term_stride] f32
 * For Q6_K the q array is indexed by (block, unit u=(n,lh)), quarter k, and
 * bs holds 4 x int32 per unit (32*bsum of its 4 groups), see k_gemv_q6_k. */

__device__ __forceinline__ uint32_t find_segment(const SegTable &t, uint32_t wg)
{
    uint32_t s = 0;
    while (s + 1 < t.n && wg >= t.wg_begin[s + 1]) s++;
    return s;
}

__device__ __forceinline__ void
row_sums(const float *terms, uint32_t lane, uint32_t NV, uint32_t nrows, uint32_t RW,
         uint32_t B, uint32_t term_stride, float *out, uint32_t out_stride, uint32_t row0);

/* Q4_K x Q8_K.  Four lanes per super-block: lane (b, s) owns nibble bytes
 * [32s, 32s+32) of block b, i.e. sub-blocks 2s (low nibbles) and 2s+1 (high
 * nibbles), elements [64s, 64s+64).  16 blocks = 2304 contiguous bytes per
 * wave pass. */
template <bool DUMP>
__global__ __launch_bounds__(OXH_GEMV_WAVES * 64) void
k_gemv_q4_k(const SegTable segs, const GemvParams p, const uint8_t *__restrict__ acts)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t B = p.blocks;
    const uint32_t NV = p.n_vec;

    const uint32_t seg = find_segment(segs, blockIdx.x);
    const uint32_t wg_in_seg = blockIdx.x - segs.wg_begin[seg];
    const uint32_t seg_rows = segs.rows[seg];

    const uint32_t act_lds = q8k_lds_bytes(B);               /* per activation */
    float *const terms = reinterpret_cast<float *>(lds + (size_t)act_lds * NV) +
                         (size_t)wave * NV * p.rows_per_wave * p.term_stride;

    /* stage the segment's activations */
    for (uint32_t v = 0; v < NV; v++) {
        const uint8_t *a = acts + (size_t)(segs.act_first[seg] + v) * p.act_bytes;
        uint8_t *base = lds + (size_t)v * act_lds;
        uint32_t *qd = reinterpret_cast<uint32_t *>(base);
        uint32_t *bs = reinterpret_cast<uint32_t *>(base + B * 256u);
        float *dq = reinterpret_cast<float *>(base + B * 256u + B * 16u);
        for (uint32_t j = tid; j < B * 64u; j += OXH_GEMV_WAVES * 64u) {
            const uint32_t blk = j >> 6, w = j & 63u;
            const uint32_t c = w >> 2, s = c >> 2, i = c & 3u;
            const uint32_t val = *reinterpret_cast<const uint32_t *>(a + (size_t)blk * 292u + 4u + 4u * w);
            qd[((i * B * 4u) + blk * 4u + s) * 4u + (w & 3u)] = val;
        }
        for (uint32_t j = tid; j < B * 4u; j += OXH_GEMV_WAVES * 64u) {
            const uint32_t blk = j >> 2, s = j & 3u;
            const uint32_t *sp = reinterpret_cast<const uint32_t *>(a + (size_t)blk * 292u + 260u) + 2u * s;
            const uint32_t p0 = sp[0], p1 = sp[1];
            const int b0 = (int)(int16_t)(p0 & 0xFFFFu) + (int)(int16_t)(p0 >> 16);
            const int b1 = (int)(int16_t)(p1 & 0xFFFFu) + (int)(int16_t)(p1 >> 16);
            bs[j] = ((uint32_t)b0 & 0xFFFFu) | ((uint32_t)b1 << 16);
        }
        for (uint32_t j = tid; j < B; j += OXH_GEMV_WAVES * 64u)
            dq[j] = *reinterpret_cast<const float *>(a + (size_t)j * 292u);
    }
    __syncthreads();

    const uint32_t RW = p.rows_per_wave;
    const uint32_t row0 = (wg_in_seg * OXH_GEMV_WAVES + wave) * RW;
    if (row0 >= seg_rows) return;
    const uint32_t nrows = min(RW, seg_rows - row0);
    const uint32_t nblk = nrows * B;
    const uint32_t s = lane & 3u;
    const bool hi = s >= 2u;
    const uint32_t sh = (s & 1u) * 16u;
    const uint32_t mask_a = hi ? 0x0F0F0F0Fu : 0x3F3F3F3Fu;
    const uint32_t mask_b = hi ? 0x30303030u : 0u;

    const uint8_t *wbase = segs.w[seg] + (size_t)row0 * B * 144u;

    for (uint32_t g0 = 0; g0 < nblk; g0 += 16u) {
        const uint32_t g = g0 + (lane >> 2);
        const bool live = g < nblk;
        const uint32_t gc = live ? g : 0u;
        const uint32_t r = (B == 1u) ? gc : __umulhi(gc, p.magic);
        const uint32_t blk = gc - r * B;
        const uint8_t *wb = wbase + (size_t)gc * 144u;
        const u32x4 hdr = *reinterpret_cast<const u32x4 *>(wb);
        const u32x4 na = *reinterpret_cast<const u32x4 *>(wb + 16u + 32u * s);
        const u32x4 nb = *reinterpret_cast<const u32x4 *>(wb + 32u + 32u * s);

        /* 6-bit scale/min unpack for this lane's two sub-blocks */
        const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
        const uint32_t scw = ((hi ? u2 : u0) & mask_a) | ((u0 >> 2) & mask_b);
        const uint32_t mnw = ((hi ? (u2 >> 4) : u1) & mask_a) | ((u1 >> 2) & mask_b);
        const int sc_a = (int)((scw >> sh) & 0xFFu), sc_b = (int)((scw >> (sh + 8u)) & 0xFFu);
        const int mn_a = (int)((mnw >> sh) & 0xFFu), mn_b = (int)((mnw >> (sh + 8u)) & 0xFFu);
        const float dw = half_bits_to_float(hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_float(hdr.x >> 16);

        const uint32_t slot = blk * 4u + s;
        for (uint32_t v = 0; v < NV; v++) {
            const uint8_t *base = lds + (size_t)v * act_lds;
            const u32x4 *qv = reinterpret_cast<const u32x4 *>(base);
            const u32x4 a0 = qv[slot], a1 = qv[B * 4u + slot];
            const u32x4 a2 = qv[B * 8u + slot], a3 = qv[B * 12u + slot];
            const uint32_t bsp = reinterpret_cast<const uint32_t *>(base + B * 256u)[slot];
            const float dq = reinterpret_cast<const float *>(base + B * 256u + B * 16u)[blk];

            int s_lo = 0, s_hi = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                s_lo = dot4(na[k] & 0x0F0F0F0Fu, a0[k], s_lo);
                s_lo = dot4(nb[k] & 0x0F0F0F0Fu, a1[k], s_lo);
                s_hi = dot4((na[k] >> 4) & 0x0F0F0F0Fu, a2[k], s_hi);
                s_hi = dot4((nb[k] >> 4) & 0x0F0F0F0Fu, a3[k], s_hi);
            }
            if (DUMP) {
                if (live) {
                    int32_t *o = p.dump + ((size_t)(row0 * B + gc)) * 8u + 2u * s;
                    o[0] = s_lo;
                    o[1] = s_hi;
                }
            }
            int pos = sc_a * s_lo + sc_b * s_hi;
            int mn = mn_a * (int)(int16_t)(bsp & 0xFFFFu) + mn_b * ((int)bsp >> 16);
            pos = quad_sum(pos);
            mn = quad_sum(mn);
            const float t_pos = dw * dq;
            const float t_min = dmin * dq;
            const float up = t_pos * (float)pos;
            const float dn = t_min * (float)mn;
            if (live && s == 0u)
                terms[((size_t)v * RW + r) * p.term_stride + blk] = up - dn;
        }
    }

    row_sums(terms, lane, NV, nrows, RW, B, p.term_stride, segs.out[seg], p.out_stride, row0);
}

/* Shared tail: strictly sequential per-row sums, one lane per (vector, row). */
__device__ __forceinline__ void
row_sums(const float *terms, uint32_t lane, uint32_t NV, uint32_t nrows, uint32_t RW,
         uint32_t B, uint32_t term_stride, float *out, uint32_t out_stride, uint32_t row0)
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    for (uint32_t idx = lane; idx < NV * nrows; idx += 64u) {
        const uint32_t v = idx / nrows, r = idx - v * nrows;
        const float *t = terms + ((size_t)v * RW + r) * term_stride;
        float sum = 0.0f;
        for (uint32_t b = 0; b < B; b++) sum += t[b];
        out[(size_t)v * out_stride + row0 + r] = sum;
    }
}

/* Q6_K x Q8_K.  Four lanes per super-block: lane (b, u) with u = 2n + lh owns
 * the 64 weights e = 128n + 32k + 16lh + i (k < 4, i < 16): 16 bytes of ql at
 * 64n+16lh (low nibbles -> k=0, high -> k=2), 16 bytes at 64n+32+16lh (k=1,
 * k=3) and 16 bytes of qh at 32n+16lh (two bits per k).  Each k is one
 * 16-weight scale group g = 8n + 2k + lh.  Blocks are 210 bytes, so every
 * load here is only 2-byte aligned. */
template <bool DUMP>
__global__ __launch_bounds__(OXH_GEMV_WAVES * 64) void
k_gemv_q6_k(const SegTable segs, const GemvParams p, const uint8_t *__restrict__ acts)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t B = p.blocks;
    const uint32_t NV = p.n_vec;

    const uint32_t seg = find_segment(segs, blockIdx.x);
    const uint32_t wg_in_seg = blockIdx.x - segs.wg_begin[seg];
    const uint32_t seg_rows = segs.rows[seg];

    const uint32_t act_lds = q8k6_lds_bytes(B);
    float *const terms = reinterpret_cast<float *>(lds + (size_t)act_lds * NV) +
                         (size_t)wave * NV * p.rows_per_wave * p.term_stride;

    for (uint32_t v = 0; v < NV; v++) {
        const uint8_t *a = acts + (size_t)(segs.act_first[seg] + v) * p.act_bytes;
        uint8_t *base = lds + (size_t)v * act_lds;
        uint32_t *qd = reinterpret_cast<uint32_t *>(base);
        int32_t *bs = reinterpret_cast<int32_t *>(base + B * 256u);
        float *dq = reinterpret_cast<float *>(base + B * 256u + B * 64u);
        for (uint32_t j = tid; j < B * 64u; j += OXH_GEMV_WAVES * 64u) {
            const uint32_t blk = j >> 6, w = j & 63u;
            const uint32_t e = 4u * w;
            const uint32_t n = e >> 7, k = (e >> 5) & 3u, lh = (e >> 4) & 1u;
            const uint32_t val = *reinterpret_cast<const uint32_t *>(a + (size_t)blk * 292u + 4u + 4u * w);
            qd[((k * B * 4u) + blk * 4u + 2u * n + lh) * 4u + (w & 3u)] = val;
        }
        for (uint32_t j = tid; j < B * 16u; j += OXH_GEMV_WAVES * 64u) {
            const uint32_t blk = j >> 4, g = j & 15u;
            const uint32_t n = g >> 3, k = (g >> 1) & 3u, lh = g & 1u;
            const int16_t sum = *reinterpret_cast<const int16_t *>(a + (size_t)blk * 292u + 260u + 2u * g);
            bs[(blk * 4u + 2u * n + lh) * 4u + k] = 32 * (int32_t)sum;
        }
        for (uint32_t j = tid; j < B; j += OXH_GEMV_WAVES * 64u)
            dq[j] = *reinterpret_cast<const float *>(a + (size_t)j * 292u);
    }
    __syncthreads();

    const uint32_t RW = p.rows_per_wave;
    const uint32_t row0 = (wg_in_seg * OXH_GEMV_WAVES + wave) * RW;
    if (row0 >= seg_rows) return;
    const uint32_t nrows = min(RW, seg_rows - row0);
    const uint32_t nblk = nrows * B;
    const uint32_t u = lane & 3u;
    const uint32_t n = u >> 1, lh = u & 1u;
    const uint8_t *wbase = segs.w[seg] + (size_t)row0 * B * 210u;

    for (uint32_t g0 = 0; g0 < nblk; g0 += 16u) {
        const uint32_t g = g0 + (lane >> 2);
        const bool live = g < nblk;
        const uint32_t gc = live ? g : 0u;
        const uint32_t r = (B == 1u) ? gc : __umulhi(gc, p.magic);
        const uint32_t blk = gc - r * B;
        const uint8_t *wb = wbase + (size_t)gc * 210u;
        const U32x4u2 la = *reinterpret_cast<const U32x4u2 *>(wb + 64u * n + 16u * lh);
        const U32x4u2 lb = *reinterpret_cast<const U32x4u2 *>(wb + 64u * n + 32u + 16u * lh);
        const U32x4u2 hh = *reinterpret_cast<const U32x4u2 *>(wb + 128u + 32u * n + 16u * lh);
        const uint32_t sc_lo = reinterpret_cast<const U32u2 *>(wb + 192u + 8u * n)->v;
        const uint32_t sc_hi = reinterpret_cast<const U32u2 *>(wb + 196u + 8u * n)->v;
        const uint32_t dbits = *reinterpret_cast<const uint16_t *>(wb + 208u);
        /* scale bytes lh, lh+2 (low word) and lh+4, lh+6 (high word) */
        const int sc0 = (int)(int8_t)(sc_lo >> (8u * lh));
        const int sc1 = (int)(int8_t)(sc_lo >> (8u * lh + 16u));
        const int sc2 = (int)(int8_t)(sc_hi >> (8u * lh));
        const int sc3 = (int)(int8_t)(sc_hi >> (8u * lh + 16u));
        const float dw = half_bits_to_float(dbits);
        const uint32_t qa[4] = { la.x, la.y, la.z, la.w };
        const uint32_t qb[4] = { lb.x, lb.y, lb.z, lb.w };
        const uint32_t qh[4] = { hh.x, hh.y, hh.z, hh.w };

        const uint32_t slot = blk * 4u + u;
        for (uint32_t v = 0; v < NV; v++) {
            const uint8_t *base = lds + (size_t)v * act_lds;
            const u32x4 *qv = reinterpret_cast<const u32x4 *>(base);
            const u32x4 a0 = qv[slot], a1 = qv[B * 4u + slot];
            const u32x4 a2 = qv[B * 8u + slot], a3 = qv[B * 12u + slot];
            const u32x4 off = reinterpret_cast<const u32x4 *>(base + B * 256u)[slot];
            const float dq = reinterpret_cast<const float *>(base + B * 256u + B * 64u)[blk];

            int g0s = 0, g1s = 0, g2s = 0, g3s = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t c0 = (qa[i] & 0x0F0F0F0Fu) | ((qh[i] << 4) & 0x30303030u);
                const uint32_t c1 = (qb[i] & 0x0F0F0F0Fu) | ((qh[i] << 2) & 0x30303030u);
                const uint32_t c2 = ((qa[i] >> 4) & 0x0F0F0F0Fu) | (qh[i] & 0x30303030u);
                const uint32_t c3 = ((qb[i] >> 4) & 0x0F0F0F0Fu) | ((qh[i] >> 2) & 0x30303030u);
                g0s = dot4(c0, a0[i], g0s);
                g1s = dot4(c1, a1[i], g1s);
                g2s = dot4(c2, a2[i], g2s);
                g3s = dot4(c3, a3[i], g3s);
            }
            if (DUMP) {
                if (live) {
                    int32_t *o = p.dump + ((size_t)(row0 * B + gc)) * 16u + 8u * n + lh;
                    o[0] = g0s; o[2] = g1s; o[4] = g2s; o[6] = g3s;
                }
            }
            /* sum_g sc_g * (G_g - 32*bsum_g) == pos - 32*minc, in integers */
            int tot = sc0 * (g0s - (int)off[0]) + sc1 * (g1s - (int)off[1]) +
                      sc2 * (g2s - (int)off[2]) + sc3 * (g3s - (int)off[3]);
            tot = quad_sum(tot);
            const float t = dw * dq;
            if (live && u == 0u)
                terms[((size_t)v * RW + r) * p.term_stride + blk] = t * (float)tot;
        }
    }
    row_sums(terms, lane, NV, nrows, RW, B, p.term_stride, segs.out[seg], p.out_stride, row0);
}

/* Q8_0 x Q8_0.  One lane per 34-byte block, 64 blocks (2176 contiguous bytes)
 * per wave pass.  The per-block integer dot is exact; the f32 result is the
 * block-sequential chain of oxk.c:224-241 (the reference's x86 decode path
 * accumulates the same terms in a different order, so f32 outputs agree with
 * it to tolerance, not to the bit). */
template <bool DUMP>
__global__ __launch_bounds__(OXH_GEMV_WAVES * 64) void
k_gemv_q8_0(const SegTable segs, const GemvParams p, const uint8_t *__restrict__ acts)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t B = p.blocks;
    const uint32_t NV = p.n_vec;

    const uint32_t seg = find_segment(segs, blockIdx.x);
    const uint32_t wg_in_seg = blockIdx.x - segs.wg_begin[seg];
    const uint32_t seg_rows = segs.rows[seg];

    const uint32_t act_lds = q80_lds_bytes(B);
    float *const terms = reinterpret_cast<float *>(lds + (size_t)act_lds * NV) +
                         (size_t)wave * NV * p.rows_per_wave * p.term_stride;

    for (uint32_t v = 0; v < NV; v++) {
        const uint8_t *a = acts + (size_t)(segs.act_first[seg] + v) * p.act_bytes;
        uint8_t *base = lds + (size_t)v * act_lds;
        uint32_t *qd = reinterpret_cast<uint32_t *>(base);
        float *dq = reinterpret_cast<float *>(base + B * 32u);
        for (uint32_t j = tid; j < B * 8u; j += OXH_GEMV_WAVES * 64u) {
            const uint32_t blk = j >> 3, w = j & 7u;
            const uint32_t val = reinterpret_cast<const U32u2 *>(a + (size_t)blk * 34u + 2u + 4u * w)->v;
            qd[(((w >> 2) * B) + blk) * 4u + (w & 3u)] = val;
        }
        for (uint32_t j = tid; j < B; j += OXH_GEMV_WAVES * 64u)
            dq[j] = half_bits_to_float(*reinterpret_cast<const uint16_t *>(a + (size_t)j * 34u));
    }
    __syncthreads();

    const uint32_t RW = p.rows_per_wave;
    const uint32_t row0 = (wg_in_seg * OXH_GEMV_WAVES + wave) * RW;
    if (row0 >= seg_rows) return;
    const uint32_t nrows = min(RW, seg_rows - row0);
    const uint32_t nblk = nrows * B;
    const uint8_t *wbase = segs.w[seg] + (size_t)row0 * B * 34u;

    for (uint32_t g0 = 0; g0 < nblk; g0 += 64u) {
        const uint32_t g = g0 + lane;
        const bool live = g < nblk;
        const uint32_t gc = live ? g : 0u;
        const uint32_t r = (B == 1u) ? gc : __umulhi(gc, p.magic);
        const uint32_t blk = gc - r * B;
        const uint8_t *wb = wbase + (size_t)gc * 34u;
        const uint32_t dbits = *reinterpret_cast<const uint16_t *>(wb);
        const U32x4u2 w0 = *reinterpret_cast<const U32x4u2 *>(wb + 2u);
        const U32x4u2 w1 = *reinterpret_cast<const U32x4u2 *>(wb + 18u);
        const float dw = half_bits_to_float(dbits);

        for (uint32_t v = 0; v < NV; v++) {
            const uint8_t *base = lds + (size_t)v * act_lds;
            const u32x4 *qv = reinterpret_cast<const u32x4 *>(base);
            const u32x4 a0 = qv[blk], a1 = qv[B + blk];
            const float dq = reinterpret_cast<const float *>(base + B * 32u)[blk];
            int isum = 0;
            isum = dot4(w0.x, a0[0], isum); isum = dot4(w0.y, a0[1], isum);
            isum = dot4(w0.z, a0[2], isum); isum = dot4(w0.w, a0[3], isum);
            isum = dot4(w1.x, a1[0], isum); isum = dot4(w1.y, a1[1], isum);
            isum = dot4(w1.z, a1[2], isum); isum = dot4(w1.w, a1[3], isum);
            if (DUMP) {
                if (live) p.dump[(size_t)row0 * B + gc] = isum;
            }
            const float t = dw * dq;
            if (live) terms[((size_t)v * RW + r) * p.term_stride + blk] = t * (float)isum;
        }
    }
    row_sums(terms, lane, NV, nrows, RW, B, p.term_stride, segs.out[seg], p.out_stride, row0);
}

/* ─── prefill matmul (MMQ) ────────────────────────────────────────────── */

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define MMQ_WAVES 4
#define MMQ_ROWS (MMQ_WAVES * 32)   /* weight rows per workgroup          */
#define MMQ_TOK 64                  /* tokens per workgroup (two tiles)   */

/* Q4_K weights x Q8_K activations on v_mfma_i32_32x32x32_i8.
 *
 * One MFMA covers 32 tokens x 32 weight rows x one 32-wide sub-block, so each
 * result tile is exactly the sub-block sums S_j of oxk.c:263-270 for 1024
 * (token, row) pairs.  M = tokens (A operand, int8 activations staged in
 * LDS), N = weight rows (B operand, nibble codes unpacked in registers): the
 * accumulator of lane l then belongs to weight row l%32, so the 6-bit scale
 * is one register per lane and `pos += sc_j * S_j` is an integer multiply-add
 * per accumulator.  The min term sum_j m_j*B_j is formed by a second MFMA per
 * sub-block with the B operand set to m_j in every byte (sum_k m_j*q_k over
 * the sub-block is m_j*B_j), accumulated over the whole super-block.
 * Per super-block the f32 step is the reference's, in its order:
 *   acc += (dw*dq)*(float)pos - (dmin*dq)*(float)min_acc      (oxk.c:286-294)
 * so every output is bit-identical to the single-vector GEMV.
 *
 * Lane l supplies, for both operands, the 16 values k = 16*(l/32) .. +15 of
 * the sub-block; A and B use the same assignment, so the product does not
 * depend on how the hardware numbers k internally. */
__global__ __launch_bounds__(MMQ_WAVES * 64) void
k_mmq_q4_k(const uint8_t *__restrict__ w, uint32_t rows, uint32_t B,
           const uint8_t *__restrict__ acts, uint32_t n_vec, float *__restrict__ out,
           size_t out_stride)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds_q[MMQ_TOK * 256];
    __shared__ float lds_dq[MMQ_TOK];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t n = lane & 31u;          /* weight row / token within a tile */
    const uint32_t h = lane >> 5;           /* which 16 of the sub-block's 32   */
    const uint32_t row_base = blockIdx.x * MMQ_ROWS + wave * 32u;
    const uint32_t tok_base = blockIdx.y * MMQ_TOK;
    const uint32_t row = row_base + n;
    const uint32_t row_c = row < rows ? row : rows - 1u;
    const uint8_t *wrow = w + (size_t)row_c * B * 144u;
    const size_t act_stride = (size_t)B * 292u;

    float acc[2][16];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.0f;

    for (uint32_t b = 0; b < B; b++) {
        __syncthreads();
        /* stage this super-block of 64 tokens: value dword wd of token t goes
         * to [tile][j][h][token-in-tile] x 16 B */
        for (uint32_t idx = tid; idx < MMQ_TOK * 64u; idx += MMQ_WAVES * 64u) {
            const uint32_t t = idx >> 6, wd = idx & 63u;
            const uint32_t tok = tok_base + t;
            uint32_t val = 0u;
            if (tok < n_vec)
                val = *reinterpret_cast<const uint32_t *>(acts + (size_t)tok * act_stride +
                                                          (size_t)b * 292u + 4u + 4u * wd);
            const uint32_t j = wd >> 3, hh = (wd >> 2) & 1u;
            const uint32_t slot = (((t >> 5) * 8u + j) * 2u + hh) * 32u + (t & 31u);
            reinterpret_cast<uint32_t *>(lds_q)[slot * 4u + (wd & 3u)] = val;
        }
        if (tid < MMQ_TOK) {
            const uint32_t tok = tok_base + tid;
            lds_dq[tid] = tok < n_vec
                ? *reinterpret_cast<const float *>(acts + (size_t)tok * act_stride + (size_t)b * 292u)
                : 0.0f;
        }
        /* this lane's weights: header and its half of each 32-byte nibble group */
        const uint8_t *wb = wrow + (size_t)b * 144u;
        const u32x4 hdr = *reinterpret_cast<const u32x4 *>(wb);
        u32x4 nib[4];
#pragma unroll
        for (int gp = 0; gp < 4; gp++)
            nib[gp] = *reinterpret_cast<const u32x4 *>(wb + 16u + 32u * gp + 16u * h);
        __syncthreads();

        const uint32_t u0 = hdr.y, u1 = hdr.z, u2 = hdr.w;
        const uint32_t sc_lo = u0 & 0x3F3F3F3Fu;
        const uint32_t mn_lo = u1 & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (u2 & 0x0F0F0F0Fu) | ((u0 >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((u2 >> 4) & 0x0F0F0F0Fu) | ((u1 >> 2) & 0x30303030u);
        const float dw = half_bits_to_float(hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_float(hdr.x >> 16);

        v16i pos[2], mn[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) { pos[t][i] = 0; mn[t][i] = 0; }

#pragma unroll
        for (int j = 0; j < 8; j++) {
            const u32x4 raw = nib[j >> 1];
            v4i bw;
#pragma unroll
            for (int k = 0; k < 4; k++)
                bw[k] = (int)((j & 1) ? ((raw[k] >> 4) & 0x0F0F0F0Fu) : (raw[k] & 0x0F0F0F0Fu));
            const uint32_t scw = j < 4 ? sc_lo : sc_hi;
            const uint32_t mnw = j < 4 ? mn_lo : mn_hi;
            const int sc = (int)((scw >> (8 * (j & 3))) & 0xFFu);
            const int mj = (int)(((mnw >> (8 * (j & 3))) & 0xFFu) * 0x01010101u);
            const v4i bm = { mj, mj, mj, mj };
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4i a = *reinterpret_cast<const v4i *>(
                    lds_q + ((((uint32_t)t * 8u + (uint32_t)j) * 2u + h) * 32u + n) * 16u);
                const v16i zero = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
                const v16i sj = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bw, zero, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 16; i++) pos[t][i] += __mul24(sc, sj[i]);
                mn[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bm, mn[t], 0, 0, 0);
            }
        }
        /* accumulator i of lane l is token 8*(i/4) + 4*(l/32) + i%4 of the tile */
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t m = 8u * (uint32_t)(i >> 2) + 4u * h + (uint32_t)(i & 3);
                const float dq = lds_dq[t * 32 + m];
                const float t_pos = dw * dq;
                const float t_min = dmin * dq;
                const float up = t_pos * (float)pos[t][i];
                const float dn = t_min * (float)mn[t][i];
                acc[t][i] += up - dn;
            }
    }
    if (row < rows) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t m = 8u * (uint32_t)(i >> 2) + 4u * h + (uint32_t)(i & 3);
                const uint32_t tok = tok_base + (uint32_t)t * 32u + m;
                if (tok < n_vec) out[(size_t)tok * out_stride + row] = acc[t][i];
            }
    }
}

/* ─── host side of layer 2 ────────────────────────────────────────────── */

static int g_device = -1;
static hipStream_t g_stream = nullptr;
static int g_n_cu = 0;

extern "C" int oxh_init(int device)
{
    if (g_device >= 0) {
        if (device == g_device) return OXH_OK;
        return arg_fail("oxh_init: already initialised on another device");
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        snprintf(g_err, sizeof g_err, "no HIP device available (%s)",
                 e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        return OXH_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= n) return arg_fail("oxh_init: device index out of range");
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    g_n_cu = prop.multiProcessorCount;
    HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    g_device = device;
    return OXH_OK;
}

extern "C" void oxh_shutdown(void)
{
    if (g_device < 0) return;
    if (g_stream) (void)hipStreamDestroy(g_stream);
    g_stream = nullptr;
    g_device = -1;
}

static int ensure_init(void)
{
    if (g_device >= 0) return OXH_OK;
    return oxh_init(0);
}

static hipStream_t pick_stream(void *stream)
{
    return stream ? (hipStream_t)stream : g_stream;
}

extern "C" void *oxh_internal_stream(void) { return (void *)g_stream; }

extern "C" int oxh_act_kind(uint32_t qtype, size_t cols)
{
    switch (qtype) {
    case OXH_Q8_0:   return (cols % OXH_QK8_0 == 0) ? 1 : 0;
    case OXH_Q4_K_S:
    case OXH_Q4_K_M:
    case OXH_Q6_K:   return (cols % OXH_QK_K == 0) ? 2 : 0;
    default:         return 0;
    }
}

static size_t block_bytes(uint32_t qtype)
{
    switch (qtype) {
    case OXH_Q8_0:   return OXH_Q8_0_BYTES;
    case OXH_Q4_K_S:
    case OXH_Q4_K_M: return OXH_Q4_K_BYTES;
    case OXH_Q6_K:   return OXH_Q6_K_BYTES;
    default:         return 0;
    }
}

extern "C" size_t oxh_row_bytes(uint32_t qtype, size_t cols)
{
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) return 0;
    const size_t nb = kind == 2 ? cols / OXH_QK_K : cols / OXH_QK8_0;
    const size_t bb = block_bytes(qtype);
    if (nb != 0 && bb > SIZE_MAX / nb) return 0;
    return nb * bb;
}

extern "C" size_t oxh_act_bytes(uint32_t qtype, size_t cols)
{
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) return 0;
    return kind == 2 ? cols / OXH_QK_K * OXH_Q8_K_BYTES : cols / OXH_QK8_0 * OXH_Q8_0_BYTES;
}

extern "C" int oxh_quantize_q8_k(const float *d_x, size_t in_stride, size_t n_vec,
                                 size_t cols, void *d_act, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (n_vec == 0 || cols == 0) return OXH_OK;
    if (!d_x || !d_act) return arg_fail("oxh_quantize_q8_k: NULL pointer");
    if (cols % OXH_QK_K) return arg_fail("oxh_quantize_q8_k: cols not a multiple of 256");
    if (in_stride < cols) return arg_fail("oxh_quantize_q8_k: in_stride < cols");
    const size_t bpv = cols / OXH_QK_K;
    if (bpv > 0xFFFFFFFFull / n_vec) return arg_fail("oxh_quantize_q8_k: too many blocks");
    const uint32_t total = (uint32_t)(bpv * n_vec);
    hipLaunchKernelGGL(k_quantize_q8_k, dim3((total + 3u) / 4u), dim3(256), 0,
                       pick_stream(stream), d_x, in_stride, (uint32_t)bpv, total,
                       (uint8_t *)d_act);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_quantize_q8_0(const float *d_x, size_t in_stride, size_t n_vec,
                                 size_t cols, void *d_act, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (n_vec == 0 || cols == 0) return OXH_OK;
    if (!d_x || !d_act) return arg_fail("oxh_quantize_q8_0: NULL pointer");
    if (cols % OXH_QK8_0) return arg_fail("oxh_quantize_q8_0: cols not a multiple of 32");
    if (in_stride < cols) return arg_fail("oxh_quantize_q8_0: in_stride < cols");
    const size_t bpv = cols / OXH_QK8_0;
    const size_t spans = (bpv + 7u) / 8u;
    if (spans > 0xFFFFFFFFull / n_vec || n_vec > 0xFFFFFFFFull)
        return arg_fail("oxh_quantize_q8_0: too many blocks");
    const uint32_t total = (uint32_t)(spans * n_vec);
    hipLaunchKernelGGL(k_quantize_q8_0, dim3((total + 3u) / 4u), dim3(256), 0,
                       pick_stream(stream), d_x, in_stride, (uint32_t)bpv,
                       (uint32_t)n_vec, (uint8_t *)d_act);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* Rows each wave takes: large enough to amortise the per-row tail, small
 * enough that the launch still has several waves per SIMD on every CU. */
static uint32_t choose_rows_per_wave(size_t total_rows, uint32_t blocks, uint32_t lanes_per_block)
{
    const size_t target_waves = (size_t)(g_n_cu > 0 ? g_n_cu : 256) * 16u;
    size_t rw = total_rows / target_waves;
    if (rw < 1) rw = 1;
    if (rw > 16) rw = 16;
    /* whole passes when possible: rw*blocks a multiple of blocks-per-pass */
    const uint32_t per_pass = 64u / lanes_per_block;
    while (rw > 1 && ((rw * blocks) % per_pass) != 0) rw--;
    return (uint32_t)rw;
}

static bool is_q4k(uint32_t qtype) { return qtype == OXH_Q4_K_S || qtype == OXH_Q4_K_M; }

static uint32_t act_lds_bytes(uint32_t qtype, uint32_t blocks)
{
    if (qtype == OXH_Q8_0) return q80_lds_bytes(blocks);
    if (qtype == OXH_Q6_K) return q8k6_lds_bytes(blocks);
    return q8k_lds_bytes(blocks);
}

static size_t gemv_lds_bytes(uint32_t qtype, uint32_t blocks, size_t n_vec, uint32_t rows_per_wave)
{
    return n_vec * (size_t)act_lds_bytes(qtype, blocks) +
           (size_t)OXH_GEMV_WAVES * n_vec * rows_per_wave * (blocks + 1u) * 4u;
}

extern "C" size_t oxh_gemv_max_nvec(uint32_t qtype, size_t cols)
{
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) return 0;
    const size_t blocks = kind == 2 ? cols / OXH_QK_K : cols / OXH_QK8_0;
    if (blocks > 0xFFFFu) return 0;
    size_t nv = OXH_MAX_NV;
    while (nv > 0 && gemv_lds_bytes(qtype, (uint32_t)blocks, nv, 1) > 65536u) nv--;
    return nv;
}

static int launch_gemv(uint32_t qtype, const OxhSegment *segs, size_t n_segs, size_t cols,
                       const void *d_acts, size_t n_vec, size_t out_stride, int32_t *dump,
                       void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (n_segs == 0) return OXH_OK;
    if (!segs || !d_acts) return arg_fail("gemv: NULL pointer");
    if (n_vec < 1 || n_vec > OXH_MAX_NV) return arg_fail("gemv: n_vec must be 1..8");
    if (n_segs > OXH_MAX_SEGS) return arg_fail("gemv: more than 32 segments in one launch");
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) {
        snprintf(g_err, sizeof g_err, "gemv: qtype %u with cols %zu has no integer path", qtype, cols);
        return OXH_DECLINED;
    }
    const size_t blocks = kind == 2 ? cols / OXH_QK_K : cols / OXH_QK8_0;
    const size_t bbytes = block_bytes(qtype);
    if (blocks > 0xFFFFu) {
        snprintf(g_err, sizeof g_err, "gemv: cols %zu too wide", cols);
        return OXH_ERR_TOO_WIDE;
    }
    size_t total_rows = 0, max_act = 0;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows > 0x7FFFFFFFull / (blocks * 16u)) return arg_fail("gemv: segment too large");
        if (segs[i].rows && (!segs[i].d_w || !segs[i].d_out)) return arg_fail("gemv: NULL segment pointer");
        total_rows += segs[i].rows;
        if (segs[i].act_first > max_act) max_act = segs[i].act_first;
    }
    if (total_rows == 0) return OXH_OK;
    if (out_stride > 0xFFFFFFFFull || max_act + n_vec > 0xFFFFFFFFull) return arg_fail("gemv: stride too large");
    (void)bbytes;

    const uint32_t lanes_per_block = qtype == OXH_Q8_0 ? 1u : 4u;
    GemvParams p;
    p.blocks = (uint32_t)blocks;
    p.magic = (uint32_t)((0x100000000ull + blocks - 1u) / blocks);
    p.rows_per_wave = choose_rows_per_wave(total_rows, p.blocks, lanes_per_block);
    p.n_vec = (uint32_t)n_vec;
    p.act_bytes = (uint32_t)oxh_act_bytes(qtype, cols);
    p.out_stride = (uint32_t)out_stride;
    p.term_stride = p.blocks + 1u;
    p.dump = dump;

    size_t lds = gemv_lds_bytes(qtype, p.blocks, n_vec, p.rows_per_wave);
    while (lds > 65536u && p.rows_per_wave > 1) {
        p.rows_per_wave--;
        lds = gemv_lds_bytes(qtype, p.blocks, n_vec, p.rows_per_wave);
    }
    if (lds > 65536u) {
        snprintf(g_err, sizeof g_err, "gemv: cols %zu x n_vec %zu needs %zu B of LDS (max 65536)",
                 cols, n_vec, lds);
        return OXH_ERR_TOO_WIDE;
    }

    SegTable t;
    memset(&t, 0, sizeof t);
    uint32_t wg = 0;
    uint32_t n = 0;
    const uint32_t rows_per_wg = p.rows_per_wave * OXH_GEMV_WAVES;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows == 0) continue;
        t.w[n] = (const uint8_t *)segs[i].d_w;
        t.out[n] = segs[i].d_out;
        t.rows[n] = (uint32_t)segs[i].rows;
        t.act_first[n] = (uint32_t)segs[i].act_first;
        t.wg_begin[n] = wg;
        wg += (uint32_t)((segs[i].rows + rows_per_wg - 1u) / rows_per_wg);
        n++;
    }
    t.wg_begin[n] = wg;
    t.n = n;

    const dim3 grid(wg), block(OXH_GEMV_WAVES * 64);
    hipStream_t st = pick_stream(stream);
    const uint8_t *a = (const uint8_t *)d_acts;
    if (is_q4k(qtype)) {
        if (dump) hipLaunchKernelGGL(k_gemv_q4_k<true>, grid, block, lds, st, t, p, a);
        else      hipLaunchKernelGGL(k_gemv_q4_k<false>, grid, block, lds, st, t, p, a);
    } else if (qtype == OXH_Q6_K) {
        if (dump) hipLaunchKernelGGL(k_gemv_q6_k<true>, grid, block, lds, st, t, p, a);
        else      hipLaunchKernelGGL(k_gemv_q6_k<false>, grid, block, lds, st, t, p, a);
    } else {
        if (dump) hipLaunchKernelGGL(k_gemv_q8_0<true>, grid, block, lds, st, t, p, a);
        else      hipLaunchKernelGGL(k_gemv_q8_0<false>, grid, block, lds, st, t, p, a);
    }
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_gemv_segments(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                                 size_t cols, const void *d_acts, size_t n_vec,
                                 size_t out_stride, void *stream)
{
    return launch_gemv(qtype, segs, n_segs, cols, d_acts, n_vec, out_stride, nullptr, stream);
}

extern "C" int oxh_debug_subblock_sums(uint32_t qtype, const void *d_w, size_t rows,
                                       size_t cols, const void *d_act, int32_t *d_sums,
                                       void *stream)
{
    if (!d_sums) return arg_fail("oxh_debug_subblock_sums: NULL output");
    int rc = ensure_init();
    if (rc) return rc;
    float *scratch = nullptr;
    HIP_TRY(hipMalloc((void **)&scratch, (rows ? rows : 1) * sizeof(float)));
    OxhSegment s = { d_w, scratch, rows, 0 };
    rc = launch_gemv(qtype, &s, 1, cols, d_act, 1, rows, d_sums, stream);
    hipError_t e = hipStreamSynchronize(pick_stream(stream));
    (void)hipFree(scratch);
    if (rc) return rc;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return OXH_OK;
}

extern "C" int oxh_mmq(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                       const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
                       void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0 || n_vec == 0) return OXH_OK;
    if (!d_w || !d_acts || !d_out) return arg_fail("oxh_mmq: NULL pointer");
    if (!is_q4k(qtype) || oxh_act_kind(qtype, cols) != 2) {
        snprintf(g_err, sizeof g_err, "oxh_mmq: qtype %u with cols %zu has no MFMA kernel", qtype, cols);
        return OXH_DECLINED;
    }
    if (out_stride < rows) return arg_fail("oxh_mmq: out_stride < rows");
    const size_t blocks = cols / OXH_QK_K;
    if (rows > 0x7FFFFFFFull || n_vec > 0x7FFFFFFFull || blocks > 0xFFFFFFull)
        return arg_fail("oxh_mmq: dimension too large");
    const dim3 grid((uint32_t)((rows + MMQ_ROWS - 1) / MMQ_ROWS),
                    (uint32_t)((n_vec + MMQ_TOK - 1) / MMQ_TOK));
    hipLaunchKernelGGL(k_mmq_q4_k, grid, dim3(MMQ_WAVES * 64), 0, pick_stream(stream),
                       (const uint8_t *)d_w, (uint32_t)rows, (uint32_t)blocks,
                       (const uint8_t *)d_acts, (uint32_t)n_vec, d_out, out_stride);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* ─── memory / stream / event plumbing ────────────────────────────────── */

extern "C" int oxh_malloc(void **d_ptr, size_t bytes)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (!d_ptr) return arg_fail("oxh_malloc: NULL");
    hipError_t e = hipMalloc(d_ptr, bytes ? bytes : 1);
    if (e == hipErrorOutOfMemory) {
        snprintf(g_err, sizeof g_err, "out of device memory allocating %zu bytes", bytes);
        (void)hipGetLastError();
        return OXH_ERR_NOMEM;
    }
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    return OXH_OK;
}

extern "C" int oxh_free(void *d_ptr)
{
    if (!d_ptr) return OXH_OK;
    HIP_TRY(hipFree(d_ptr));
    return OXH_OK;
}

extern "C" int oxh_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    HIP_TRY(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    HIP_TRY(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_memset(void *d_dst, int value, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    HIP_TRY(hipMemsetAsync(d_dst, value, bytes, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_stream_create(void **stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s;
    HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = (void *)s;
    return OXH_OK;
}

extern "C" int oxh_stream_destroy(void *stream)
{
    if (stream) HIP_TRY(hipStreamDestroy((hipStream_t)stream));
    return OXH_OK;
}

extern "C" int oxh_stream_sync(void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    HIP_TRY(hipStreamSynchronize(pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_event_create(void **event)
{
    int rc = ensure_init();
    if (rc) return rc;
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    *event = (void *)e;
    return OXH_OK;
}

extern "C" int oxh_event_destroy(void *event)
{
    if (event) HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return OXH_OK;
}

extern "C" int oxh_event_record(void *event, void *stream)
{
    HIP_TRY(hipEventRecord((hipEvent_t)event, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_event_sync(void *event)
{
    HIP_TRY(hipEventSynchronize((hipEvent_t)event));
    return OXH_OK;
}

extern "C" int oxh_event_elapsed_ms(void *start, void *stop, float *ms)
{
    HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return OXH_OK;
}

extern "C" int oxh_graph_begin(void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    HIP_TRY(hipStreamBeginCapture(pick_stream(stream), hipStreamCaptureModeThreadLocal));
    return OXH_OK;
}

extern "C" int oxh_graph_end(void *stream, void **graph_exec)
{
    if (!graph_exec) return arg_fail("oxh_graph_end: NULL");
    hipGraph_t graph = nullptr;
    HIP_TRY(hipStreamEndCapture(pick_stream(stream), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate");
    *graph_exec = (void *)exec;
    return OXH_OK;
}

extern "C" int oxh_graph_launch(void *graph_exec, void *stream)
{
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_graph_destroy(void *graph_exec)
{
    if (graph_exec) HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return OXH_OK;
}

extern "C" int oxh_device_info(char *name, size_t name_len, int *n_cu, int *clock_mhz,
                               size_t *mem_bytes)
{
    int rc = ensure_init();
    if (rc) return rc;
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, g_device));
    if (name && name_len) {
        strncpy(name, prop.name, name_len - 1);
        name[name_len - 1] = 0;
    }
    if (n_cu) *n_cu = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (mem_bytes) *mem_bytes = prop.totalGlobalMem;
    return OXH_OK;
}
