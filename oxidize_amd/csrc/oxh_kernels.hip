/*
 * oxh_kernels.hip — gfx950 kernels and the thin device-resident C ABI of
 * liboxhip (layer 2 of include/oxhip.h).
 *
 * Arithmetic contract (all paths relative to the reference checkout):
 *   Q8_K / Q8_0 activation bytes  oxidize-c/src/compute/matvec.c:276-316, :130-155
 *   f32 -> f16 (round half up)    oxidize-c/src/compute/flash_attention.c:149-185
 *   Q4_K x Q8_K block dot         oxidize-c/src/compute/oxk.c:243-297
 *   Q5_K x Q8_K block dot         oxidize-c/src/compute/oxk.c:849-911
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
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "oxhip.h"
#include "oxhip_lab.h"
#include "oxh_internal.h"

#pragma clang fp contract(off)

/* ─── error plumbing ──────────────────────────────────────────────────── */

static thread_local char g_err[512] = "";

extern "C" const char *oxh_last_error(void) { return g_err; }

extern "C" void oxh_set_error(const char *fmt, const char *a, const char *b)
{
    snprintf(g_err, sizeof g_err, fmt, a ? a : "", b ? b : "");
}

extern "C" int oxh_internal_errorf(int status, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return status;
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

#include "oxh_device.inc"

/* ─── activation quantisers ───────────────────────────────────────────── */

/* One wave per 256-value block; lane l owns values 4l..4l+3.  Two optional
 * extras for the mixture-of-experts path: `row_index` makes output vector v
 * read input row row_index[v] (the gather of each expert's tokens), and `up`
 * (laid out like x, same row) makes the value quantised silu(x) * up. */
__global__ __launch_bounds__(256) void
k_quantize_q8_k(const float *__restrict__ x, size_t in_stride, uint32_t blocks_per_vec,
                uint32_t total_blocks, uint8_t *__restrict__ act,
                const uint32_t *__restrict__ row_index, const float *__restrict__ up)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t gb = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (gb >= total_blocks) return;
    const uint32_t vec = gb / blocks_per_vec;
    const uint32_t blk = gb - vec * blocks_per_vec;
    const size_t at = (size_t)(row_index ? row_index[vec] : vec) * in_stride + (size_t)blk * 256u + 4u * lane;
    const float *src = x + at;
    float v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];
    if (up) {
        const float *u = up + at;
        const float s0 = 1.0f / (1.0f + expf(-v0)), s1 = 1.0f / (1.0f + expf(-v1));
        const float s2 = 1.0f / (1.0f + expf(-v2)), s3 = 1.0f / (1.0f + expf(-v3));
        v0 = v0 * s0 * u[0]; v1 = v1 * s1 * u[1]; v2 = v2 * s2 * u[2]; v3 = v3 * s3 * u[3];
    }

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

/* ─── embedding lookup: packed rows -> f32 ────────────────────────────── */

/* out[t][:] = dequantised row ids[t] of a packed matrix, in the reference's
 * arithmetic (oxidize-c/src/compute/quantization.c:486-503 Q8_0, :633-670
 * Q4_K, :672-721 Q5_K, :723-766 Q6_K), so the values equal the CPU path's to
 * the bit.  One wave per 256 values, lane l producing values 4l .. 4l+3 (they
 * share a sub-block / scale group); grid.y walks the ids.  An id beyond the
 * matrix yields a row of zeros rather than a read outside it.
 * KIND: 0 Q4_K, 1 Q5_K, 2 Q6_K, 3 Q8_0, 4 Q4_0, 5 Q4_1, 6 Q5_0, 7 Q5_1, 8 Q2_K, 9 Q3_K, 10 AL5_XS. */
template <int KIND>
__global__ __launch_bounds__(256) void
k_get_rows(const uint8_t *__restrict__ w, uint32_t rows, uint32_t cols, uint32_t row_bytes,
           const uint32_t *__restrict__ ids, float *__restrict__ out, size_t out_stride)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t unit = blockIdx.x * 4u + (threadIdx.x >> 6);     /* 256-value span of the row */
    const uint32_t e0 = unit * 256u + 4u * lane;                    /* this lane's first element */
    if (e0 >= cols) return;
    const uint32_t id = ids[blockIdx.y];
    float *dst = out + (size_t)blockIdx.y * out_stride + e0;
    float v[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
    if (id < rows) {
        const uint8_t *row = w + (size_t)id * row_bytes;
        if (KIND == 10) {
            /* thirty-two 3-bit codes behind an f16 d, element i at bits [3i, 3i+3) (quantization.c:802-832):
             * this lane's four codes are twelve bits starting at bit 3*(e0 % 32), inside one or two of the
             * block's six 16-bit words */
            const uint8_t *blk = row + (size_t)(e0 >> 5) * 14u;
            const float d = half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk));
            const uint32_t bit = 3u * (e0 & 31u), word = bit >> 4;          /* bit = 12 * (lane % 8) */
            const uint32_t lo16 = *reinterpret_cast<const uint16_t *>(blk + 2u + 2u * word);
            const uint32_t hi16 = word < 5u ? *reinterpret_cast<const uint16_t *>(blk + 4u + 2u * word) : 0u;
            const uint32_t c = ((lo16 | (hi16 << 16)) >> (bit & 15u)) & 0xFFFu;
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = (float)((int)((c >> (3 * i)) & 7u) - 4) * d;
        } else if (KIND >= 8) {
            /* 2-bit codes: element 128n + 32k + l is bits [2k, 2k+2) of qs[32n + l]; Q3_K adds bit
             * 4n + k of hmask[l] as the third bit (quantization.c:521-630) */
            const uint8_t *blk = row + (size_t)unit * (KIND == 9 ? 110u : 84u);
            const uint32_t e = 4u * lane, n = e >> 7, k = (e >> 5) & 3u, l32 = e & 31u, g = e >> 4;
            if (KIND == 8) {
                const uint32_t dd = *reinterpret_cast<const uint32_t *>(blk + 80u);
                const uint32_t sb = blk[g];
                const float dl = half_to_float_hw(dd & 0xFFFFu) * (float)(sb & 15u);
                const float ml = half_to_float_hw(dd >> 16) * (float)(sb >> 4);
                const uint32_t q = *reinterpret_cast<const uint32_t *>(blk + 16u + 32u * n + l32) >> (2u * k);
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = dl * (float)((q >> (8 * i)) & 3u) - ml;
            } else {
                const uint8_t *sp = blk + 96u;
                const uint32_t lo4 = g < 8u ? (sp[g] & 15u) : (uint32_t)(sp[g - 8u] >> 4);
                const uint32_t hi2 = (sp[8u + (g & 3u)] >> (2u * (g >> 2))) & 3u;
                const float dl = half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk + 108u)) *
                                 (float)((int)(lo4 | (hi2 << 4)) - 32);
                const uint32_t q = reinterpret_cast<const U32u2 *>(blk + 32u + 32u * n + l32)->v >> (2u * k);
                const uint32_t h = reinterpret_cast<const U32u2 *>(blk + l32)->v >> (4u * n + k);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    v[i] = dl * (float)((int)(((q >> (8 * i)) & 3u) | (((h >> (8 * i)) & 1u) << 2)) - 4);
            }
        } else if (KIND >= 4) {
            /* 32-value blocks [f16 d][f16 m: Q4_1, Q5_1][4 B fifth bits: Q5_0, Q5_1][16 B nibbles]; value i
             * is the low nibble of byte i, value i + 16 the high nibble (quantization.c:386-474) */
            const bool has_m = KIND == 5 || KIND == 7, has_h = KIND >= 6;
            const uint32_t qh_at = has_m ? 4u : 2u, qs_at = qh_at + (has_h ? 4u : 0u);
            const uint8_t *blk = row + (size_t)(e0 >> 5) * (qs_at + 16u);
            const uint32_t i0 = e0 & 31u;
            const float d = half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk));
            const float m = has_m ? half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk + 2u)) : 0.0f;
            const uint32_t q = reinterpret_cast<const U32u2 *>(blk + qs_at + (i0 & 15u))->v >> (i0 & 16u ? 4u : 0u);
            const uint32_t h = has_h ? reinterpret_cast<const U32u2 *>(blk + qh_at)->v >> i0 : 0u;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t code = ((q >> (8 * i)) & 15u) | (((h >> i) & 1u) << 4);
                if (has_m) v[i] = (float)code * d + m;
                else v[i] = (float)((int)code - (has_h ? 16 : 8)) * d;
            }
        } else if (KIND == 3) {
            const uint8_t *blk = row + (size_t)(e0 >> 5) * 34u;
            const float d = half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk));
            const uint32_t q = reinterpret_cast<const U32u2 *>(blk + 2u + (e0 & 31u))->v;
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = (float)(int8_t)(q >> (8 * i)) * d;
        } else if (KIND == 2) {
            const uint8_t *blk = row + (size_t)unit * 210u;
            const uint32_t e = 4u * lane, n = e >> 7, k = (e >> 5) & 3u, l32 = e & 31u;
            const uint32_t lo = reinterpret_cast<const U32u2 *>(blk + 64u * n + 32u * (k & 1u) + l32)->v;
            const uint32_t hi = reinterpret_cast<const U32u2 *>(blk + 128u + 32u * n + l32)->v;
            const float d = half_to_float_hw(*reinterpret_cast<const uint16_t *>(blk + 208u));
            const float sc = (float)(int8_t)blk[192u + (e >> 4)];
            const float ds = d * sc;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lb = (lo >> (8 * i)) & 0xFFu, hb = (hi >> (8 * i)) & 0xFFu;
                const int code = (int)((k < 2u ? (lb & 15u) : (lb >> 4)) | (((hb >> (2u * k)) & 3u) << 4)) - 32;
                v[i] = ds * (float)code;
            }
        } else {
            const uint32_t bs = KIND == 1 ? 176u : 144u;
            const uint8_t *blk = row + (size_t)unit * bs;
            const uint32_t e = 4u * lane, j = e >> 5, l32 = e & 31u;
            const uint32_t hdr = *reinterpret_cast<const uint32_t *>(blk);
            const float d = half_to_float_hw(hdr & 0xFFFFu), dmin = half_to_float_hw(hdr >> 16);
            /* 6-bit scale and min of sub-block j (oxk.c:60-75) */
            const uint8_t *q = blk + 4u;
            uint32_t sc, mn;
            if (j < 4u) { sc = q[j] & 63u; mn = q[j + 4u] & 63u; }
            else { sc = (q[j + 4u] & 15u) | ((q[j - 4u] >> 6) << 4); mn = (q[j + 4u] >> 4) | ((q[j] >> 6) << 4); }
            const float ds = d * (float)sc, ms = dmin * (float)mn;
            const uint32_t nib = *reinterpret_cast<const uint32_t *>(blk + (KIND == 1 ? 48u : 16u) + 32u * (j >> 1) + l32);
            uint32_t fifth = 0u;
            if (KIND == 1) fifth = *reinterpret_cast<const uint32_t *>(blk + 16u + l32) >> j;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t byte = (nib >> (8 * i)) & 0xFFu;
                uint32_t code = (j & 1u) ? (byte >> 4) : (byte & 15u);
                if (KIND == 1) code += ((fifth >> (8 * i)) & 1u) << 4;
                v[i] = ds * (float)code - ms;
            }
        }
    }
    *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
}

/* Measurement aid: a kernel that only reads.  Each workgroup streams one
 * contiguous share of the buffer with 16-byte loads, four in flight per lane,
 * and folds the data into a value that is stored only if it matches a constant
 * (so the loads cannot be dropped).  What it reaches on a buffer is the rate
 * no GEMV over the same bytes can exceed on this device. */
__global__ __launch_bounds__(1024) void
k_read_probe(const u32x4 *__restrict__ p, size_t n16, uint32_t *__restrict__ sink)
{
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t b = (size_t)blockIdx.x * per, e = b + per < n16 ? b + per : n16;
    u32x4 acc = { 0u, 0u, 0u, 0u };
    size_t i = b + threadIdx.x;
    for (; i + 3u * blockDim.x < e; i += 4u * blockDim.x) {
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = __builtin_nontemporal_load(p + i + (size_t)k * blockDim.x);
#pragma unroll
        for (int k = 0; k < 4; k++) acc ^= v[k];
    }
    for (; i < e; i += blockDim.x) acc ^= p[i];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5EED5EEDu && sink) *sink = 1u;
}

/* Q3_K rows rewritten as Q6_K rows, exactly.  A Q3_K weight is d * (sc - 32) * (code - 4) with a
 * 3-bit code; Q6_K's is d * sc6 * (code6 - 32) with a 6-bit code and an int8 scale, over the same
 * sixteen groups in the same element order (element 128n + 32k + l).  With code6 = code + 28 and
 * sc6 = sc - 32 the two are the same integer times the same d, so the block term
 * d*dq*(float)(pos - 4*off) of oxk.c:624-652 and d*dq*(float)(pos - 32*minc) of oxk.c:913-964 are the
 * same float: the reference itself prepares Q3_K rows into its Q6_K batch layout (oxk.c:734-745).
 * Four lanes per block, split like the Q6_K GEMV: lane (n, lh) owns l = 16lh .. 16lh+15 of half n.
 *   low nibble of code + 28:  q2 | 12 when the third bit h is 0 (28 + q2 = 16 + 12 + q2), q2 when it
 *   is 1 (32 + q2);  upper two bits: 1 when h = 0, 2 when h = 1. */
__global__ __launch_bounds__(256) void
k_q3k_to_q6k(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, uint32_t n_blocks)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const uint32_t b = t >> 2, u = t & 3u, n = u >> 1, lh = u & 1u;
    if (b >= n_blocks) return;
    const uint8_t *s = src + (size_t)b * 110u;
    uint8_t *d = dst + (size_t)b * 210u;
    const U32x4u2 hm = *reinterpret_cast<const U32x4u2 *>(s + 16u * lh);
    const U32x4u2 qs = *reinterpret_cast<const U32x4u2 *>(s + 32u + 32u * n + 16u * lh);
    const uint32_t h4[4] = { hm.x, hm.y, hm.z, hm.w }, q4[4] = { qs.x, qs.y, qs.z, qs.w };
    uint32_t la[4], lb[4], hh[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t nib[4], hi2[4];
#pragma unroll
        for (uint32_t k = 0; k < 4u; k++) {
            const uint32_t q2 = (q4[i] >> (2u * k)) & 0x03030303u;
            const uint32_t h = (h4[i] >> (4u * n + k)) & 0x01010101u;
            const uint32_t nh = h ^ 0x01010101u;
            nib[k] = q2 | (nh << 2) | (nh << 3);
            hi2[k] = (h << 1) | nh;
        }
        la[i] = nib[0] | (nib[2] << 4);
        lb[i] = nib[1] | (nib[3] << 4);
        hh[i] = hi2[0] | (hi2[1] << 2) | (hi2[2] << 4) | (hi2[3] << 6);
    }
    U32x4u2 o;
    o.x = la[0]; o.y = la[1]; o.z = la[2]; o.w = la[3];
    *reinterpret_cast<U32x4u2 *>(d + 64u * n + 16u * lh) = o;
    o.x = lb[0]; o.y = lb[1]; o.z = lb[2]; o.w = lb[3];
    *reinterpret_cast<U32x4u2 *>(d + 64u * n + 32u + 16u * lh) = o;
    o.x = hh[0]; o.y = hh[1]; o.z = hh[2]; o.w = hh[3];
    *reinterpret_cast<U32x4u2 *>(d + 128u + 32u * n + 16u * lh) = o;
    if (u == 0u) {
        /* the sixteen 6-bit scales (oxk.c:556-573), minus 32, as int8; then d */
        const U32u2 *p = reinterpret_cast<const U32u2 *>(s + 96u);
        const uint32_t a0 = p[0].v, a1 = p[1].v, tt = p[2].v;
        uint32_t w[4];
        w[0] = (a0 & 0x0F0F0F0Fu) | ((tt & 0x03030303u) << 4);
        w[1] = (a1 & 0x0F0F0F0Fu) | (((tt >> 2) & 0x03030303u) << 4);
        w[2] = ((a0 >> 4) & 0x0F0F0F0Fu) | (((tt >> 4) & 0x03030303u) << 4);
        w[3] = ((a1 >> 4) & 0x0F0F0F0Fu) | (((tt >> 6) & 0x03030303u) << 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            /* x - 32 per byte, x in 0..63: clear bit 5 when set, else set the top three bits */
            const uint32_t below = (~w[i]) & 0x20202020u;
            w[i] = (w[i] & 0x1F1F1F1Fu) | below | (below << 1) | (below << 2);
        }
        o.x = w[0]; o.y = w[1]; o.z = w[2]; o.w = w[3];
        *reinterpret_cast<U32x4u2 *>(d + 192u) = o;
        *reinterpret_cast<uint16_t *>(d + 208u) = *reinterpret_cast<const uint16_t *>(s + 108u);
    }
}

/* Q6_K blocks regrouped for the decode kernels (the layout q6k_load<.., true> reads): inside every run of
 * eight consecutive blocks the 16-byte pieces a lane loads are stored piece-major.  One thread per
 * 16-byte destination piece, 105 pieces per group; same bytes, same size. */
__global__ __launch_bounds__(256) void
k_q6k_group(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, uint32_t n_groups)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const uint32_t grp = t / 105u, piece = t - grp * 105u;
    if (grp >= n_groups) return;
    const uint8_t *sg = src + (size_t)grp * Q6K_GROUP_BYTES;
    uint8_t *dg = dst + (size_t)grp * Q6K_GROUP_BYTES + 16u * piece;
    uint16_t v[8];
    if (piece < 104u) {
        const uint32_t part = piece >> 5;               /* 0 la, 1 lb, 2 hh, 3 scales */
        const uint32_t j = part < 3u ? (piece & 31u) >> 2 : piece & 7u;
        const uint32_t u = piece & 3u, n = u >> 1, lh = u & 1u;
        const uint32_t from = part == 0u ? 64u * n + 16u * lh
                            : part == 1u ? 64u * n + 32u + 16u * lh
                            : part == 2u ? 128u + 32u * n + 16u * lh : 192u;
        const uint16_t *sp = reinterpret_cast<const uint16_t *>(sg + 210u * j + from);   /* 2-byte aligned */
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = sp[i];
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = *reinterpret_cast<const uint16_t *>(sg + 210u * (uint32_t)i + 208u);
    }
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (uint32_t)v[2 * i] | ((uint32_t)v[2 * i + 1] << 16);
    *reinterpret_cast<u32x4 *>(dg) = u32x4{ o[0], o[1], o[2], o[3] };
}

/* Q2_K rows widened to 210-byte blocks for the tile kernel's Q2 mode.  A Q2_K weight is
 * d * sc * code - dmin * m with 4-bit sc and m per group of 16 and a 2-bit code (oxk.c:592-622), over
 * the groups and the element order of Q6_K.  sc * code is at most 45 and goes into the 6-bit field
 * of the Q6_K layout (low nibbles in bytes 0..127, upper two bits in bytes 128..191); bytes 192..199
 * take the sixteen minima as nibbles (group g in byte g / 2, even groups low), bytes 200..201 dmin,
 * bytes 202..207 zero, bytes 208..209 d.  Lane split as in k_q3k_to_q6k. */
__global__ __launch_bounds__(256) void
k_q2k_widen(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, uint32_t n_blocks)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const uint32_t b = t >> 2, u = t & 3u, n = u >> 1, lh = u & 1u;
    if (b >= n_blocks) return;
    const uint8_t *s = src + (size_t)b * 84u;
    uint8_t *d = dst + (size_t)b * 210u;
    const U32x4u2 sm = *reinterpret_cast<const U32x4u2 *>(s);
    const U32x4u2 qs = *reinterpret_cast<const U32x4u2 *>(s + 16u + 32u * n + 16u * lh);
    const uint32_t q4[4] = { qs.x, qs.y, qs.z, qs.w };
    const uint32_t sw[4] = { sm.x, sm.y, sm.z, sm.w };
    /* scale of group 8n + 2k + lh: byte 2k + lh of words 2n, 2n + 1 */
    uint32_t sc[4];
#pragma unroll
    for (uint32_t k = 0; k < 4u; k++) {
        const uint32_t word = n ? sw[2u + (k >> 1)] : sw[k >> 1];
        sc[k] = (word >> (16u * (k & 1u) + 8u * lh)) & 15u;
    }
    uint32_t la[4], lb[4], hh[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t p[4];
#pragma unroll
        for (uint32_t k = 0; k < 4u; k++)
            p[k] = ((q4[i] >> (2u * k)) & 0x03030303u) * sc[k];      /* at most 45 per byte: no carries */
        la[i] = (p[0] & 0x0F0F0F0Fu) | ((p[2] & 0x0F0F0F0Fu) << 4);
        lb[i] = (p[1] & 0x0F0F0F0Fu) | ((p[3] & 0x0F0F0F0Fu) << 4);
        hh[i] = ((p[0] >> 4) & 0x03030303u) | (((p[1] >> 4) & 0x03030303u) << 2) |
                (((p[2] >> 4) & 0x03030303u) << 4) | (((p[3] >> 4) & 0x03030303u) << 6);
    }
    U32x4u2 o;
    o.x = la[0]; o.y = la[1]; o.z = la[2]; o.w = la[3];
    *reinterpret_cast<U32x4u2 *>(d + 64u * n + 16u * lh) = o;
    o.x = lb[0]; o.y = lb[1]; o.z = lb[2]; o.w = lb[3];
    *reinterpret_cast<U32x4u2 *>(d + 64u * n + 32u + 16u * lh) = o;
    o.x = hh[0]; o.y = hh[1]; o.z = hh[2]; o.w = hh[3];
    *reinterpret_cast<U32x4u2 *>(d + 128u + 32u * n + 16u * lh) = o;
    if (u == 0u) {
        uint32_t pk[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t h = (sw[i] >> 4) & 0x0F0F0F0Fu, tt = h | (h >> 4);
            pk[i] = (tt & 0xFFu) | ((tt >> 8) & 0xFF00u);            /* four minima -> 16 bits */
        }
        const uint32_t dd = reinterpret_cast<const U32u2 *>(s + 80u)->v;    /* d | dmin << 16 */
        o.x = pk[0] | (pk[1] << 16);
        o.y = pk[2] | (pk[3] << 16);
        o.z = dd >> 16;
        o.w = 0u;
        *reinterpret_cast<U32x4u2 *>(d + 192u) = o;
        *reinterpret_cast<uint16_t *>(d + 208u) = (uint16_t)(dd & 0xFFFFu);
    }
}

#include "gemv_kernels.inc"
#include "mmq_kernels.inc"
#include "moe_kernels.inc"
#include "iq_kernels.inc"

/* ─── several GEMVs of one 32-value format in one launch ──────────────── */

/* A run of rows of one operation, given to one workgroup: what the GEMV kernel's steps need of it, in
 * device memory.  Workgroup b walks items[first[b]] .. items[first[b+1] - 1]. */
struct GemvMultiItem {
    SegInfo seg;                /* w and out already point at the run's first row; wg_begin 0 */
    GemvParams p;               /* act_out only in the item that holds the operation's first row */
    uint32_t same_x;            /* the previous item of this workgroup staged the same input */
    uint32_t pad[3];
};

/* the per-format pieces of the GEMV kernels (gemv_q8_0, gemv_legacy) under one name */
template <int WHICH> struct MultiFmt {
    typedef LegRegs Regs;
    static constexpr uint32_t BYTES = LegGeom<WHICH ? WHICH : 1>::BYTES;
};
template <> struct MultiFmt<0> {
    typedef Q80Regs Regs;
    static constexpr uint32_t BYTES = 34u;
};
template <int WHICH>
__device__ __forceinline__ void multi_load(typename MultiFmt<WHICH>::Regs &r, const WSrc &w, uint32_t g)
{
    if constexpr (WHICH == 0) q80_load<false>(r, w, g);
    else leg_load<WHICH, false>(r, w, g);
}
template <int WHICH>
__device__ __forceinline__ void
multi_pass(const typename MultiFmt<WHICH>::Regs &r, const GemvParams &p, const uint8_t *lds, uint32_t act_lds,
           uint32_t B, uint32_t g, uint32_t nblk, uint32_t row0, float *terms)
{
    if constexpr (WHICH == 0) q80_pass<1, false>(r, p, lds, act_lds, 1u, B, g, nblk, row0, terms);
    else leg_pass<WHICH, 1, false>(r, p, lds, act_lds, 1u, B, g, nblk, row0, terms);
}

/* what a wave needs of one item: the launch parameters and its share of the rows */
struct MultiState {
    GemvParams p;
    WaveWork ww;
    WSrc src;
    uint32_t nblk, same_x;
};

template <int WHICH>
__device__ __forceinline__ MultiState multi_state(const GemvMultiItem *it, uint32_t wave)
{
    MultiState st;
    st.p = it->p;
    st.ww.seg = it->seg;
    st.ww.seg.w = as_global(st.ww.seg.w);
    st.ww.seg.out = as_global(st.ww.seg.out);
    st.p.x = as_global(st.p.x);
    st.p.act_out = as_global(st.p.act_out);
    st.same_x = it->same_x;
    st.ww.seg_index = 0u;
    st.ww.wg_in_seg = 0u;
    const uint32_t q = st.ww.seg.rows_q, rem = st.ww.seg.rows_rem;
    st.ww.row0 = wave * q + min(wave, rem);
    st.ww.nrows = q + (wave < rem ? 1u : 0u);
    bool paired;
    st.src = wsrc_for<false>(st.ww, nullptr, st.p.blocks, MultiFmt<WHICH>::BYTES, st.nblk, paired);
    return st;
}

/* Operations that do not depend on each other (every input there when the launch starts) in ONE
 * launch, split in space rather than in time: the rows of all operations are cut into runs and
 * dealt to the workgroups so that every workgroup streams about the same number of bytes, and a
 * workgroup walks its few runs with the GEMV kernel's own steps (input quantised into LDS, passes over
 * two register sets, ordered row sums), requesting the next run's input and first two passes of
 * weights before it sums the rows of the current one.  No workgroup waits for another.  The matrices
 * of a Qwen2.5-0.5B-shaped Q8_0 model are 0.9-9 MB each: launched one by one a decode step of 97
 * matmuls takes 540 us, of which the kernels stream for a fifth, and walking the operations one after
 * the other with the whole grid still pays 3.5 us of staging, barrier, one pass and row sums per
 * operation.  WHICH: 0 = Q8_0, 1..5 = the LEG of gemv_legacy (Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS).  A row's
 * arithmetic does not depend on who owns it: same bits as the launches one by one. */
template <int WHICH>
__global__ __launch_bounds__(GEMV_MAX_THREADS) void
k_gemv_multi(const GemvMultiItem *__restrict__ items, const uint32_t *__restrict__ first)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    typedef typename MultiFmt<WHICH>::Regs Regs;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t i0 = first[blockIdx.x], i1 = first[blockIdx.x + 1u];
    if (i0 >= i1) return;
    MultiState cur = multi_state<WHICH>(items + i0, wave);
    XAhead xr = stage_begin<2, GEMV_PRO_NONE>(cur.ww.seg, cur.p, nullptr, lds, q80_lds_bytes(cur.p.blocks), 1u);
    Regs A, Bq;
    {
        const uint32_t last = cur.nblk ? cur.nblk - 1u : 0u;
        multi_load<WHICH>(A, cur.src, min(lane, last));
        multi_load<WHICH>(Bq, cur.src, min(64u + lane, last));
    }
    bool staged = false;
    for (uint32_t i = i0; i < i1; i++) {
        /* the next item's table entry, on its way while this one is staged and walked (the last item
         * stands in for the one after it: what is requested for that is never used) */
        const MultiState nxt = multi_state<WHICH>(items + min(i + 1u, i1 - 1u), wave);
        const uint32_t B = cur.p.blocks, act_lds = q80_lds_bytes(B);
        if (!(staged && cur.same_x))
            stage_end<2, GEMV_PRO_NONE>(xr, cur.ww.seg, cur.p, cur.ww.wg_in_seg, lds, act_lds, 1u,
                                        reinterpret_cast<float *>(lds + act_lds));
        staged = true;
        __syncthreads();
        float *const terms = reinterpret_cast<float *>(lds + act_lds) + (size_t)wave * cur.p.rows_cap * cur.p.term_stride;
        const uint32_t nblk = cur.nblk, last = nblk ? nblk - 1u : 0u, npass = (nblk + 63u) / 64u;
        if (nblk != 0u) {
            uint32_t k = 0;
            while (k + 3u < npass) {
                multi_pass<WHICH>(A, cur.p, lds, act_lds, B, k * 64u + lane, nblk, cur.ww.row0, terms);
                multi_load<WHICH>(A, cur.src, min((k + 2u) * 64u + lane, last));
                multi_pass<WHICH>(Bq, cur.p, lds, act_lds, B, (k + 1u) * 64u + lane, nblk, cur.ww.row0, terms);
                multi_load<WHICH>(Bq, cur.src, min((k + 3u) * 64u + lane, last));
                k += 2u;
            }
            const uint32_t rem = npass - k;                 /* 1, 2 or 3 */
            multi_pass<WHICH>(A, cur.p, lds, act_lds, B, k * 64u + lane, nblk, cur.ww.row0, terms);
            if (rem == 3u) multi_load<WHICH>(A, cur.src, min((k + 2u) * 64u + lane, last));
            if (rem >= 2u) multi_pass<WHICH>(Bq, cur.p, lds, act_lds, B, (k + 1u) * 64u + lane, nblk, cur.ww.row0, terms);
            if (rem == 3u) multi_pass<WHICH>(A, cur.p, lds, act_lds, B, (k + 2u) * 64u + lane, nblk, cur.ww.row0, terms);
        }
        /* the next item's input and first weights, requested before this one's rows are summed */
        xr = stage_begin<2, GEMV_PRO_NONE>(nxt.ww.seg, nxt.p, nullptr, lds, q80_lds_bytes(nxt.p.blocks), 1u);
        {
            const uint32_t nlast = nxt.nblk ? nxt.nblk - 1u : 0u;
            multi_load<WHICH>(A, nxt.src, min(lane, nlast));
            multi_load<WHICH>(Bq, nxt.src, min(64u + lane, nlast));
        }
        row_sums<1>(terms, lane, 1u, cur.ww.nrows, cur.p.rows_cap, B, cur.p.term_stride, cur.ww.seg.out,
                    cur.p.out_stride, cur.ww.row0);
        __syncthreads();        /* the next item keeps its terms (and maybe its input) where this one's were */
        cur = nxt;
    }
}

/* ─── host side of layer 2 ────────────────────────────────────────────── */

static hipError_t raise_all_lds_ceilings(void);
static int resolve_scratch(int device);

static std::atomic<int> g_device{-1};
static hipStream_t g_stream = nullptr;
static int g_n_cu = 0;
static std::mutex g_init_lock;

extern "C" int oxh_init(int device)
{
    if (g_device.load(std::memory_order_acquire) == device) return OXH_OK;
    std::lock_guard<std::mutex> hold(g_init_lock);
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
    const hipError_t e2 = raise_all_lds_ceilings();
    if (e2 != hipSuccess) {
        (void)hipStreamDestroy(g_stream);
        g_stream = nullptr;
        return hip_fail(e2, "hipFuncSetAttribute");
    }
    /* device `device` is current: look up where its copy of the static workspace lives */
    const int rs = resolve_scratch(device);
    if (rs) {
        (void)hipStreamDestroy(g_stream);
        g_stream = nullptr;
        return rs;
    }
    g_device.store(device, std::memory_order_release);
    return OXH_OK;
}

/* Everything the library made on the device goes: registered and cached weights, staging buffers, the
 * stream.  Buffers the caller got from oxh_malloc stay the caller's. */
extern "C" void oxh_shutdown(void)
{
    if (g_device < 0) return;
    oxh_internal_host_reset();
    std::lock_guard<std::mutex> hold(g_init_lock);
    if (g_stream) {
        (void)hipStreamSynchronize(g_stream);
        (void)hipStreamDestroy(g_stream);
    }
    g_stream = nullptr;
    g_device.store(-1, std::memory_order_release);
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
extern "C" int oxh_internal_n_cu(void) { return g_n_cu; }
extern "C" int oxh_internal_device(void) { return g_device.load(std::memory_order_acquire); }

/* AL5, AL6 and AL8 are the Q4_0, Q5_0 and Q8_0 block layouts under ids of
 * their own (oxidize-c/src/compute/quantization.c:207-214; the encoder
 * differs, the bytes and the dot do not: matvec.c:323-329). */
static uint32_t canon_qtype(uint32_t qtype)
{
    switch (qtype) {
    case OXH_AL5: return OXH_Q4_0;
    case OXH_AL6: return OXH_Q5_0;
    case OXH_AL8: return OXH_Q8_0;
    case OXH_Q3_K_S:                    /* one Q3_K layout under three ids */
    case OXH_Q3_K_L: return OXH_Q3_K_M;
    default:      return qtype;
    }
}

extern "C" int oxh_act_kind(uint32_t qtype, size_t cols)
{
    switch (canon_qtype(qtype)) {
    case OXH_Q4_0:
    case OXH_Q4_1:
    case OXH_Q5_0:
    case OXH_Q5_1:
    case OXH_AL5_XS:
    case OXH_Q8_0_T16:
    case OXH_Q8_0:   return (cols % OXH_QK8_0 == 0) ? 1 : 0;
    case OXH_Q2_K:
    case OXH_Q3_K_M:
    case OXH_Q4_K_S:
    case OXH_Q4_K_M:
    case OXH_Q5_K_S:
    case OXH_Q5_K_M:
    case OXH_Q6_K:
    case OXH_IQ3_S:                     /* the two codebook formats the reference's integer path takes */
    case OXH_IQ1_XXXS: return (cols % OXH_QK_K == 0) ? 2 : 0;
    case OXH_Q6_K_G8:  return (cols % (8u * OXH_QK_K) == 0) ? 2 : 0;     /* whole groups of eight blocks per row */
    case OXH_Q4_K_T16:
    case OXH_Q5_K_T16: return (cols % OXH_QK_K == 0) ? 2 : 0;
    default:         return 0;
    }
}

static size_t block_bytes(uint32_t qtype)
{
    switch (canon_qtype(qtype)) {
    case OXH_Q4_0:   return OXH_Q4_0_BYTES;
    case OXH_Q4_1:   return OXH_Q4_1_BYTES;
    case OXH_Q5_0:   return OXH_Q5_0_BYTES;
    case OXH_Q5_1:   return OXH_Q5_1_BYTES;
    case OXH_AL5_XS: return OXH_AL5_XS_BYTES;
    case OXH_Q8_0_T16:
    case OXH_Q8_0:   return OXH_Q8_0_BYTES;
    case OXH_Q4_K_S:
    case OXH_Q4_K_T16:
    case OXH_Q4_K_M: return OXH_Q4_K_BYTES;
    case OXH_Q5_K_S:
    case OXH_Q5_K_T16:
    case OXH_Q5_K_M: return OXH_Q5_K_BYTES;
    case OXH_Q6_K:
    case OXH_Q6_K_G8: return OXH_Q6_K_BYTES;
    case OXH_Q2_K:   return OXH_Q2_K_BYTES;
    case OXH_Q3_K_M: return OXH_Q3_K_BYTES;
    case OXH_IQ3_S:  return OXH_IQ3_S_BYTES;
    case OXH_IQ1_XXXS: return OXH_IQ1_XXXS_BYTES;
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

extern "C" size_t oxh_f32_path_row_bytes(uint32_t qtype, size_t cols)
{
    if (cols == 0) return 0;
    if (qtype == OXH_IQ4_NL) return cols % OXH_QK8_0 ? 0 : cols / OXH_QK8_0 * OXH_IQ4_NL_BYTES;
    if (qtype == OXH_IQ4_XS) return cols % OXH_QK_K ? 0 : cols / OXH_QK_K * OXH_IQ4_XS_BYTES;
    return 0;
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
                       (uint8_t *)d_act, (const uint32_t *)nullptr, (const float *)nullptr);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* the gather / SwiGLU forms used by the mixture-of-experts layer */
static int quantize_q8_k_ex(const float *d_x, size_t in_stride, size_t n_vec, size_t cols, void *d_act,
                            const uint32_t *d_row_index, const float *d_up, void *stream)
{
    const size_t bpv = cols / OXH_QK_K;
    if (n_vec == 0 || bpv == 0) return OXH_OK;
    if (bpv > 0xFFFFFFFFull / n_vec) return arg_fail("moe: too many blocks");
    const uint32_t total = (uint32_t)(bpv * n_vec);
    hipLaunchKernelGGL(k_quantize_q8_k, dim3((total + 3u) / 4u), dim3(256), 0,
                       pick_stream(stream), d_x, in_stride, (uint32_t)bpv, total,
                       (uint8_t *)d_act, d_row_index, d_up);
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

/* gfx950 has 160 KiB of LDS per CU; one workgroup may take all of it once the
 * kernel's dynamic-LDS ceiling is raised (done once in oxh_init). */
#define GEMV_LDS_LIMIT (160u * 1024u)

template <typename K>
static hipError_t raise_lds_ceiling(K kernel)
{
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMV_LDS_LIMIT);
}

static hipError_t raise_all_lds_ceilings(void)
{
    hipError_t e;
#define OXH_RAISE(KERNEL)                                                     \
    if ((e = raise_lds_ceiling(KERNEL<0, true>)) != hipSuccess) return e;     \
    if ((e = raise_lds_ceiling(KERNEL<1, false>)) != hipSuccess) return e;    \
    if ((e = raise_lds_ceiling(KERNEL<0, false>)) != hipSuccess) return e;
    OXH_RAISE(k_gemv_q4_k)
    OXH_RAISE(k_gemv_q5_k)
    OXH_RAISE(k_gemv_q6_k)
    OXH_RAISE(k_gemv_q6_kg)
    OXH_RAISE(k_gemv_q2_k)
    OXH_RAISE(k_gemv_q3_k)
    OXH_RAISE(k_gemv_q8_0)
    OXH_RAISE(k_gemv_q4_0)
    OXH_RAISE(k_gemv_q4_1)
    OXH_RAISE(k_gemv_q5_0)
    OXH_RAISE(k_gemv_q5_1)
    OXH_RAISE(k_gemv_al5_xs)
    OXH_RAISE(k_gemv_iq3_s)
    OXH_RAISE(k_gemv_iq1_xxxs)
#undef OXH_RAISE
    if ((e = raise_lds_ceiling(k_gemv_multi<0>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<4, 2, false>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<8, 2, false>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<16, 2, false>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_multi<8, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_multi<16, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<16, 2, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<1, 2, false>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<4, 2, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<8, 2, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_q80t_segments<1, 2, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_gemv_multi<1>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_gemv_multi<2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_gemv_multi<3>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_gemv_multi<4>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_gemv_multi<5>)) != hipSuccess) return e;
#define OXH_RAISE_PRO1(KERNEL, PRO)                                                               \
    if ((e = raise_lds_ceiling(KERNEL<1, PRO, false>)) != hipSuccess) return e;                   \
    if ((e = raise_lds_ceiling(KERNEL<0, PRO, false>)) != hipSuccess) return e;                   \
    if ((e = raise_lds_ceiling(KERNEL<1, PRO, true>)) != hipSuccess) return e;                    \
    if ((e = raise_lds_ceiling(KERNEL<0, PRO, true>)) != hipSuccess) return e;
#define OXH_RAISE_PRO(KERNEL)                                                                     \
    OXH_RAISE_PRO1(KERNEL, GEMV_PRO_NONE)                                                         \
    OXH_RAISE_PRO1(KERNEL, GEMV_PRO_RMSNORM)                                                      \
    OXH_RAISE_PRO1(KERNEL, GEMV_PRO_SWIGLU)                                                       \
    OXH_RAISE_PRO1(KERNEL, GEMV_PRO_ADD_RMSNORM)
    OXH_RAISE_PRO(k_gemv_q4_k_pro)
    OXH_RAISE_PRO(k_gemv_q5_k_pro)
    OXH_RAISE_PRO(k_gemv_q6_k_pro)
    OXH_RAISE_PRO(k_gemv_q6_kg_pro)
    OXH_RAISE_PRO(k_gemv_q2_k_pro)
    OXH_RAISE_PRO(k_gemv_q3_k_pro)
    OXH_RAISE_PRO(k_gemv_q8_0_pro)
    OXH_RAISE_PRO(k_gemv_q4_0_pro)
    OXH_RAISE_PRO(k_gemv_q4_1_pro)
    OXH_RAISE_PRO(k_gemv_q5_0_pro)
    OXH_RAISE_PRO(k_gemv_q5_1_pro)
    OXH_RAISE_PRO(k_gemv_al5_xs_pro)
    OXH_RAISE_PRO(k_gemv_iq3_s_pro)
    OXH_RAISE_PRO(k_gemv_iq1_xxxs_pro)
#undef OXH_RAISE_PRO
#undef OXH_RAISE_PRO1
    if ((e = raise_lds_ceiling(k_mmq_q4_k<8, 2, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q4_k<4, 1, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q5_k<8, 1, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q5_k<4, 1, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q4_k<8, 2, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q4_k<4, 1, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q5_k<8, 1, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q5_k<4, 1, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<8, 1, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<4, 1, 8>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<8, 1, 4>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<8, 1, 4, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<8, 1, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k<4, 1, 8, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 0>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 1>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 3>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 4>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mfma_q8_0_segments<4, 5>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<0>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<1>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<3>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<4>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q80<5>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_segments<1, 1, 4, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_split<2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_split<2, true>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_split<false, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_split<true, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_split<2, false, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_split<2, true, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_split<false, 2, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_split<true, 2, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_experts<1, 1, 4, 2>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q4_k_segments<1, 1, 8, 3>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_experts<1, 1, 8, false, 3>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q6_k_experts<4, 1, 8, 1>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_experts<4, 1, 8, false, 1>)) != hipSuccess) return e;
    if ((e = raise_lds_ceiling(k_mmq_q45_k_experts<4, 1, 8, true, 1>)) != hipSuccess) return e;
    return hipSuccess;
}

static bool is_q4k(uint32_t qtype) { return qtype == OXH_Q4_K_S || qtype == OXH_Q4_K_M; }
static bool is_q5k(uint32_t qtype) { return qtype == OXH_Q5_K_S || qtype == OXH_Q5_K_M; }
/* the tile-major forms of Q4_K and Q5_K, which only the MFMA tile kernels read, and the file type whose
 * arithmetic each one keeps */
static bool is_t16(uint32_t qtype) { return qtype == OXH_Q4_K_T16 || qtype == OXH_Q5_K_T16; }
static uint32_t t16_base(uint32_t qtype)
{
    return qtype == OXH_Q4_K_T16 ? OXH_Q4_K_M : (qtype == OXH_Q5_K_T16 ? OXH_Q5_K_M : qtype);
}
/* (OXH_Q8_0_T16, the tile-major form of Q8_0, has a kernel of its own: k_q80t_segments) */

static uint32_t act_lds_bytes(uint32_t qtype, uint32_t blocks)
{
    if (oxh_act_kind(qtype, 32) == 1) return q80_lds_bytes(blocks);
    qtype = canon_qtype(qtype);
    if (qtype == OXH_Q6_K || qtype == OXH_Q6_K_G8 || qtype == OXH_Q2_K || qtype == OXH_Q3_K_M)
        return q8k6_lds_bytes(blocks);
    return q8k_lds_bytes(blocks);
}

static bool is_iq(uint32_t qtype) { return qtype == OXH_IQ3_S || qtype == OXH_IQ1_XXXS; }

/* floats a block leaves in the term table: IQ3_S keeps eight running sums per row (oxk.c:1070-1086) */
static uint32_t terms_per_block(uint32_t qtype) { return qtype == OXH_IQ3_S ? 8u : 1u; }

static size_t gemv_lds_bytes(uint32_t qtype, uint32_t blocks, size_t n_vec, uint32_t waves,
                             uint32_t rows_cap)
{
    return n_vec * (size_t)act_lds_bytes(qtype, blocks) +
           (size_t)waves * n_vec * rows_cap * (terms_per_block(qtype) * blocks + 1u) * 4u +
           (is_iq(qtype) ? IQ_TABLE_BYTES : 0u);       /* the codebook */
}

static uint32_t env_u32(const char *name, uint32_t dflt, uint32_t lo, uint32_t hi)
{
    const char *e = getenv(name);
    if (!e || !*e) return dflt;
    const long v = strtol(e, nullptr, 10);
    if (v < (long)lo || v > (long)hi) return dflt;
    return (uint32_t)v;
}

/* Launch shape knobs (tuning aids; the defaults are what the benchmarks use):
 * OXH_GEMV_WAVES = waves per workgroup (1..16), OXH_GEMV_WG_PER_CU = how many
 * workgroups per compute unit the grid is sized for. */
static uint32_t gemv_waves(void)
{
    static uint32_t w = 0;
    if (!w) w = env_u32("OXH_GEMV_WAVES", 16, 1, 16);
    return w;
}

/* One 16-wave workgroup per CU is resident at a time.  A launch sized at one
 * workgroup per CU starts every wave at once, which is best while a wave has
 * only a handful of passes; past ~8 passes per wave a second round of
 * workgroups balances the tail better (measured: Q8_0 151936 x 896 goes from
 * 50 us to 35 us, the Llama decode shapes are best at one). */
static uint32_t gemv_wg_per_cu(size_t total_passes, uint32_t waves)
{
    static int forced = -1;
    if (forced < 0) forced = (int)env_u32("OXH_GEMV_WG_PER_CU", 0, 0, 64);
    if (forced > 0) return (uint32_t)forced;
    const size_t one_round = (size_t)(g_n_cu > 0 ? g_n_cu : 256) * waves;
    return total_passes > one_round * 8u ? 2u : 1u;
}

extern "C" size_t oxh_gemv_max_nvec(uint32_t qtype, size_t cols)
{
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) return 0;
    const size_t blocks = kind == 2 ? cols / OXH_QK_K : cols / OXH_QK8_0;
    if (blocks > 0xFFFFu) return 0;
    size_t nv = OXH_MAX_NV;
    while (nv > 0 && gemv_lds_bytes(qtype, (uint32_t)blocks, nv, 1, 1) > GEMV_LDS_LIMIT) nv--;
    return nv;
}

/* Launches over a 32-value format that hand over a buffer for the quantised activations run on the
 * MFMA kernel from five activations on, and that kernel takes up to sixteen. */
extern "C" size_t oxh_gemv_max_nvec_buffered(uint32_t qtype, size_t cols)
{
    const size_t plain = oxh_gemv_max_nvec(qtype, cols);
    if (oxh_act_kind(qtype, 32) != 1 || plain == 0) return plain;
    if (cols / OXH_QK8_0 * block_bytes(qtype) < 16u) return plain;
    static const uint32_t min_nv = env_u32("OXH_Q80_MFMA_MIN_NV", 5, 0, 64);
    if (min_nv == 0 || min_nv > MQ80_TOK) return plain;
    return (size_t)mq80_lds_bytes((uint32_t)(cols / OXH_QK8_0), MQ80_TOK, 4u) <= GEMV_LDS_LIMIT ? MQ80_TOK : plain;
}

struct GemvIo {
    const void *d_acts;     /* pre-quantised activations, or NULL            */
    const float *d_x;       /* f32 inputs to quantise in the kernel, or NULL */
    size_t x_stride;
    void *d_act_out;        /* optional store of the quantised bytes         */
    const OxhPrologue *pro; /* fused prologue in front of the quantiser, or NULL */
};

/* Q4_K, Q5_K and Q6_K with several activations per weight go to the matrix cores when the launch is
 * large enough for them: the dot-instruction GEMV repeats its integer work per activation (a launch
 * grows by 15-22 % per activation), while a tile kernel's workgroup needs 0.75 us per super-block of
 * its rows whatever the batch (1.2 us for Q6_K), so a launch of few tiles is paced by that and not by
 * the weight stream.  Measured (us, 2 / 3 / 4 / 6 / 8 activations, dot kernel against tiles):
 * 4096 x 4096 Q4_K 5.8 / 6.5 / 7.3 / 8.8 / 10.3 against 12.4; 6144 x 4096 7.3 / 8.4 / 9.5 / 11.7 / 13.8
 * against 12.6; 14336 x 4096 10.9 / 13.0 / 15.0 / 18.9 / 22.9 against 13.6; 28672 x 4096 15.4 / 18.7 /
 * 21.9 / 28.3 / 34.0 against 20.6; 4096 x 14336 Q6_K 14.3 / 17.0 / 19.6 / 24.7 / 42.8 against 66.  So:
 * tiles from four activations on where the launch has at least half a tile of 64 rows per CU, the
 * dot kernel below that (OXH_GEMV_MFMA_MIN_NV moves the first threshold, 0 = never;
 * OXH_GEMV_MFMA_MIN_TILES the second, in tiles).  Nine activations and more have no dot kernel.  The
 * MFMA kernel reads Q8_K activations, so an f32 launch qualifies only if it has somewhere to put the
 * quantised bytes. */
static bool gemv_wants_mfma(uint32_t qtype, const GemvIo &io, size_t max_nv, const int32_t *dump, size_t tiles64)
{
    static int min_nv = -1;
    if (min_nv < 0) min_nv = (int)env_u32("OXH_GEMV_MFMA_MIN_NV", 4, 0, 64);
    static const uint32_t min_tiles = env_u32("OXH_GEMV_MFMA_MIN_TILES", (uint32_t)(g_n_cu > 0 ? g_n_cu : 256) / 2u, 0, 1u << 20);
    if ((!is_q4k(qtype) && !is_q5k(qtype) && qtype != OXH_Q6_K) || dump || min_nv == 0 ||
        max_nv < (size_t)min_nv) return false;
    if (max_nv <= OXH_MAX_NV && tiles64 < min_tiles) return false;
    /* a prologue lives in the GEMV kernels' quantiser only */
    if (io.pro) return false;
    return io.d_acts != nullptr || io.d_act_out != nullptr;
}

/* The 64-row MFMA tile keeps one super-block per wave on its way; a launch with
 * at most two workgroups per CU cannot fill the memory system like that and
 * takes the variant with two super-blocks per stage (twice the LDS). */
static bool mmq_deep_stages(uint32_t wg)
{
    static const uint32_t force = env_u32("OXH_MMQ_DEEP", 2, 0, 2);     /* 0 never, 1 always, 2 by launch size */
    if (force < 2u) return force == 1u;
    return wg <= 2u * (uint32_t)(g_n_cu > 0 ? g_n_cu : 256);
}

/* Launches over a 32-value format (Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS) with five or more
 * activations per weight go to the MFMA kernel (OXH_Q80_MFMA_MIN_NV moves the threshold, 0 = never)
 * when the quantised activations exist or have somewhere to go and the staged activations fit LDS. */
static bool q80_wants_mfma(uint32_t qtype, const GemvIo &io, size_t max_nv, size_t blocks, const int32_t *dump,
                           size_t tiles64)
{
    static int min_nv = -1;
    if (min_nv < 0) min_nv = (int)env_u32("OXH_Q80_MFMA_MIN_NV", 5, 0, 64);
    /* as for the K-quants, a launch of few tiles is paced by a wave's walk over its rows' blocks and stays on
     * the dot kernel while that takes the batch (Q8_0, 5 / 6 / 8 activations: 4864 x 896 7.3 / 8.1 / 9.7 against
     * 9.4 us, 896 x 4864 13.4 / 14.8 / 17.9 against 25.8 us); OXH_Q80_MFMA_MIN_TILES moves the threshold */
    static const uint32_t min_tiles = env_u32("OXH_Q80_MFMA_MIN_TILES", (uint32_t)(g_n_cu > 0 ? g_n_cu : 256) / 2u, 0, 1u << 20);
    if (oxh_act_kind(qtype, 32) != 1 || dump || io.pro || min_nv == 0 || max_nv < (size_t)min_nv ||
        max_nv > MQ80_TOK)
        return false;
    if (max_nv <= OXH_MAX_NV && tiles64 < min_tiles) return false;
    if (blocks * block_bytes(qtype) < 16u) return false;        /* rows shorter than one 16-byte piece */
    if ((size_t)mq80_lds_bytes((uint32_t)blocks, max_nv > 8 ? 16u : 8u, 4u) > GEMV_LDS_LIMIT) return false;
    return io.d_acts != nullptr || io.d_act_out != nullptr;
}

static int launch_q80_mfma_segments(uint32_t qtype, const OxhSegment *segs, size_t n_segs, size_t cols, size_t blocks,
                                    const GemvIo &io, size_t n_vec_default, size_t n_acts, size_t out_stride,
                                    void *stream)
{
    const uint8_t *acts = (const uint8_t *)io.d_acts;
    if (!acts) {
        int rc = oxh_quantize_q8_0(io.d_x, io.x_stride, n_acts, cols, io.d_act_out, stream);
        if (rc) return rc;
        acts = (const uint8_t *)io.d_act_out;
    }
    /* Tiles of 64 rows per workgroup.  With more than eight activations staged only one workgroup fits a
     * compute unit, and a workgroup that owned one tile would ask for its rows, wait, compute and leave
     * with nothing on its way meanwhile: such launches give a workgroup several tiles in a row (as many as
     * leaves every unit four workgroups or so, at most eight), the next tile's rows requested while the
     * current one is computed and the activations staged once for all of them: vocabulary head 151936 x
     * 896 at 16 activations 73 -> 61 us.  With eight or fewer staged, two workgroups share a unit and
     * cover for each other; there it measured 2-4 % slower and is not used.  OXH_Q80_MFMA_GROUPS fixes
     * the number. */
    size_t tiles = 0, most_nv = 0;
    for (size_t i = 0; i < n_segs; i++) {
        tiles += (segs[i].rows + 63u) / 64u;
        const size_t nv = segs[i].n_vec ? segs[i].n_vec : n_vec_default;
        if (segs[i].rows && nv > most_nv) most_nv = nv;
    }
    static const uint32_t forced_groups = env_u32("OXH_Q80_MFMA_GROUPS", 0, 0, 64);
    const size_t per_cu4 = 4u * (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    uint32_t groups = forced_groups ? forced_groups : (most_nv > 8u ? (uint32_t)(tiles / per_cu4) : 1u);
    if (groups < 1u) groups = 1u;
    if (!forced_groups && groups > 8u) groups = 8u;
    SegTable t;
    memset(&t, 0, sizeof t);
    uint32_t wg = 0, n = 0;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows == 0) continue;
        t.s[n].w = (const uint8_t *)segs[i].d_w;
        t.s[n].out = segs[i].d_out;
        t.s[n].rows = (uint32_t)segs[i].rows;
        t.s[n].act_first = (uint32_t)segs[i].act_first;
        t.s[n].nv = (uint32_t)(segs[i].n_vec ? segs[i].n_vec : n_vec_default);
        t.s[n].wg_begin = wg;
        wg += (uint32_t)((segs[i].rows + 64u * groups - 1u) / (64u * groups));
        n++;
    }
    t.n = n;
    for (uint32_t i = 1; i < 4 && i < n; i++) t.bound[i - 1] = t.s[i].wg_begin;
    uint32_t toks = 8u;
    for (uint32_t i = 0; i < n; i++) if (t.s[i].nv > 8u) toks = 16u;
    const size_t lds = mq80_lds_bytes((uint32_t)blocks, toks, 4u);
    hipStream_t st = pick_stream(stream);
#define OXH_MQ80(LEG) hipLaunchKernelGGL((k_mfma_q8_0_segments<4, LEG>), dim3(wg), dim3(256), lds, st, t, \
                                         (uint32_t)blocks, acts, out_stride, toks, groups)
    switch (qtype) {
    case OXH_Q4_0:   OXH_MQ80(1); break;
    case OXH_Q4_1:   OXH_MQ80(2); break;
    case OXH_Q5_0:   OXH_MQ80(3); break;
    case OXH_Q5_1:   OXH_MQ80(4); break;
    case OXH_AL5_XS: OXH_MQ80(5); break;
    default:         OXH_MQ80(0); break;
    }
#undef OXH_MQ80
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* Tile-major Q8_0: every wave streams a run of consecutive 16-row groups straight into registers.  Eight
 * (or four) waves share a workgroup's staged activations; a launch with fewer groups than would give every
 * CU four four-wave workgroups runs one wave per workgroup instead, so that a small matrix still spreads
 * over the device.  Groups per wave: as many as leave about four workgroups per CU, at most 32; measured on
 * the 151936 x 896 head, more and shorter waves win (one group per wave 31.9 us at eight activations, two
 * 34.0, four 37): a wave keeps two to four units on their way, and it is the number of waves that fills the
 * memory system
 * (OXH_Q80T_GPW fixes the number, OXH_Q80T_WAVES the waves per workgroup). */
static int launch_q80t_segments(const OxhSegment *segs, size_t n_segs, size_t cols, size_t blocks, const GemvIo &io,
                                size_t n_vec_default, size_t n_acts, size_t out_stride, void *stream)
{
    size_t n_groups = 0, most_nv = 0;
    for (size_t i = 0; i < n_segs; i++) {
        n_groups += (segs[i].rows + 15u) / 16u;
        const size_t nv = segs[i].n_vec ? segs[i].n_vec : n_vec_default;
        if (segs[i].rows && nv > most_nv) most_nv = nv;
        if (segs[i].rows > 0xFFFFFFF0ull / (blocks * 34u)) return arg_fail("gemv: segment too large");
    }
    if (blocks % 4u) {
        snprintf(g_err, sizeof g_err, "gemv: tile-major Q8_0 needs columns in whole runs of four blocks (cols %zu)", cols);
        return OXH_DECLINED;
    }
    const size_t image = blocks * Q80T_ACT_BLOCK;
    if (image > GEMV_LDS_LIMIT) {
        snprintf(g_err, sizeof g_err, "gemv: %zu columns x 16 staged activations do not fit 160 KiB of LDS", cols);
        return OXH_ERR_TOO_WIDE;
    }
    static const uint32_t forced_gpw = env_u32("OXH_Q80T_GPW", 0, 0, 1024);
    static const uint32_t forced_waves = env_u32("OXH_Q80T_WAVES", 0, 0, 16);
    const size_t cus = (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    /* Waves per workgroup: a wave per row group is all the parallelism there is, so the smallest workgroup
     * with which every group's wave is resident at once (a compute unit holds 32 waves, and as many
     * workgroups as their staged activations leave LDS for: one, for 4864 columns); launches with more
     * groups than that run in rounds of eight-wave workgroups.  24 matrices of 896 x 4864 in one launch
     * (1344 groups, 87 KB of LDS per workgroup): one wave per workgroup is one wave per compute unit. */
    uint32_t waves = 8u;
    for (uint32_t w = 1u; w <= 16u; w = w == 1u ? 4u : 2u * w) {
        const size_t wg_per_cu = GEMV_LDS_LIMIT / image ? GEMV_LDS_LIMIT / image : 1u;
        const size_t per_cu = wg_per_cu * w < 32u ? wg_per_cu * w : 32u;
        if (cus * per_cu >= n_groups) { waves = w; break; }
    }
    if (forced_waves == 1u || forced_waves == 4u || forced_waves == 8u || forced_waves == 16u) waves = forced_waves;
    const size_t lds = image;
    /* f32 inputs: with up to four activations per segment the workgroups quantise them themselves while
     * they stage them (a launch less: head at one activation 28.4 against 30 us, at four 30.5 against 31.1);
     * with more, that work, repeated by every workgroup, costs what the quantiser's launch costs (eight
     * activations 32.6 against 32.1 us, sixteen 39 against 33.5), and one-wave workgroups would each repeat
     * all of it.  Without a buffer for the blocks there is no choice.  (OXH_Q80T_FUSE_NV moves the
     * threshold.) */
    static const uint32_t fuse_nv = env_u32("OXH_Q80T_FUSE_NV", 4, 0, 16);
    bool fused = false;
    uint8_t *acts = (uint8_t *)const_cast<void *>(io.d_acts);
    if (!acts) {
        fused = !io.d_act_out || (most_nv <= fuse_nv && waves >= 4u);
        acts = (uint8_t *)io.d_act_out;
        if (fused && io.x_stride > 0xFFFFFFFFull) return arg_fail("gemv: stride too large");
        if (!fused) {
            int rc = oxh_quantize_q8_0(io.d_x, io.x_stride, n_acts, cols, io.d_act_out, stream);
            if (rc) return rc;
        }
    }
    size_t gpw = forced_gpw ? forced_gpw : n_groups / (waves * 4u * cus);
    if (gpw < 1u) gpw = 1u;
    if (!forced_gpw && gpw > 32u) gpw = 32u;
    SegTable t;
    memset(&t, 0, sizeof t);
    uint32_t wg = 0, n = 0;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows == 0) continue;
        t.s[n].w = (const uint8_t *)segs[i].d_w;
        t.s[n].out = segs[i].d_out;
        t.s[n].rows = (uint32_t)segs[i].rows;
        t.s[n].act_first = (uint32_t)segs[i].act_first;
        t.s[n].nv = (uint32_t)(segs[i].n_vec ? segs[i].n_vec : n_vec_default);
        t.s[n].wg_begin = wg;
        const size_t groups = (segs[i].rows + 15u) / 16u;
        wg += (uint32_t)((groups + waves * gpw - 1u) / (waves * gpw));
        n++;
    }
    t.n = n;
    for (uint32_t i = 1; i < 4 && i < n; i++) t.bound[i - 1] = t.s[i].wg_begin;
    hipStream_t st = pick_stream(stream);
#define OXH_Q80T(WAVES, FUSED) hipLaunchKernelGGL((k_q80t_segments<WAVES, 2, FUSED>), dim3(wg), dim3(WAVES * 64), lds, \
                                                  st, t, (uint32_t)blocks, acts, out_stride, (uint32_t)gpw, io.d_x,   \
                                                  (uint32_t)io.x_stride)
    if (waves == 16u) { if (fused) OXH_Q80T(16, true); else OXH_Q80T(16, false); }
    else if (waves == 8u) { if (fused) OXH_Q80T(8, true); else OXH_Q80T(8, false); }
    else if (waves == 4u) { if (fused) OXH_Q80T(4, true); else OXH_Q80T(4, false); }
    else { if (fused) OXH_Q80T(1, true); else OXH_Q80T(1, false); }
#undef OXH_Q80T
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

static int launch_mmq_segments(uint32_t qtype, const OxhSegment *segs, size_t n_segs, size_t cols, size_t blocks,
                               const GemvIo &io, size_t n_vec_default, size_t n_acts,
                               size_t out_stride, void *stream, uint32_t tile_major = 0u)
{
    typedef MmqGeom<1, 1, 4> G;
    if (blocks * 292u * 256u > 0xFFFFFFFFull) return arg_fail("gemv: cols too large");
    const uint8_t *acts = (const uint8_t *)io.d_acts;
    if (!acts) {
        int rc = oxh_quantize_q8_k(io.d_x, io.x_stride, n_acts, cols, io.d_act_out, stream);
        if (rc) return rc;
        acts = (const uint8_t *)io.d_act_out;
    }
    /* A Q4_K launch whose 64-row tiles would give at most two workgroups per CU, but whose 128-row tiles
     * still give nearly every CU one, can take those on eight waves with three super-blocks per stage: half as
     * much again in flight per CU.  Off by default (OXH_MOE_WIDE_SMALL=1 switches it on): launched
     * continuously, Mixtral's down projections at 16 tokens run faster on the 64-row tiles with two
     * super-blocks per stage (an expert step 154.5 against 158.5 us); the wider tile only won when the
     * launches were timed right after an idle period. */
    static const uint32_t wide_ok = env_u32("OXH_MOE_WIDE_SMALL", 0, 0, 1);
    const size_t cus = (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    size_t wg64 = 0, wg128 = 0;
    for (size_t i = 0; i < n_segs; i++) {
        wg64 += (segs[i].rows + 63) / 64;
        wg128 += (segs[i].rows + 127) / 128;
    }
    const bool wide = wide_ok && is_q4k(qtype) && wg64 <= 2u * cus && wg128 >= cus - cus / 8;
    const size_t tile_rows = wide ? 128 : G::ROWS;
    SegTable t;
    memset(&t, 0, sizeof t);
    uint32_t wg = 0, n = 0;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows == 0) continue;
        t.s[n].w = (const uint8_t *)segs[i].d_w;
        t.s[n].out = segs[i].d_out;
        t.s[n].rows = (uint32_t)segs[i].rows;
        t.s[n].act_first = (uint32_t)segs[i].act_first;
        t.s[n].nv = (uint32_t)(segs[i].n_vec ? segs[i].n_vec : n_vec_default);
        t.s[n].wg_begin = wg;
        wg += (uint32_t)((segs[i].rows + tile_rows - 1) / tile_rows);
        n++;
    }
    t.n = n;
    for (uint32_t i = 1; i < 4 && i < n; i++) t.bound[i - 1] = t.s[i].wg_begin;
    if (wide) {
        typedef MmqGeom<1, 1, 8> W4;
        static_assert(W4::ROWS == 128, "128-row tiles");
        hipLaunchKernelGGL((k_mmq_q4_k_segments<1, 1, 8, 3>), dim3(wg), dim3(512), 3 * W4::LDS_BYTES,
                           pick_stream(stream), t, (uint32_t)blocks, acts, out_stride, tile_major);
        HIP_TRY(hipGetLastError());
        return OXH_OK;
    }
    typedef Mmq6Geom<1, 1, 4> G6;                           /* same 64-row tiles */
    typedef MmqGeom<1, 1, 4, true> G5;
    static_assert(G6::ROWS == G::ROWS && G5::ROWS == G::ROWS, "segment tiling is shared by all formats");
    hipStream_t st = pick_stream(stream);
    const uint32_t nb = (uint32_t)blocks;
#define OXH_SEG_LAUNCH(KERNEL, GEOM, KB, ...)                                                         \
    hipLaunchKernelGGL((KERNEL<1, 1, 4, KB>), dim3(wg), dim3(4 * 64), (KB) * GEOM::LDS_BYTES, st, t, nb, acts, \
                       out_stride, ##__VA_ARGS__)
    if (mmq_deep_stages(wg)) {
        if (qtype == OXH_Q6_K) OXH_SEG_LAUNCH(k_mmq_q6_k_segments, G6, 2);
        else if (is_q5k(qtype)) OXH_SEG_LAUNCH(k_mmq_q5_k_segments, G5, 2, tile_major);
        else OXH_SEG_LAUNCH(k_mmq_q4_k_segments, G, 2, tile_major);
    } else {
        if (qtype == OXH_Q6_K) OXH_SEG_LAUNCH(k_mmq_q6_k_segments, G6, 1);
        else if (is_q5k(qtype)) OXH_SEG_LAUNCH(k_mmq_q5_k_segments, G5, 1, tile_major);
        else OXH_SEG_LAUNCH(k_mmq_q4_k_segments, G, 1, tile_major);
    }
#undef OXH_SEG_LAUNCH
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

static int launch_gemv(uint32_t qtype, const OxhSegment *segs, size_t n_segs, size_t cols,
                       const GemvIo &io, size_t n_vec, size_t out_stride, int32_t *dump,
                       void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    qtype = canon_qtype(qtype);
    if (n_segs == 0) return OXH_OK;
    if (!segs || (!io.d_acts && !io.d_x)) return arg_fail("gemv: NULL pointer");
    if (n_vec < 1 || n_vec > MQ80_TOK) return arg_fail("gemv: n_vec must be 1..8");
    const size_t n_vec_default = n_vec;
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) {
        snprintf(g_err, sizeof g_err, "gemv: qtype %u with cols %zu has no integer path", qtype, cols);
        return OXH_DECLINED;
    }
    if (n_segs > OXH_MAX_SEGS) {
        /* A launch's segment table holds 32: more segments go out in launches of 32, over activations that
         * are quantised once for all of them (f32 inputs need the buffer for the quantised bytes). */
        if (dump || io.pro) return arg_fail("gemv: more than 32 segments take no prologue and no sub-block dump");
        GemvIo each = io;
        if (!io.d_acts) {
            if (!io.d_act_out) return arg_fail("gemv: more than 32 segments over f32 inputs need d_act_out");
            size_t act_end = 0;
            for (size_t i = 0; i < n_segs; i++) {
                const size_t nv = segs[i].n_vec ? segs[i].n_vec : n_vec;
                if (nv > MQ80_TOK || segs[i].act_first > 0xFFFFFFFFull) return arg_fail("gemv: segment n_vec or act_first out of range");
                if (segs[i].rows && segs[i].act_first + nv > act_end) act_end = segs[i].act_first + nv;
            }
            if (act_end == 0) return OXH_OK;
            rc = kind == 2 ? oxh_quantize_q8_k(io.d_x, io.x_stride, act_end, cols, io.d_act_out, stream)
                           : oxh_quantize_q8_0(io.d_x, io.x_stride, act_end, cols, io.d_act_out, stream);
            if (rc) return rc;
            each.d_acts = io.d_act_out;
            each.d_x = nullptr;
            each.d_act_out = nullptr;
        }
        for (size_t k = 0; k < n_segs; k += OXH_MAX_SEGS) {
            const size_t n = n_segs - k < OXH_MAX_SEGS ? n_segs - k : OXH_MAX_SEGS;
            if ((rc = launch_gemv(qtype, segs + k, n, cols, each, n_vec, out_stride, nullptr, stream))) return rc;
        }
        return OXH_OK;
    }
    const size_t blocks = kind == 2 ? cols / OXH_QK_K : cols / OXH_QK8_0;
    if (blocks > 0xFFFFu) {
        snprintf(g_err, sizeof g_err, "gemv: cols %zu too wide", cols);
        return OXH_ERR_TOO_WIDE;
    }
    if (io.d_x && io.x_stride < cols) return arg_fail("gemv: x_stride < cols");
    size_t total_rows = 0, max_act = 0, act_end = 0;     /* act_end: one past the last activation any segment reads */
    /* a segment may carry its own activation count; the launch value is the default */
    size_t max_nv = 0;
    bool all_one = true, any_pair = false;
    /* a paired segment walks two matrices: it counts twice wherever work is sized */
    size_t total_work = 0, tiles64 = 0;
    for (size_t i = 0; i < n_segs; i++) {
        const size_t nv = segs[i].n_vec ? segs[i].n_vec : n_vec;
        if (nv < 1 || nv > MQ80_TOK) return arg_fail("gemv: segment n_vec must be 1..8");
        if (segs[i].rows) {
            if (nv > max_nv) max_nv = nv;
            if (nv != 1) all_one = false;
            if (segs[i].d_w_pair) any_pair = true;
        }
        if (segs[i].rows > 0x3FFFFFFFull / (blocks * 16u)) return arg_fail("gemv: segment too large");
        if (segs[i].rows && (!segs[i].d_w || !segs[i].d_out)) return arg_fail("gemv: NULL segment pointer");
        total_rows += segs[i].rows;
        tiles64 += (segs[i].rows + 63u) / 64u;
        total_work += segs[i].rows * (segs[i].d_w_pair ? 2u : 1u);
        if (segs[i].act_first > max_act) max_act = segs[i].act_first;
        if (segs[i].rows && segs[i].act_first + nv > act_end) act_end = segs[i].act_first + nv;
    }
    if (total_rows == 0) return OXH_OK;
    if (qtype == OXH_Q8_0_T16) {
        if (any_pair || dump || io.pro) {
            snprintf(g_err, sizeof g_err, "gemv: tile-major Q8_0 takes no paired segment, prologue or sub-block dump");
            return OXH_DECLINED;
        }
        return launch_q80t_segments(segs, n_segs, cols, blocks, io, n_vec_default, act_end, out_stride, stream);
    }
    if (is_t16(qtype)) {
        /* tile-major weights exist for the MFMA tile kernel alone, whatever the launch's size */
        if (any_pair || dump || io.pro || (!io.d_acts && !io.d_act_out)) {
            snprintf(g_err, sizeof g_err, "gemv: tile-major weights (type %u) take quantised activations or a buffer "
                     "for them, and no paired segment, prologue or sub-block dump", qtype);
            return OXH_DECLINED;
        }
        return launch_mmq_segments(t16_base(qtype), segs, n_segs, cols, blocks, io, n_vec_default, act_end,
                                   out_stride, stream, 1u);
    }
    if (any_pair && dump) return arg_fail("gemv: no sub-block dump of a paired launch");
    if (is_iq(qtype) && dump) return arg_fail("gemv: no sub-block dump for the codebook formats");
    if (!any_pair && gemv_wants_mfma(qtype, io, max_nv, dump, tiles64))
        return launch_mmq_segments(qtype, segs, n_segs, cols, blocks, io, n_vec_default, act_end,
                                   out_stride, stream);
    if (!any_pair && q80_wants_mfma(qtype, io, max_nv, blocks, dump, tiles64))
        return launch_q80_mfma_segments(qtype, segs, n_segs, cols, blocks, io, n_vec_default, act_end,
                                        out_stride, stream);
    /* only that kernel takes 9 to 16 activations per weight */
    if (max_nv > OXH_MAX_NV)
        return arg_fail("gemv: n_vec must be 1..8 (up to 16 only where the launch runs on the matrix cores: "
                        "not Q2_K or Q3_K, a buffer for the quantised activations, staged activations within LDS)");
    n_vec = max_nv;                        /* sizes LDS from here on */
    if (out_stride > 0xFFFFFFFFull || io.x_stride > 0xFFFFFFFFull || max_act + n_vec > 0xFFFFFFFFull)
        return arg_fail("gemv: stride too large");

    /* Deal workgroups to segments in proportion to their rows; every wave
     * then owns ceil(rows / waves) whole rows of its segment. */
    uint32_t W = gemv_waves();
    const size_t blocks_per_pass = kind == 1 ? 64u : 16u;
    const size_t target = (size_t)(g_n_cu > 0 ? g_n_cu : 256) *
                          gemv_wg_per_cu(total_work * blocks / blocks_per_pass, W);
    uint32_t cap_limit = GEMV_ROWS_CAP;
    uint32_t n_wg[OXH_MAX_SEGS];
    uint32_t rows_cap = 1;
    for (;;) {
        rows_cap = 1;
        for (size_t i = 0; i < n_segs; i++) {
            const size_t rows = segs[i].rows;
            if (rows == 0) { n_wg[i] = 0; continue; }
            const size_t mult = segs[i].d_w_pair ? 2u : 1u;     /* table rows per owned row */
            size_t share = (target * rows * mult + total_work / 2) / total_work;
            const size_t own_limit = cap_limit / mult ? cap_limit / mult : 1u;
            const size_t lo = (rows + (size_t)W * own_limit - 1) / ((size_t)W * own_limit);
            const size_t hi = (rows + W - 1) / W;
            if (share < lo) share = lo;
            if (share > hi) share = hi;
            if (share < 1) share = 1;
            n_wg[i] = (uint32_t)share;
            const uint32_t rpw = (uint32_t)((rows + share * W - 1) / (share * W) * mult);   /* (q + (rem != 0)) * mult */
            if (rpw > rows_cap) rows_cap = rpw;
        }
        if (gemv_lds_bytes(qtype, (uint32_t)blocks, n_vec, W, rows_cap) <= GEMV_LDS_LIMIT) break;
        if (cap_limit > 1) { cap_limit = rows_cap > 1 ? rows_cap - 1 : 1; continue; }
        if (W > 1) { W /= 2; cap_limit = GEMV_ROWS_CAP; continue; }
        snprintf(g_err, sizeof g_err, "gemv: cols %zu x n_vec %zu does not fit 160 KiB of LDS", cols, n_vec);
        return OXH_ERR_TOO_WIDE;
    }
    const size_t lds = gemv_lds_bytes(qtype, (uint32_t)blocks, n_vec, W, rows_cap);

    GemvParams p;
    memset(&p, 0, sizeof p);
    p.blocks = (uint32_t)blocks;
    p.magic = (uint32_t)((0x100000000ull + blocks - 1u) / blocks);
    p.act_bytes = (uint32_t)oxh_act_bytes(qtype, cols);
    p.out_stride = (uint32_t)out_stride;
    p.term_stride = terms_per_block(qtype) * p.blocks + 1u;
    p.rows_cap = rows_cap;
    p.x = io.d_x;
    p.x_stride = (uint32_t)io.x_stride;
    p.act_out = (uint8_t *)io.d_act_out;
    p.dump = dump;
    uint32_t pro = io.pro ? io.pro->kind : 0u;
    if (pro) {
        p.pro_b = io.pro->d_b;
        p.pro_out = io.pro->d_out;
        p.pro_eps = io.pro->eps;
        p.pro_add = io.pro->d_add;
        p.pro_sum_out = io.pro->d_sum_out;
        if (pro == OXH_PRO_RMSNORM && io.pro->d_add) pro = GEMV_PRO_ADD_RMSNORM;
    }

    SegTable t;
    memset(&t, 0, sizeof t);
    PairTable pairs;
    memset(&pairs, 0, sizeof pairs);
    uint32_t wg = 0, n = 0;
    for (size_t i = 0; i < n_segs; i++) {
        if (segs[i].rows == 0) continue;
        t.s[n].w = (const uint8_t *)segs[i].d_w;
        pairs.w2[n] = (const uint8_t *)segs[i].d_w_pair;
        t.s[n].out = segs[i].d_out;
        t.s[n].rows = (uint32_t)segs[i].rows;
        t.s[n].act_first = (uint32_t)segs[i].act_first;
        t.s[n].nv = (uint32_t)(segs[i].n_vec ? segs[i].n_vec : n_vec_default);
        t.s[n].wg_begin = wg;
        t.s[n].rows_q = (uint32_t)(segs[i].rows / ((size_t)n_wg[i] * W));
        t.s[n].rows_rem = (uint32_t)(segs[i].rows % ((size_t)n_wg[i] * W));
        wg += n_wg[i];
        n++;
    }
    t.n = n;
    for (uint32_t i = 1; i < 4 && i < n; i++) t.bound[i - 1] = t.s[i].wg_begin;

    const dim3 grid(wg), block(W * 64u);
    hipStream_t st = pick_stream(stream);
    const uint8_t *a = (const uint8_t *)io.d_acts;
#define OXH_LAUNCH(KERNEL)                                                              \
    do {                                                                                \
        if (dump)            hipLaunchKernelGGL((KERNEL<0, true>), grid, block, lds, st, t, p, a);  \
        else if (all_one)    hipLaunchKernelGGL((KERNEL<1, false>), grid, block, lds, st, t, p, a); \
        else                 hipLaunchKernelGGL((KERNEL<0, false>), grid, block, lds, st, t, p, a); \
    } while (0)
#define OXH_LAUNCH_PRO(KERNEL, PRO)                                                     \
    do {                                                                                \
        if (any_pair) {                                                                 \
            if (all_one) hipLaunchKernelGGL((KERNEL<1, PRO, true>), grid, block, lds, st, t, p, a, pairs);  \
            else         hipLaunchKernelGGL((KERNEL<0, PRO, true>), grid, block, lds, st, t, p, a, pairs);  \
        } else {                                                                        \
            if (all_one) hipLaunchKernelGGL((KERNEL<1, PRO, false>), grid, block, lds, st, t, p, a, pairs); \
            else         hipLaunchKernelGGL((KERNEL<0, PRO, false>), grid, block, lds, st, t, p, a, pairs); \
        }                                                                               \
    } while (0)
#define OXH_LAUNCH_ANY(PLAIN, WITH_PRO)                                                 \
    do {                                                                                \
        if (pro == GEMV_PRO_ADD_RMSNORM) OXH_LAUNCH_PRO(WITH_PRO, GEMV_PRO_ADD_RMSNORM); \
        else if (pro == OXH_PRO_RMSNORM) OXH_LAUNCH_PRO(WITH_PRO, GEMV_PRO_RMSNORM);    \
        else if (pro == OXH_PRO_SWIGLU) OXH_LAUNCH_PRO(WITH_PRO, GEMV_PRO_SWIGLU);      \
        else if (any_pair)              OXH_LAUNCH_PRO(WITH_PRO, GEMV_PRO_NONE);        \
        else                            OXH_LAUNCH(PLAIN);                              \
    } while (0)
    if (is_q4k(qtype))          OXH_LAUNCH_ANY(k_gemv_q4_k, k_gemv_q4_k_pro);
    else if (is_q5k(qtype))     OXH_LAUNCH_ANY(k_gemv_q5_k, k_gemv_q5_k_pro);
    else if (qtype == OXH_Q6_K) OXH_LAUNCH_ANY(k_gemv_q6_k, k_gemv_q6_k_pro);
    else if (qtype == OXH_Q6_K_G8) OXH_LAUNCH_ANY(k_gemv_q6_kg, k_gemv_q6_kg_pro);
    else if (qtype == OXH_Q2_K) OXH_LAUNCH_ANY(k_gemv_q2_k, k_gemv_q2_k_pro);
    else if (qtype == OXH_Q3_K_M) OXH_LAUNCH_ANY(k_gemv_q3_k, k_gemv_q3_k_pro);
    else if (qtype == OXH_Q4_0) OXH_LAUNCH_ANY(k_gemv_q4_0, k_gemv_q4_0_pro);
    else if (qtype == OXH_Q4_1) OXH_LAUNCH_ANY(k_gemv_q4_1, k_gemv_q4_1_pro);
    else if (qtype == OXH_Q5_0) OXH_LAUNCH_ANY(k_gemv_q5_0, k_gemv_q5_0_pro);
    else if (qtype == OXH_Q5_1) OXH_LAUNCH_ANY(k_gemv_q5_1, k_gemv_q5_1_pro);
    else if (qtype == OXH_AL5_XS) OXH_LAUNCH_ANY(k_gemv_al5_xs, k_gemv_al5_xs_pro);
    else if (qtype == OXH_IQ3_S) OXH_LAUNCH_ANY(k_gemv_iq3_s, k_gemv_iq3_s_pro);
    else if (qtype == OXH_IQ1_XXXS) OXH_LAUNCH_ANY(k_gemv_iq1_xxxs, k_gemv_iq1_xxxs_pro);
    else                        OXH_LAUNCH_ANY(k_gemv_q8_0, k_gemv_q8_0_pro);
#undef OXH_LAUNCH_ANY
#undef OXH_LAUNCH_PRO
#undef OXH_LAUNCH
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_gemv_segments(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                                 size_t cols, const void *d_acts, size_t n_vec,
                                 size_t out_stride, void *stream)
{
    if (!d_acts && n_segs) return arg_fail("oxh_gemv_segments: NULL activations");
    const GemvIo io = { d_acts, nullptr, 0, nullptr, nullptr };
    return launch_gemv(qtype, segs, n_segs, cols, io, n_vec, out_stride, nullptr, stream);
}

/* IQ4_NL / IQ4_XS: the weights expanded on the fly against the f32 inputs themselves, a launch per
 * segment.  There is no quantised activation to hand back. */
static int launch_gemv_iq4(uint32_t qtype, const OxhSegment *segs, size_t n_segs, size_t cols, const float *d_x,
                           size_t x_stride, void *d_act_out, size_t n_vec, size_t out_stride, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    const size_t rb = oxh_f32_path_row_bytes(qtype, cols);
    if (rb == 0) {
        snprintf(g_err, sizeof g_err, "oxh_gemv_segments_f32: qtype %u with cols %zu is not a whole number of blocks", qtype, cols);
        return OXH_DECLINED;
    }
    if (d_act_out) return arg_fail("oxh_gemv_segments_f32: these types run on the f32 inputs, there are no quantised activations to return");
    if (n_segs == 0) return OXH_OK;
    if (!segs) return arg_fail("oxh_gemv_segments_f32: NULL segments");
    if (x_stride < cols || (x_stride & 3u) || ((uintptr_t)d_x & 15u))
        return arg_fail("oxh_gemv_segments_f32: input rows must be 16-byte aligned and x_stride >= cols");
    const size_t lds = 64u + cols * sizeof(float);
    if (lds > 160u * 1024u || cols > 0xFFFFFFFFull || rb > 0xFFFFFFFFull) {
        snprintf(g_err, sizeof g_err, "oxh_gemv_segments_f32: cols %zu too wide for one workgroup's LDS", cols);
        return OXH_ERR_TOO_WIDE;
    }
    const bool xs = qtype == OXH_IQ4_XS;
    const void *kern = xs ? reinterpret_cast<const void *>(k_gemv_iq4_f32<true>) : reinterpret_cast<const void *>(k_gemv_iq4_f32<false>);
    HIP_TRY(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipStream_t st = pick_stream(stream);
    const uint32_t n_cu = (uint32_t)(g_n_cu > 0 ? g_n_cu : 256);
    for (size_t k = 0; k < n_segs; k++) {
        const OxhSegment &sg = segs[k];
        const size_t nv = sg.n_vec ? sg.n_vec : n_vec;
        if (sg.rows == 0 || nv == 0) continue;
        if (!sg.d_w || !sg.d_out) return arg_fail("oxh_gemv_segments_f32: NULL segment pointer");
        if (sg.d_w_pair) return arg_fail("oxh_gemv_segments_f32: paired segments need an integer-path type");
        if (out_stride < sg.rows || sg.rows > 0xFFFFFFFFull || nv > 0xFFFFFFFFull)
            return arg_fail("oxh_gemv_segments_f32: out_stride < rows or too many rows");
        /* enough workgroups for eight waves per SIMD at most, every wave with a row */
        const uint32_t grid = (uint32_t)((sg.rows + 3u) / 4u < 8u * n_cu ? (sg.rows + 3u) / 4u : 8u * n_cu);
        const float *x = d_x + sg.act_first * x_stride;
        if (xs) hipLaunchKernelGGL(k_gemv_iq4_f32<true>, dim3(grid), dim3(256), lds, st, (const uint8_t *)sg.d_w, (uint32_t)sg.rows,
                                   (uint32_t)cols, (uint32_t)rb, x, x_stride, (uint32_t)nv, sg.d_out, out_stride);
        else    hipLaunchKernelGGL(k_gemv_iq4_f32<false>, dim3(grid), dim3(256), lds, st, (const uint8_t *)sg.d_w, (uint32_t)sg.rows,
                                   (uint32_t)cols, (uint32_t)rb, x, x_stride, (uint32_t)nv, sg.d_out, out_stride);
        HIP_TRY(hipGetLastError());
    }
    return OXH_OK;
}

extern "C" int oxh_gemv_segments_f32(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                                     size_t cols, const float *d_x, size_t x_stride,
                                     void *d_act_out, size_t n_vec, size_t out_stride,
                                     void *stream)
{
    if (!d_x && n_segs) return arg_fail("oxh_gemv_segments_f32: NULL input");
    if (qtype == OXH_IQ4_NL || qtype == OXH_IQ4_XS)
        return launch_gemv_iq4(qtype, segs, n_segs, cols, d_x, x_stride, d_act_out, n_vec, out_stride, stream);
    const GemvIo io = { nullptr, d_x, x_stride, d_act_out, nullptr };
    return launch_gemv(qtype, segs, n_segs, cols, io, n_vec, out_stride, nullptr, stream);
}

/* ─── plans over the 32-value formats (oxh_plan_* hands them here) ────── */

struct GemvMulti {
    GemvMultiItem *d_items;
    Q80tItem *d_titems;         /* which == MULTI_TILED */
    uint32_t *d_first;
    uint32_t n_ops, n_items, grid, waves;
    int which;
    size_t lds;
};
#define MULTI_TILED 6           /* tile-major Q8_0, up to sixteen activations per segment */

static int mmq80_leg(uint32_t qtype);

extern "C" int oxh_internal_multi_which(uint32_t qtype)
{
    if (qtype == OXH_Q8_0_T16) return MULTI_TILED;
    qtype = canon_qtype(qtype);
    if (qtype == OXH_Q8_0) return 0;
    const int leg = mmq80_leg(qtype);
    return leg >= 1 ? leg : -1;
}

/* Plans over tile-major Q8_0.  Every segment is cut into runs of whole 16-row groups, a run's cost for
 * its workgroup being the units its busiest wave streams (groups shared between the waves, a group's
 * units = blocks / 4), and the runs are dealt to the least loaded workgroup in turn, the segments with
 * the longest rows first (their runs are the coarsest), each workgroup taking as many rounds of a
 * segment as still fit its share: a workgroup's items are few and mostly consecutive runs of one
 * operation, so its activations are staged once. */
static int multi_create_tiled(const OxhPlanOp *ops, size_t n_ops, void **handle)
{
    const uint32_t n_cu = (uint32_t)(g_n_cu > 0 ? g_n_cu : 256);
    static const uint32_t forced_waves = env_u32("OXH_Q80T_PLAN_WAVES", 0, 0, 16);
    struct Piece { uint32_t op, seg, runs, groups, nv; };
    size_t n_pieces = 0, max_blocks = 0;
    for (size_t i = 0; i < n_ops; i++) {
        const OxhPlanOp &o = ops[i];
        if (o.qtype != OXH_Q8_0_T16 || o.pro || !o.segs || o.n_segs == 0 || !o.d_x || o.cols == 0 || o.cols % 128u) {
            snprintf(g_err, sizeof g_err, "plan: operation %zu: the operations of a plan over tile-major Q8_0 are all of "
                     "that form (cols a multiple of 128), without prologue, with segments and an input", i);
            return OXH_DECLINED;
        }
        const size_t blocks = o.cols / OXH_QK8_0;
        if (blocks * Q80T_ACT_BLOCK > GEMV_LDS_LIMIT) {
            snprintf(g_err, sizeof g_err, "plan: operation %zu: cols %zu too wide for one workgroup", i, o.cols);
            return OXH_ERR_TOO_WIDE;
        }
        if (blocks > max_blocks) max_blocks = blocks;
        size_t live = 0;
        for (size_t k = 0; k < o.n_segs; k++) {
            const OxhSegment &sg = o.segs[k];
            if (!sg.rows) continue;
            const size_t nv = sg.n_vec ? sg.n_vec : 1u;
            if (nv > 16u || sg.d_w_pair || !sg.d_w || !sg.d_out || sg.rows > 0x3FFFFFFFull || sg.act_first > 0xFFFFFFu)
                return arg_fail("plan: tile-major segments have 1..16 activations, a matrix and an output, and are unpaired");
            if (nv > 1u && (o.out_stride == 0 || o.out_stride > 0xFFFFFFFFull))
                return arg_fail("plan: an operation with several activations per segment needs out_stride");
            live++;
        }
        if (live == 0) return arg_fail("plan: an operation has no rows");
        n_pieces += live;
    }
    /* LDS of a workgroup: the widest operation's staged activations.  Sixteen waves, one workgroup per
     * compute unit (eight: two where LDS holds two) */
    const size_t lds = max_blocks * Q80T_ACT_BLOCK;
    const uint32_t waves = forced_waves == 8u || forced_waves == 16u ? forced_waves : 16u;
    const uint32_t per_cu = (waves == 8u && 2u * lds <= GEMV_LDS_LIMIT) ? 2u : 1u;
    const uint32_t n_wg = n_cu * per_cu;

    Piece *pieces = (Piece *)calloc(n_pieces, sizeof *pieces);
    double *load = (double *)calloc(n_wg, sizeof *load);
    uint32_t *count = (uint32_t *)calloc(n_wg + 1u, sizeof *count);
    if (!pieces || !load || !count) {
        free(pieces); free(load); free(count);
        snprintf(g_err, sizeof g_err, "out of host memory building a plan");
        return OXH_ERR_NOMEM;
    }
    size_t np = 0, cap_items = 0;
    double total = 0.0;
    for (size_t i = 0; i < n_ops; i++)
        for (size_t k = 0; k < ops[i].n_segs; k++) {
            const OxhSegment &sg = ops[i].segs[k];
            if (!sg.rows) continue;
            Piece &pc = pieces[np++];
            pc.op = (uint32_t)i;
            pc.seg = (uint32_t)k;
            pc.runs = (uint32_t)(ops[i].cols / 128u);
            pc.groups = (uint32_t)((sg.rows + 15u) / 16u);
            pc.nv = (uint32_t)(sg.n_vec ? sg.n_vec : 1u);
            total += (double)pc.groups / waves * pc.runs;
            cap_items += pc.groups / waves + 2u;
        }
    /* longest rows first; the order of the operations otherwise (insertion sort: stable) */
    for (size_t a = 1; a < np; a++) {
        const Piece key = pieces[a];
        size_t b = a;
        while (b > 0 && pieces[b - 1].runs < key.runs) { pieces[b] = pieces[b - 1]; b--; }
        pieces[b] = key;
    }
    struct Dealt { Q80tItem it; uint32_t wg; };
    Dealt *dealt = (Dealt *)calloc(cap_items, sizeof *dealt);
    if (!dealt) {
        free(pieces); free(load); free(count);
        snprintf(g_err, sizeof g_err, "out of host memory building a plan");
        return OXH_ERR_NOMEM;
    }
    const double target = total / n_wg;
    size_t n_items = 0;
    for (size_t a = 0; a < np; a++) {
        const Piece &pc = pieces[a];
        const OxhPlanOp &o = ops[pc.op];
        const OxhSegment &sg = o.segs[pc.seg];
        const uint32_t B = 4u * pc.runs;
        /* the first run of a segment stores the quantised activations unless an earlier segment of the
         * operation has stored the same ones */
        bool keep = o.d_act_out != nullptr;
        for (size_t k = 0; k < pc.seg && keep; k++) {
            const OxhSegment &e = o.segs[k];
            if (e.rows && e.act_first == sg.act_first && (e.n_vec ? e.n_vec : 1u) >= pc.nv) keep = false;
        }
        uint32_t g = 0;
        while (g < pc.groups) {
            uint32_t wg = 0;
            for (uint32_t w = 1; w < n_wg; w++) if (load[w] < load[wg]) wg = w;
            const double room = target - load[wg];
            uint32_t rounds = room >= (double)pc.runs ? (uint32_t)(room / (double)pc.runs) : 1u;
            if (rounds > 0xFFFFu) rounds = 0xFFFFu;
            uint32_t take = pc.groups - g;
            if (take > rounds * waves) take = rounds * waves;
            if (n_items >= cap_items) {          /* cannot happen: every item but a segment's last is a whole round */
                free(pieces); free(load); free(count); free(dealt);
                return arg_fail("plan: item table overflow");
            }
            Dealt &d = dealt[n_items++];
            d.wg = wg;
            d.it.w = (const uint8_t *)sg.d_w + (size_t)g * pc.runs * Q80T_UNIT;
            d.it.out = sg.d_out;
            d.it.x = o.d_x + sg.act_first * o.cols;
            d.it.keep = keep ? (uint8_t *)o.d_act_out + sg.act_first * (size_t)B * 34u : nullptr;
            d.it.row0 = 16u * g;
            d.it.rows = (uint32_t)sg.rows;
            d.it.groups = take;
            d.it.B = B;
            d.it.nv = pc.nv;
            d.it.out_stride = (uint32_t)o.out_stride;
            d.it.same_x = 0;
            d.it.pad = 0;
            keep = false;
            load[wg] += (double)((take + waves - 1u) / waves) * pc.runs;
            count[wg + 1u]++;
            g += take;
        }
    }
    /* the table in workgroup order (a workgroup's items in the order they were dealt) */
    Q80tItem *h = (Q80tItem *)calloc(n_items ? n_items : 1u, sizeof *h);
    uint32_t *first = count;                    /* counts -> first indices, in place */
    uint32_t *fill = (uint32_t *)calloc(n_wg, sizeof *fill);
    if (!h || !fill) {
        free(pieces); free(load); free(count); free(dealt); free(h); free(fill);
        snprintf(g_err, sizeof g_err, "out of host memory building a plan");
        return OXH_ERR_NOMEM;
    }
    for (uint32_t w = 0; w < n_wg; w++) first[w + 1u] += first[w];
    for (size_t k = 0; k < n_items; k++) {
        const uint32_t w = dealt[k].wg;
        const uint32_t at = first[w] + fill[w]++;
        h[at] = dealt[k].it;
        if (fill[w] > 1u) {
            const Q80tItem &pv = h[at - 1u];
            h[at].same_x = (pv.x == h[at].x && pv.B == h[at].B && pv.nv == h[at].nv && !h[at].keep) ? 1u : 0u;
        }
    }
    free(pieces); free(load); free(dealt); free(fill);
    int rc = OXH_OK;
    GemvMulti *m = (GemvMulti *)calloc(1, sizeof *m);
    if (!m) { snprintf(g_err, sizeof g_err, "out of host memory building a plan"); rc = OXH_ERR_NOMEM; }
    if (!rc) {
        hipError_t e = hipMalloc((void **)&m->d_titems, (n_items ? n_items : 1u) * sizeof *h);
        if (e == hipSuccess) e = hipMalloc((void **)&m->d_first, (size_t)(n_wg + 1u) * sizeof *first);
        if (e == hipSuccess) e = hipMemcpy(m->d_titems, h, (n_items ? n_items : 1u) * sizeof *h, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = hipMemcpy(m->d_first, first, (size_t)(n_wg + 1u) * sizeof *first, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            if (m->d_titems) (void)hipFree(m->d_titems);
            if (m->d_first) (void)hipFree(m->d_first);
            free(m);
            m = nullptr;
            rc = hip_fail(e, "plan table");
        }
    }
    free(h);
    free(count);
    if (rc) return rc;
    m->n_ops = (uint32_t)n_ops;
    m->n_items = (uint32_t)n_items;
    m->grid = n_wg;
    m->waves = waves;
    m->which = MULTI_TILED;
    m->lds = lds;
    *handle = m;
    return OXH_OK;
}

/* Cuts the rows of all operations into runs of at most 16 x rows_cap rows (what a workgroup's term
 * tables hold) and deals them in order: a workgroup is full when it has its share of the bytes. */
extern "C" int oxh_internal_multi_create(const OxhPlanOp *ops, size_t n_ops, void **handle)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (!ops || !handle || n_ops == 0 || n_ops > 0xFFFFu) return arg_fail("plan: 1..65535 operations");
    *handle = nullptr;
    const int which = oxh_internal_multi_which(ops[0].qtype);
    if (which < 0) {
        snprintf(g_err, sizeof g_err, "plan: qtype %u has no multi-operation launch", ops[0].qtype);
        return OXH_DECLINED;
    }
    if (which == MULTI_TILED) return multi_create_tiled(ops, n_ops, handle);
    const uint32_t W = GEMV_MAX_THREADS / 64u;
    const uint32_t n_cu = (uint32_t)(g_n_cu > 0 ? g_n_cu : 256);
    /* pass 1: check, and add up the bytes */
    double total = 0.0;
    for (size_t i = 0; i < n_ops; i++) {
        const OxhPlanOp &o = ops[i];
        if (oxh_internal_multi_which(o.qtype) != which || o.pro || !o.segs || o.n_segs == 0 || !o.d_x ||
            oxh_act_kind(o.qtype, o.cols) != 1) {
            snprintf(g_err, sizeof g_err, "plan: operation %zu: the operations of a plan over a 32-value format are of "
                     "that one format (cols a multiple of 32), without prologue, with segments and an input", i);
            return OXH_DECLINED;
        }
        const size_t blocks = o.cols / OXH_QK8_0;
        if (blocks > 0xFFFFu || gemv_lds_bytes(o.qtype, (uint32_t)blocks, 1, W, 1) > GEMV_LDS_LIMIT) {
            snprintf(g_err, sizeof g_err, "plan: operation %zu: cols %zu too wide for one workgroup", i, o.cols);
            return OXH_ERR_TOO_WIDE;
        }
        size_t live = 0;
        for (size_t k = 0; k < o.n_segs; k++) {
            const OxhSegment &sg = o.segs[k];
            if (!sg.rows) continue;
            if (sg.act_first != 0 || sg.n_vec > 1 || sg.d_w_pair || !sg.d_w || !sg.d_out || sg.rows > 0x3FFFFFFFull)
                return arg_fail("plan: segments over activation 0, one vector, unpaired, with matrix and output");
            total += (double)sg.rows * (double)oxh_row_bytes(o.qtype, o.cols);
            live++;
        }
        if (live == 0) return arg_fail("plan: an operation has no rows");
    }
    const double target = total / n_cu;
    /* pass 2: the runs.  Sized generously first (a run has at least 16 rows unless the segment ends) */
    size_t cap_items = 0;
    for (size_t i = 0; i < n_ops; i++)
        for (size_t k = 0; k < ops[i].n_segs; k++) cap_items += ops[i].segs[k].rows / 16u + 2u;
    cap_items += n_cu;
    GemvMultiItem *h = (GemvMultiItem *)calloc(cap_items, sizeof *h);
    uint32_t *first = (uint32_t *)calloc(n_cu + 1u, sizeof *first);
    if (!h || !first) {
        free(h);
        free(first);
        snprintf(g_err, sizeof g_err, "out of host memory building a plan");
        return OXH_ERR_NOMEM;
    }
    uint32_t wg = 0, n_items = 0;
    double used = 0.0;
    size_t lds = 0;
    const void *prev_x = nullptr;
    size_t prev_cols = 0;
    bool wg_empty = true;
    for (size_t i = 0; i < n_ops; i++) {
        const OxhPlanOp &o = ops[i];
        const uint32_t blocks = (uint32_t)(o.cols / OXH_QK8_0);
        const size_t row_bytes = oxh_row_bytes(o.qtype, o.cols);
        uint32_t cap = GEMV_ROWS_CAP;
        while (cap > 1u && gemv_lds_bytes(o.qtype, blocks, 1, W, cap) > GEMV_LDS_LIMIT) cap--;
        const size_t run_max = (size_t)W * cap;
        bool op_first = true;
        for (size_t k = 0; k < o.n_segs; k++) {
            const OxhSegment &sg = o.segs[k];
            size_t r = 0;
            while (r < sg.rows) {
                if (!wg_empty && used >= target && wg + 1u < n_cu) {        /* this workgroup has its share */
                    wg++;
                    first[wg] = n_items;
                    used = 0.0;
                    wg_empty = true;
                    prev_x = nullptr;
                }
                size_t take = sg.rows - r;
                if (take > run_max) take = run_max;
                const double room = target - used;
                size_t fit = room > 0.0 ? (size_t)(room / (double)row_bytes) : 0u;
                fit = (fit + 15u) & ~(size_t)15u;                            /* whole rows per wave, rounded up */
                if (fit < 16u) fit = 16u;
                if (wg + 1u < n_cu && take > fit) take = fit;
                GemvMultiItem &it = h[n_items++];
                it.seg.w = (const uint8_t *)sg.d_w + r * row_bytes;
                it.seg.out = sg.d_out + r;
                it.seg.rows = (uint32_t)take;
                it.seg.act_first = 0;
                it.seg.wg_begin = 0;
                it.seg.rows_q = (uint32_t)(take / W);
                it.seg.rows_rem = (uint32_t)(take % W);
                it.seg.nv = 1;
                it.p.blocks = blocks;
                it.p.magic = (uint32_t)((0x100000000ull + blocks - 1u) / blocks);
                it.p.act_bytes = (uint32_t)oxh_act_bytes(o.qtype, o.cols);
                it.p.out_stride = 0;
                it.p.term_stride = terms_per_block(o.qtype) * blocks + 1u;
                it.p.rows_cap = (uint32_t)((take + W - 1u) / W);
                it.p.x = o.d_x;
                it.p.x_stride = (uint32_t)o.cols;
                it.p.act_out = op_first ? (uint8_t *)o.d_act_out : nullptr;
                it.same_x = (!wg_empty && prev_x == (const void *)o.d_x && prev_cols == o.cols && !it.p.act_out) ? 1u : 0u;
                const size_t need = gemv_lds_bytes(o.qtype, blocks, 1, W, it.p.rows_cap);
                if (need > lds) lds = need;
                op_first = false;
                wg_empty = false;
                prev_x = o.d_x;
                prev_cols = o.cols;
                used += (double)take * (double)row_bytes;
                r += take;
            }
        }
    }
    const uint32_t grid = wg + 1u;
    for (uint32_t b = grid; b <= n_cu; b++) first[b] = n_items;
    first[grid] = n_items;
    GemvMulti *m = (GemvMulti *)calloc(1, sizeof *m);
    if (!m) { snprintf(g_err, sizeof g_err, "out of host memory building a plan"); rc = OXH_ERR_NOMEM; }
    if (!rc) {
        hipError_t e = hipMalloc((void **)&m->d_items, (size_t)n_items * sizeof *h);
        if (e == hipSuccess) e = hipMalloc((void **)&m->d_first, (size_t)(grid + 1u) * sizeof *first);
        if (e == hipSuccess) e = hipMemcpy(m->d_items, h, (size_t)n_items * sizeof *h, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = hipMemcpy(m->d_first, first, (size_t)(grid + 1u) * sizeof *first, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            if (m->d_items) (void)hipFree(m->d_items);
            if (m->d_first) (void)hipFree(m->d_first);
            free(m);
            m = nullptr;
            rc = hip_fail(e, "plan table");
        }
    }
    free(h);
    free(first);
    if (rc) return rc;
    m->n_ops = (uint32_t)n_ops;
    m->n_items = n_items;
    m->grid = grid;
    m->which = which;
    m->lds = lds;
    *handle = m;
    return OXH_OK;
}

extern "C" int oxh_internal_multi_launch(void *handle, void *stream)
{
    GemvMulti *m = (GemvMulti *)handle;
    if (!m) return arg_fail("plan: NULL");
    hipStream_t st = pick_stream(stream);
    if (m->which == MULTI_TILED) {
        const dim3 tgrid(m->grid);
        if (m->waves == 16u)
            hipLaunchKernelGGL((k_q80t_multi<16, 2>), tgrid, dim3(1024), m->lds, st, m->d_titems, m->d_first);
        else
            hipLaunchKernelGGL((k_q80t_multi<8, 2>), tgrid, dim3(512), m->lds, st, m->d_titems, m->d_first);
        HIP_TRY(hipGetLastError());
        return OXH_OK;
    }
    const dim3 grid(m->grid), block(GEMV_MAX_THREADS);
#define OXH_MULTI(WHICH) hipLaunchKernelGGL((k_gemv_multi<WHICH>), grid, block, m->lds, st, m->d_items, m->d_first)
    switch (m->which) {
    case 1:  OXH_MULTI(1); break;
    case 2:  OXH_MULTI(2); break;
    case 3:  OXH_MULTI(3); break;
    case 4:  OXH_MULTI(4); break;
    case 5:  OXH_MULTI(5); break;
    default: OXH_MULTI(0); break;
    }
#undef OXH_MULTI
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" void oxh_internal_multi_info(const void *handle, size_t *n_items, size_t *workgroups, size_t *lds_bytes)
{
    const GemvMulti *m = (const GemvMulti *)handle;
    if (n_items) *n_items = m->n_items;
    if (workgroups) *workgroups = m->grid;
    if (lds_bytes) *lds_bytes = m->lds;
}

extern "C" int oxh_internal_multi_destroy(void *handle)
{
    GemvMulti *m = (GemvMulti *)handle;
    if (!m) return OXH_OK;
    hipError_t e = hipFree(m->which == MULTI_TILED ? (void *)m->d_titems : (void *)m->d_items);
    const hipError_t e2 = hipFree(m->d_first);
    free(m);
    if (e == hipSuccess) e = e2;
    if (e != hipSuccess) return hip_fail(e, "hipFree");
    return OXH_OK;
}

extern "C" int oxh_gemv_segments_fused(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                                       size_t cols, const float *d_x, size_t x_stride,
                                       const OxhPrologue *pro, void *d_act_out, size_t n_vec,
                                       size_t out_stride, void *stream)
{
    if (!d_x && n_segs) return arg_fail("oxh_gemv_segments_fused: NULL input");
    if (pro) {
        if (pro->kind != OXH_PRO_RMSNORM && pro->kind != OXH_PRO_SWIGLU)
            return arg_fail("oxh_gemv_segments_fused: unknown prologue kind");
        if ((pro->d_add || pro->d_sum_out) && pro->kind != OXH_PRO_RMSNORM)
            return arg_fail("oxh_gemv_segments_fused: d_add / d_sum_out go with OXH_PRO_RMSNORM");
        if (pro->d_sum_out && !pro->d_add)
            return arg_fail("oxh_gemv_segments_fused: d_sum_out without d_add");
        if (!pro->d_b && n_segs) return arg_fail("oxh_gemv_segments_fused: prologue operand is NULL");
        if (pro->kind == OXH_PRO_RMSNORM && !(pro->eps >= 0.0f))
            return arg_fail("oxh_gemv_segments_fused: eps must be >= 0");
        /* every workgroup reads all of x while the first one of each segment
         * stores the result: the two must not overlap */
        if ((pro->d_out || pro->d_sum_out) && n_segs) {
            size_t max_act = 0;
            for (size_t i = 0; i < n_segs; i++) {
                const size_t nv = segs[i].n_vec ? segs[i].n_vec : n_vec;
                if (segs[i].rows && segs[i].act_first + nv > max_act) max_act = segs[i].act_first + nv;
            }
            const size_t span = max_act ? ((max_act - 1) * x_stride + cols) * sizeof(float) : 0;
            const size_t bspan = pro->kind == OXH_PRO_SWIGLU ? span : cols * sizeof(float);
            const char *ins[3] = { (const char *)d_x, (const char *)pro->d_b, (const char *)pro->d_add };
            const size_t in_span[3] = { span, bspan, span };
            const char *outs[2] = { (const char *)pro->d_out, (const char *)pro->d_sum_out };
            for (int o = 0; o < 2; o++) {
                if (!outs[o]) continue;
                for (int i = 0; i < 3; i++)
                    if (ins[i] && outs[o] < ins[i] + in_span[i] && ins[i] < outs[o] + span)
                        return arg_fail("oxh_gemv_segments_fused: a stored result overlaps an input");
            }
            if (outs[0] && outs[1] && outs[0] < outs[1] + span && outs[1] < outs[0] + span)
                return arg_fail("oxh_gemv_segments_fused: the two stored results overlap");
        }
    }
    const GemvIo io = { nullptr, d_x, x_stride, d_act_out, pro };
    return launch_gemv(qtype, segs, n_segs, cols, io, n_vec, out_stride, nullptr, stream);
}

extern "C" int oxh_debug_read_probe(const void *d_buf, size_t bytes, uint32_t *d_sink, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (!d_buf || ((uintptr_t)d_buf & 15u)) return arg_fail("oxh_debug_read_probe: buffer must be 16-byte aligned");
    if (bytes < 16) return OXH_OK;
    hipLaunchKernelGGL(k_read_probe, dim3((uint32_t)(g_n_cu > 0 ? g_n_cu : 256)), dim3(1024), 0, pick_stream(stream),
                       (const u32x4 *)d_buf, bytes / 16u, d_sink);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* Measurement aid: what the matrix cores deliver when vector instructions run beside them.  Every wave
 * issues `iters` x 16 independent v_mfma_i32_16x16x64_i8 (four accumulators in turn) with NV plain f32
 * multiply or add instructions, independent of the MFMAs, after each of them.  On this device the two do
 * not overlap, within a wave or between the waves of a SIMD: a launch with NV = 4 reaches 2.6 POP/s
 * against 4.9 POP/s with NV = 0 at any occupancy, i.e. an MFMA costs 16 cycles of the SIMD and a vector
 * instruction 3.5 more.  That is what bounds the prefill kernel, whose exact float step and operand
 * building are vector instructions. */
template <int NV>
__global__ __launch_bounds__(1024) void
k_mfma_probe(uint32_t iters, float *__restrict__ sink)
{
    const uint32_t lane = threadIdx.x & 63u;
    const v4i a = { (int)lane, 2, 3, 4 }, b = { 5, (int)lane, 7, 8 };
    v4i c[4] = { { 0, 0, 0, 0 }, { 0, 0, 0, 0 }, { 0, 0, 0, 0 }, { 0, 0, 0, 0 } };
    float f[4] = { (float)lane, 1.0f, 2.0f, 3.0f };
    for (uint32_t i = 0; i < iters; i++) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            c[j & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c[j & 3], 0, 0, 0);
#pragma unroll
            for (int k = 0; k < NV; k++) {
                float &v = f[(j * NV + k) & 3];
                v = ((j * NV + k) & 4) ? v + 0.5f : v * 1.0001f;
            }
        }
    }
    if (c[0][0] + c[1][1] + c[2][2] + c[3][3] == 0x7fffffff || f[0] + f[1] + f[2] + f[3] == 12345.0f)
        sink[0] = f[0];
}

extern "C" int oxh_debug_mfma_probe(int valu_per_mfma, int waves_per_simd, double *pops)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (!pops || waves_per_simd < 1 || waves_per_simd > 4) return arg_fail("oxh_debug_mfma_probe: 1..4 waves per SIMD");
    float *d_sink = nullptr;
    HIP_TRY(hipMalloc((void **)&d_sink, 64));
    const uint32_t iters = 4000, cus = (uint32_t)(g_n_cu > 0 ? g_n_cu : 256), threads = 256u * (uint32_t)waves_per_simd;
    hipStream_t st = pick_stream(nullptr);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    for (int rep = 0; rep < 2 && e == hipSuccess; rep++) {      /* the first launch warms up */
        if (rep == 1) e = hipEventRecord(e0, st);
        switch (valu_per_mfma) {
        case 0: hipLaunchKernelGGL(k_mfma_probe<0>, dim3(cus), dim3(threads), 0, st, iters, d_sink); break;
        case 1: hipLaunchKernelGGL(k_mfma_probe<1>, dim3(cus), dim3(threads), 0, st, iters, d_sink); break;
        case 2: hipLaunchKernelGGL(k_mfma_probe<2>, dim3(cus), dim3(threads), 0, st, iters, d_sink); break;
        case 4: hipLaunchKernelGGL(k_mfma_probe<4>, dim3(cus), dim3(threads), 0, st, iters, d_sink); break;
        default: e = hipErrorInvalidValue; break;
        }
    }
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(d_sink);
    if (e != hipSuccess) return valu_per_mfma == 3 || valu_per_mfma > 4 || valu_per_mfma < 0
                                    ? arg_fail("oxh_debug_mfma_probe: valu_per_mfma is 0, 1, 2 or 4") : hip_fail(e, "oxh_debug_mfma_probe");
    *pops = (double)cus * (threads / 64u) * iters * 16.0 * 32768.0 / ((double)ms * 1e12);
    return OXH_OK;
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
    OxhSegment s = { d_w, scratch, rows, 0, 0, nullptr };
    const GemvIo io = { d_act, nullptr, 0, nullptr, nullptr };
    rc = launch_gemv(qtype, &s, 1, cols, io, 1, rows, d_sums, stream);
    hipError_t e = hipStreamSynchronize(pick_stream(stream));
    (void)hipFree(scratch);
    if (rc) return rc;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return OXH_OK;
}

template <int TC, int RC, int WAVES, bool RELAXED = false>
static void mmq_launch(const void *d_w, size_t rows, size_t blocks, const void *d_acts, size_t n_vec,
                       float *d_out, size_t out_stride, void *stream)
{
    typedef MmqGeom<TC, RC, WAVES> G;
    const dim3 grid((uint32_t)((rows + G::ROWS - 1) / G::ROWS), (uint32_t)((n_vec + G::TOK - 1) / G::TOK));
    auto kernel = k_mmq_q4_k<TC, RC, WAVES, RELAXED>;
    hipLaunchKernelGGL(kernel, grid, dim3(WAVES * 64), G::LDS_BYTES, pick_stream(stream),
                       (const uint8_t *)d_w, (uint32_t)rows, (uint32_t)blocks,
                       (const uint8_t *)d_acts, (uint32_t)n_vec, d_out, out_stride);
}

template <int TC, int RC, int WAVES, bool RELAXED = false>
static void mmq5_launch(const void *d_w, size_t rows, size_t blocks, const void *d_acts, size_t n_vec,
                        float *d_out, size_t out_stride, void *stream)
{
    typedef MmqGeom<TC, RC, WAVES, true> G;
    const dim3 grid((uint32_t)((rows + G::ROWS - 1) / G::ROWS), (uint32_t)((n_vec + G::TOK - 1) / G::TOK));
    auto kernel = k_mmq_q5_k<TC, RC, WAVES, RELAXED>;
    hipLaunchKernelGGL(kernel, grid, dim3(WAVES * 64), G::LDS_BYTES, pick_stream(stream),
                       (const uint8_t *)d_w, (uint32_t)rows, (uint32_t)blocks,
                       (const uint8_t *)d_acts, (uint32_t)n_vec, d_out, out_stride);
}

template <int TC, int RC, int WAVES, bool Q2 = false>
static void mmq6_launch(const void *d_w, size_t rows, size_t blocks, const void *d_acts, size_t n_vec,
                        float *d_out, size_t out_stride, void *stream)
{
    typedef Mmq6Geom<TC, RC, WAVES> G;
    const dim3 grid((uint32_t)((rows + G::ROWS - 1) / G::ROWS), (uint32_t)((n_vec + G::TOK - 1) / G::TOK));
    auto kernel = k_mmq_q6_k<TC, RC, WAVES, Q2>;
    hipLaunchKernelGGL(kernel, grid, dim3(WAVES * 64), G::LDS_BYTES, pick_stream(stream),
                       (const uint8_t *)d_w, (uint32_t)rows, (uint32_t)blocks,
                       (const uint8_t *)d_acts, (uint32_t)n_vec, d_out, out_stride);
}

/* Which tile a matrix-core launch runs on: the largest one that still gives (nearly) every compute
 * unit a workgroup.  1: 256 x 128 (rows x tokens; 128 x 128 for the types with one row chunk per wave:
 * Q5_K, Q6_K, widened Q2_K), 2: 128 x 64, 3: 64 x 32, 4: 64 x 16, 5: 64 x 128 on four waves, which only the
 * Q6_K tile code has, for matrices with too few rows to fill the device with 128 x 128 tiles (the scaled
 * weight operands a wave builds are then still reused by 128 tokens: 4096 x 14336 x 512 takes 144 us
 * against 167 us on 128 x 64 tiles).  Pure arithmetic: OXH_MMQ_SHAPE = 1..5 overrides it at launch. */
static int mmq_tile_shape(uint32_t qtype, size_t rows, size_t n_vec, size_t cus)
{
    const size_t need = cus - cus / 8;
    /* a launch that gives no CU more than one 64 x 16 tile is paced by a workgroup's walk over the
     * super-blocks of its rows, not by the matrix cores: the smallest tiles then put the most CUs to
     * work (4096 x 4096 x 64: 13.3 against 14.9 us on 64 x 32 tiles; 4096 x 14336 Q6_K: 75 against 87) */
    const bool few_tiles = ((rows + 63) / 64) * ((n_vec + 15) / 16) <= cus;
    if (n_vec <= 16) return 4;
    if (n_vec <= 32) return few_tiles ? 4 : 3;
    if (qtype == OXH_Q6_K || is_q5k(qtype) || qtype == OXH_Q2_K_WIDE) {
        if (((rows + 127) / 128) * ((n_vec + 127) / 128) >= need) return 1;
        if (!is_q5k(qtype) && ((rows + 63) / 64) * ((n_vec + 127) / 128) >= need) return 5;
        if (((rows + 127) / 128) * ((n_vec + 63) / 64) >= need) return 2;
        return few_tiles ? 4 : 3;
    }
    if (((rows + 255) / 256) * ((n_vec + 127) / 128) >= need) return 1;
    if (((rows + 127) / 128) * ((n_vec + 63) / 64) >= need) return 2;
    return few_tiles ? 4 : 3;
}

/* the 32-value formats with a matrix-core kernel, as its LEG parameter; -1 for everything else */
static int mmq80_leg(uint32_t qtype)
{
    switch (qtype) {
    case OXH_Q8_0:   return 0;
    case OXH_Q4_0:   return 1;
    case OXH_Q4_1:   return 2;
    case OXH_Q5_0:   return 3;
    case OXH_Q5_1:   return 4;
    case OXH_AL5_XS: return 5;
    default:         return -1;
    }
}

extern "C" int oxh_mmq_tile(uint32_t qtype, size_t rows, size_t n_vec, size_t n_cu, uint32_t *tile_rows,
                            uint32_t *tile_tokens)
{
    if (mmq80_leg(canon_qtype(qtype)) >= 0 && rows && n_vec && n_cu) {       /* one tile for these */
        if (tile_rows) *tile_rows = MQT_WAVES * 16u;
        if (tile_tokens) *tile_tokens = MQT_TOK;
        return OXH_OK;
    }
    const bool one_chunk = qtype == OXH_Q6_K || is_q5k(qtype) || qtype == OXH_Q2_K_WIDE;
    if ((!is_q4k(qtype) && !one_chunk) || rows == 0 || n_vec == 0 || n_cu == 0) return OXH_DECLINED;
    static const uint32_t tr[6] = { 0, 256, 128, 64, 64, 64 }, tt[6] = { 0, 128, 64, 32, 16, 128 };
    const int shape = mmq_tile_shape(qtype, rows, n_vec, n_cu);
    if (tile_rows) *tile_rows = (shape == 1 && one_chunk) ? 128u : tr[shape];
    if (tile_tokens) *tile_tokens = tt[shape];
    return OXH_OK;
}

static int mmq_run(uint32_t qtype, const void *d_w, size_t rows, size_t cols, const void *d_acts, size_t n_vec,
                   float *d_out, size_t out_stride, bool relaxed, void *stream);

extern "C" int oxh_mmq(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                       const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
                       void *stream)
{
    return mmq_run(qtype, d_w, rows, cols, d_acts, n_vec, d_out, out_stride, false, stream);
}

/* Few tiles and many super-blocks: a tile's columns go to several workgroups (k_mmq_*_split) */
static bool mmq_split_plan(uint32_t qtype, size_t rows, size_t cols, size_t n_vec, size_t out_stride, size_t cus,
                           uint32_t *b_per_slice, uint32_t *slices, size_t *ws_bytes, uint32_t *tile_tokens = nullptr)
{
    qtype = canon_qtype(qtype);
    if (!is_q4k(qtype) && !is_q5k(qtype) && qtype != OXH_Q6_K && qtype != OXH_Q2_K_WIDE) return false;
    if (rows == 0 || n_vec == 0 || n_vec > 64 || cols == 0 || cols % OXH_QK_K || out_stride < rows) return false;
    const size_t B = cols / OXH_QK_K;
    /* 64 x 16 tiles; 64 x 32 above sixteen activations unless the narrow tiles leave three quarters of
     * the device idle anyway (a wave builds its rows' operands once per super-block whatever the tile's
     * tokens: 4096 x 14336 Q6_K under 32 activations 44.2 -> 39.9 us, 1024 x 4096 Q4_K 7.2 -> 7.9) */
    const size_t row_tiles = (rows + 63) / 64;
    const size_t tile_tok = (n_vec > 16 && row_tiles * ((n_vec + 15) / 16) > cus / 4) ? 32 : 16;
    const size_t tiles = row_tiles * ((n_vec + tile_tok - 1) / tile_tok);
    if (B < 8 || tiles > cus / 2) return false;
    const size_t want = (2 * cus) / tiles;                      /* workgroups per tile for two per CU */
    size_t per = (B + want - 1) / want;
    if (per < 2) per = 2;
    const size_t n = (B + per - 1) / per;
    if (n < 2) return false;
    size_t bytes;
    if (n_vec > SIZE_MAX / out_stride || B > SIZE_MAX / (n_vec * out_stride) / sizeof(float)) return false;
    bytes = B * n_vec * out_stride * sizeof(float);
    if (bytes > ((size_t)512 << 20)) return false;
    /* what the shorter walk saves (0.8 us a super-block) against the second launch and the terms' trip
     * through memory (written and read once at some 4 TB/s), with four microseconds to spare: 4096 x 4096
     * Q4_K under 32 activations measured 12.7 us split against 12.7, under 24 11.8 against 12.9, 6144 x 4096
     * under 17 14.0 against 13.1, 4096 x 14336 under 32 26.3 against 42.6, under 48 36.5 against 43.2 */
    const double saving_us = 0.8 * (double)(B - per), cost_us = 4.0 + 2.0 * (double)bytes / 4.0e6;
    if (saving_us < cost_us + 4.0) return false;
    if (b_per_slice) *b_per_slice = (uint32_t)per;
    if (slices) *slices = (uint32_t)n;
    if (ws_bytes) *ws_bytes = bytes;
    if (tile_tokens) *tile_tokens = (uint32_t)tile_tok;
    return true;
}

extern "C" size_t oxh_mmq_split_workspace(uint32_t qtype, size_t rows, size_t cols, size_t n_vec, size_t out_stride)
{
    size_t bytes = 0;
    const size_t cus = (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    return mmq_split_plan(qtype, rows, cols, n_vec, out_stride, cus, nullptr, nullptr, &bytes) ? bytes : 0;
}

extern "C" int oxh_mmq_split(uint32_t qtype, const void *d_w, size_t rows, size_t cols, const void *d_acts,
                             size_t n_vec, float *d_out, size_t out_stride, void *d_workspace, size_t workspace_bytes,
                             void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    uint32_t per = 0, slices = 0, tile_tok = 16;
    size_t need = 0;
    const size_t cus = (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    if (!mmq_split_plan(qtype, rows, cols, n_vec, out_stride, cus, &per, &slices, &need, &tile_tok) || !d_workspace ||
        workspace_bytes < need)
        return mmq_run(qtype, d_w, rows, cols, d_acts, n_vec, d_out, out_stride, false, stream);
    if (!d_w || !d_acts || !d_out) return arg_fail("oxh_mmq_split: NULL pointer");
    if ((uintptr_t)d_workspace % sizeof(float)) return arg_fail("oxh_mmq_split: workspace not aligned to 4 bytes");
    qtype = canon_qtype(qtype);
    const uint32_t B = (uint32_t)(cols / OXH_QK_K);
    if ((size_t)B * 292u * 256u > 0xFFFFFFFFull) return arg_fail("oxh_mmq_split: cols too large");
    const dim3 grid((uint32_t)((rows + 63) / 64), (uint32_t)((n_vec + tile_tok - 1) / tile_tok), slices), block(4 * 64);
    const size_t split_stride = n_vec * out_stride;
    hipStream_t st = pick_stream(stream);
    float *terms = (float *)d_workspace;
    const uint8_t *w8 = (const uint8_t *)d_w, *a8 = (const uint8_t *)d_acts;
    const uint32_t r32 = (uint32_t)rows, n32 = (uint32_t)n_vec;
#define OXH_SPLIT_LAUNCH(KERNEL, GEOM)                                                                        \
    do {                                                                                                      \
        auto kern = KERNEL;                                                                                   \
        hipLaunchKernelGGL(kern, grid, block, 2 * GEOM::LDS_BYTES, st, w8, r32, B, a8, n32, terms, out_stride, \
                           per, split_stride);                                                                \
    } while (0)
    typedef Mmq6Geom<1, 1, 4> G6a;
    typedef Mmq6Geom<2, 1, 4> G6b;
    typedef MmqGeom<1, 1, 4, true> G5a;
    typedef MmqGeom<2, 1, 4, true> G5b;
    typedef MmqGeom<1, 1, 4> G4a;
    typedef MmqGeom<2, 1, 4> G4b;
    const bool wide_tile = tile_tok == 32;
    if (qtype == OXH_Q6_K) {
        if (wide_tile) OXH_SPLIT_LAUNCH((k_mmq_q6_k_split<2, false, 2>), G6b);
        else OXH_SPLIT_LAUNCH((k_mmq_q6_k_split<2, false, 1>), G6a);
    } else if (qtype == OXH_Q2_K_WIDE) {
        if (wide_tile) OXH_SPLIT_LAUNCH((k_mmq_q6_k_split<2, true, 2>), G6b);
        else OXH_SPLIT_LAUNCH((k_mmq_q6_k_split<2, true, 1>), G6a);
    } else if (is_q5k(qtype)) {
        if (wide_tile) OXH_SPLIT_LAUNCH((k_mmq_q45_k_split<true, 2, 2>), G5b);
        else OXH_SPLIT_LAUNCH((k_mmq_q45_k_split<true, 2, 1>), G5a);
    } else {
        if (wide_tile) OXH_SPLIT_LAUNCH((k_mmq_q45_k_split<false, 2, 2>), G4b);
        else OXH_SPLIT_LAUNCH((k_mmq_q45_k_split<false, 2, 1>), G4a);
    }
#undef OXH_SPLIT_LAUNCH
    HIP_TRY(hipGetLastError());
    const size_t n_out = rows * n_vec;
    hipLaunchKernelGGL(k_mmq_sum_terms, dim3((uint32_t)((n_out + 255) / 256)), dim3(256), 0, st, terms, B, split_stride,
                       d_out, (uint32_t)rows, (uint32_t)n_vec, out_stride);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_mmq_ex(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                          const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
                          uint32_t flags, void *stream)
{
    if (flags & ~OXH_MMQ_RELAXED) return arg_fail("oxh_mmq_ex: unknown flag");
    return mmq_run(qtype, d_w, rows, cols, d_acts, n_vec, d_out, out_stride, (flags & OXH_MMQ_RELAXED) != 0, stream);
}

static int mmq_run(uint32_t qtype, const void *d_w, size_t rows, size_t cols, const void *d_acts, size_t n_vec,
                   float *d_out, size_t out_stride, bool relaxed, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0 || n_vec == 0) return OXH_OK;
    if (!d_w || !d_acts || !d_out) return arg_fail("oxh_mmq: NULL pointer");
    const int leg = mmq80_leg(canon_qtype(qtype));
    if (leg >= 0 && oxh_act_kind(qtype, cols) == 1) {
        /* 32-value blocks against Q8_0 activations: one tile shape, exact f32 step only */
        if (out_stride < rows) return arg_fail("oxh_mmq: out_stride < rows");
        const size_t blocks32 = cols / OXH_QK8_0;
        if (rows > 0x7FFFFFFFull || n_vec > 0x7FFFFFFFull || blocks32 > 0xFFFFFFull)
            return arg_fail("oxh_mmq: dimension too large");
        if (blocks32 * block_bytes(qtype) < 16u) {
            snprintf(g_err, sizeof g_err, "oxh_mmq: rows of qtype %u with cols %zu are shorter than 16 bytes", qtype, cols);
            return OXH_DECLINED;
        }
        const uint32_t n_rt = (uint32_t)((rows + MQT_WAVES * 16u - 1u) / (MQT_WAVES * 16u));
        const uint32_t n_tt = (uint32_t)((n_vec + MQT_TOK - 1u) / MQT_TOK);
        const uint64_t wgs = (uint64_t)((n_rt + 7u) / 8u) * 8u * n_tt;
        if (wgs > 0x7FFFFFFFull) return arg_fail("oxh_mmq: too many tiles");
        hipStream_t st = pick_stream(stream);
#define OXH_MQT(LEG) hipLaunchKernelGGL((k_mmq_q80<LEG>), dim3((uint32_t)wgs), dim3(MQT_WAVES * 64u),          \
                                        MqtGeom<LEG>::LDS_BYTES, st, (const uint8_t *)d_w, (uint32_t)rows,     \
                                        (uint32_t)blocks32, (const uint8_t *)d_acts, (uint32_t)n_vec, d_out,   \
                                        out_stride, n_rt, n_tt)
        switch (leg) {
        case 1:  OXH_MQT(1); break;
        case 2:  OXH_MQT(2); break;
        case 3:  OXH_MQT(3); break;
        case 4:  OXH_MQT(4); break;
        case 5:  OXH_MQT(5); break;
        default: OXH_MQT(0); break;
        }
#undef OXH_MQT
        HIP_TRY(hipGetLastError());
        return OXH_OK;
    }
    const bool wide2 = qtype == OXH_Q2_K_WIDE;
    if ((!is_q4k(qtype) && !is_q5k(qtype) && qtype != OXH_Q6_K && !wide2) ||
        oxh_act_kind(wide2 ? OXH_Q2_K : qtype, cols) != 2) {
        snprintf(g_err, sizeof g_err, "oxh_mmq: qtype %u with cols %zu has no MFMA kernel", qtype, cols);
        return OXH_DECLINED;
    }
    if (out_stride < rows) return arg_fail("oxh_mmq: out_stride < rows");
    const size_t blocks = cols / OXH_QK_K;
    if (rows > 0x7FFFFFFFull || n_vec > 0x7FFFFFFFull || blocks > 0xFFFFFFull)
        return arg_fail("oxh_mmq: dimension too large");
    /* the kernel addresses a workgroup's rows and tokens with 32-bit lane offsets */
    if (blocks * 292u * 256u > 0xFFFFFFFFull)
        return arg_fail("oxh_mmq: cols too large");
    static int forced = -1;
    if (forced < 0) forced = (int)env_u32("OXH_MMQ_SHAPE", 0, 0, 5);
    int shape = forced ? forced : mmq_tile_shape(qtype, rows, n_vec, (size_t)(g_n_cu > 0 ? g_n_cu : 256));
    if (qtype == OXH_Q6_K || is_q5k(qtype) || wide2) {
        if (is_q5k(qtype)) {
            if (shape == 5) shape = 2;
            if (shape == 1 && relaxed)      mmq5_launch<8, 1, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 2 && relaxed) mmq5_launch<4, 1, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 1) mmq5_launch<8, 1, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 2) mmq5_launch<4, 1, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 3) mmq5_launch<2, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else                 mmq5_launch<1, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            HIP_TRY(hipGetLastError());
            return OXH_OK;
        }
        if (wide2) {
            if (shape == 5)      mmq6_launch<8, 1, 4, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 1) mmq6_launch<8, 1, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 2) mmq6_launch<4, 1, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else if (shape == 3) mmq6_launch<2, 1, 4, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            else                 mmq6_launch<1, 1, 4, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
            HIP_TRY(hipGetLastError());
            return OXH_OK;
        }
        if (shape == 5)      mmq6_launch<8, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
        else if (shape == 1) mmq6_launch<8, 1, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
        else if (shape == 2) mmq6_launch<4, 1, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
        else if (shape == 3) mmq6_launch<2, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
        else                 mmq6_launch<1, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
        HIP_TRY(hipGetLastError());
        return OXH_OK;
    }
    if (shape == 5) shape = 2;
    /* the relaxed f32 step exists for the two prefill tiles; smaller launches are bound by the weight
     * stream and keep the exact one */
    if (shape == 1 && relaxed)      mmq_launch<8, 2, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    else if (shape == 2 && relaxed) mmq_launch<4, 1, 8, true>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    else if (shape == 1) mmq_launch<8, 2, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    else if (shape == 2) mmq_launch<4, 1, 8>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    else if (shape == 3) mmq_launch<2, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    else                 mmq_launch<1, 1, 4>(d_w, rows, blocks, d_acts, n_vec, d_out, out_stride, stream);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_get_rows(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                            const uint32_t *d_ids, size_t n_ids, float *d_out, size_t out_stride,
                            void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    qtype = canon_qtype(qtype);
    if (n_ids == 0) return OXH_OK;
    if (!d_w || !d_ids || !d_out) return arg_fail("oxh_get_rows: NULL pointer");
    /* every type with a matvec kernel but the codebook formats of the integer path; the 4-bit codebook
     * formats of the dequantise path */
    const bool iq4 = qtype == OXH_IQ4_NL || qtype == OXH_IQ4_XS;
    const size_t rb = iq4 ? oxh_f32_path_row_bytes(qtype, cols)
                          : (oxh_act_kind(qtype, cols) && !is_iq(qtype) && qtype != OXH_Q6_K_G8) ? oxh_row_bytes(qtype, cols) : 0;
    if (rb == 0) {
        snprintf(g_err, sizeof g_err, "oxh_get_rows: qtype %u with cols %zu has no kernel here", qtype, cols);
        return OXH_DECLINED;
    }
    if (out_stride < cols) return arg_fail("oxh_get_rows: out_stride < cols");
    if (rows > 0xFFFFFFFFull || cols > 0xFFFFFFFFull || rb > 0xFFFFFFFFull || n_ids > 65535u)
        return arg_fail("oxh_get_rows: dimension too large (at most 65535 ids per call)");
    if ((out_stride & 3u) || ((uintptr_t)d_out & 15u))
        return arg_fail("oxh_get_rows: output rows must be 16-byte aligned");
    const dim3 grid((uint32_t)((cols + 1023u) / 1024u), (uint32_t)n_ids), block(256);
    hipStream_t st = pick_stream(stream);
    const uint8_t *w = (const uint8_t *)d_w;
#define OXH_GET_ROWS(KIND)                                                                   \
    hipLaunchKernelGGL(k_get_rows<KIND>, grid, block, 0, st, w, (uint32_t)rows, (uint32_t)cols, \
                       (uint32_t)rb, d_ids, d_out, out_stride)
    if (iq4) {
        if (qtype == OXH_IQ4_XS) hipLaunchKernelGGL(k_get_rows_iq4<true>, grid, block, 0, st, w, (uint32_t)rows, (uint32_t)cols,
                                                    (uint32_t)rb, d_ids, d_out, out_stride);
        else                     hipLaunchKernelGGL(k_get_rows_iq4<false>, grid, block, 0, st, w, (uint32_t)rows, (uint32_t)cols,
                                                    (uint32_t)rb, d_ids, d_out, out_stride);
    }
    else if (is_q4k(qtype))     OXH_GET_ROWS(0);
    else if (is_q5k(qtype))     OXH_GET_ROWS(1);
    else if (qtype == OXH_Q6_K) OXH_GET_ROWS(2);
    else if (qtype == OXH_Q4_0) OXH_GET_ROWS(4);
    else if (qtype == OXH_Q4_1) OXH_GET_ROWS(5);
    else if (qtype == OXH_Q5_0) OXH_GET_ROWS(6);
    else if (qtype == OXH_Q5_1) OXH_GET_ROWS(7);
    else if (qtype == OXH_AL5_XS) OXH_GET_ROWS(10);
    else if (qtype == OXH_Q2_K) OXH_GET_ROWS(8);
    else if (qtype == OXH_Q3_K_M) OXH_GET_ROWS(9);
    else                        OXH_GET_ROWS(3);
#undef OXH_GET_ROWS
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_q3_k_as_q6_k(const void *d_w, size_t rows, size_t cols, void *d_q6k, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0) return OXH_OK;
    if (!d_w || !d_q6k) return arg_fail("oxh_q3_k_as_q6_k: NULL pointer");
    if (cols == 0 || cols % OXH_QK_K) return arg_fail("oxh_q3_k_as_q6_k: cols must be a whole number of 256-blocks");
    const size_t blocks = cols / OXH_QK_K;
    if (rows > 0x3FFFFFC0ull / blocks) return arg_fail("oxh_q3_k_as_q6_k: matrix too large");
    const uint32_t n_blocks = (uint32_t)(rows * blocks);
    hipLaunchKernelGGL(k_q3k_to_q6k, dim3((n_blocks * 4u + 255u) / 256u), dim3(256), 0, pick_stream(stream),
                       (const uint8_t *)d_w, (uint8_t *)d_q6k, n_blocks);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_q2_k_widen(const void *d_w, size_t rows, size_t cols, void *d_wide, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0) return OXH_OK;
    if (!d_w || !d_wide) return arg_fail("oxh_q2_k_widen: NULL pointer");
    if (cols == 0 || cols % OXH_QK_K) return arg_fail("oxh_q2_k_widen: cols must be a whole number of 256-blocks");
    const size_t blocks = cols / OXH_QK_K;
    if (rows > 0x3FFFFFC0ull / blocks) return arg_fail("oxh_q2_k_widen: matrix too large");
    const uint32_t n_blocks = (uint32_t)(rows * blocks);
    hipLaunchKernelGGL(k_q2k_widen, dim3((n_blocks * 4u + 255u) / 256u), dim3(256), 0, pick_stream(stream),
                       (const uint8_t *)d_w, (uint8_t *)d_wide, n_blocks);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_q6_k_group(const void *d_w, size_t rows, size_t cols, void *d_g8, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0) return OXH_OK;
    if (!d_w || !d_g8) return arg_fail("oxh_q6_k_group: NULL pointer");
    if (d_w == d_g8) return arg_fail("oxh_q6_k_group: source and destination must differ");
    if (cols == 0 || cols % (8u * OXH_QK_K)) {
        snprintf(g_err, sizeof g_err, "oxh_q6_k_group: cols %zu is not a multiple of 2048 (eight blocks)", cols);
        return OXH_DECLINED;
    }
    if (((uintptr_t)d_w & 1u) || ((uintptr_t)d_g8 & 15u))
        return arg_fail("oxh_q6_k_group: the source must be 2-byte and the destination 16-byte aligned");
    const size_t groups = rows * (cols / (8u * OXH_QK_K));
    if (groups > 0xFFFFFFFFull / 105u) return arg_fail("oxh_q6_k_group: matrix too large");
    const uint32_t threads = (uint32_t)groups * 105u;
    hipLaunchKernelGGL(k_q6k_group, dim3((threads + 255u) / 256u), dim3(256), 0, pick_stream(stream),
                       (const uint8_t *)d_w, (uint8_t *)d_g8, (uint32_t)groups);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" size_t oxh_tile16_bytes(uint32_t qtype, size_t rows, size_t cols)
{
    const uint32_t q = canon_qtype(qtype);
    if (q == OXH_Q8_0) return (cols == 0 || cols % (4u * OXH_QK8_0)) ? 0 : (rows + 15u) / 16u * (cols / (4u * OXH_QK8_0)) * Q80T_UNIT;
    if ((!is_q4k(q) && !is_q5k(q)) || cols == 0 || cols % OXH_QK_K) return 0;
    return (rows + 15u) / 16u * 16u * (cols / OXH_QK_K) * block_bytes(q);
}

extern "C" int oxh_tile16(uint32_t qtype, const void *d_w, size_t rows, size_t cols, void *d_t16, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (rows == 0) return OXH_OK;
    if (!d_w || !d_t16) return arg_fail("oxh_tile16: NULL pointer");
    if (d_w == d_t16) return arg_fail("oxh_tile16: source and destination must differ");
    const size_t bytes = oxh_tile16_bytes(qtype, rows, cols);
    if (!bytes) {
        snprintf(g_err, sizeof g_err, "oxh_tile16: type %u with cols %zu is not Q4_K, Q5_K or Q8_0 in whole blocks", qtype, cols);
        return OXH_DECLINED;
    }
    if (canon_qtype(qtype) == OXH_Q8_0) {
        if (((uintptr_t)d_w & 1u) || ((uintptr_t)d_t16 & 15u))
            return arg_fail("oxh_tile16: the source must be 2-byte and the destination 16-byte aligned");
        const size_t items = bytes / Q80T_UNIT * 16u;
        if (items > 0xFFFFFFFFull) return arg_fail("oxh_tile16: matrix too large");
        hipLaunchKernelGGL(k_q80_tile16, dim3((uint32_t)((items + 255u) / 256u)), dim3(256), 0, pick_stream(stream),
                           (const uint8_t *)d_w, (uint8_t *)d_t16, (uint32_t)rows, (uint32_t)(cols / OXH_QK8_0),
                           (uint32_t)items);      /* an item = (unit, row of its group) */
        HIP_TRY(hipGetLastError());
        return OXH_OK;
    }
    if (((uintptr_t)d_w & 15u) || ((uintptr_t)d_t16 & 15u))
        return arg_fail("oxh_tile16: source and destination must be 16-byte aligned");
    const size_t pieces = bytes / 16u;
    if (pieces > 0xFFFFFFFFull) return arg_fail("oxh_tile16: matrix too large");
    hipLaunchKernelGGL(k_tile16, dim3((uint32_t)((pieces + 255u) / 256u)), dim3(256), 0, pick_stream(stream),
                       (const uint8_t *)d_w, (uint8_t *)d_t16, (uint32_t)rows, (uint32_t)(cols / OXH_QK_K),
                       (uint32_t)(block_bytes(canon_qtype(qtype)) / 16u), (uint32_t)pieces);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* ─── mixture of experts ──────────────────────────────────────────────── */

static size_t align256(size_t v) { return (v + 255u) & ~(size_t)255u; }

/* Workspace layout of oxh_moe_ffn (every part 256-byte aligned). */
struct MoeLayout {
    size_t ids, wts, slot_pos, perm, counts, offsets, act_x, gate, up, act_h, y, total;
};

static int moe_layout(const OxhMoe *m, size_t n_tok, MoeLayout *l)
{
    if (!m || m->n_expert == 0 || m->n_expert > OXH_MOE_MAX_EXPERTS)
        return arg_fail("moe: n_expert must be 1..64");
    if (m->top_k == 0 || m->top_k > OXH_MOE_MAX_TOPK || m->top_k > m->n_expert)
        return arg_fail("moe: top_k must be 1..8 and at most n_expert");
    /* tile-major expert matrices are stacked in whole 16-row groups */
    const bool gu_ok = is_q4k(m->qtype_gate_up) || is_q5k(m->qtype_gate_up) || m->qtype_gate_up == OXH_Q6_K ||
                       (is_t16(m->qtype_gate_up) && m->ffn % 16u == 0);
    const bool dn_ok = is_q4k(m->qtype_down) || is_q5k(m->qtype_down) || m->qtype_down == OXH_Q6_K ||
                       (is_t16(m->qtype_down) && m->hidden % 16u == 0);
    if (!gu_ok || !dn_ok || oxh_act_kind(m->qtype_gate_up, m->hidden) != 2 || oxh_act_kind(m->qtype_down, m->ffn) != 2) {
        snprintf(g_err, sizeof g_err, "moe: expert matrices must be Q4_K, Q5_K or Q6_K with widths in whole "
                 "256-blocks, tile-major ones with rows in whole sixteens (types %u / %u, hidden %zu, ffn %zu)", m->qtype_gate_up, m->qtype_down, m->hidden, m->ffn);
        return OXH_DECLINED;
    }
    if (n_tok == 0 || n_tok > 4096) return arg_fail("moe: n_tok must be 1..4096");
    const size_t pairs = n_tok * m->top_k;
    size_t at = 0;
#define OXH_PART(FIELD, BYTES) l->FIELD = at; at = align256(at + (BYTES))
    OXH_PART(ids, pairs * 4);
    OXH_PART(wts, pairs * 4);
    OXH_PART(slot_pos, pairs * 4);
    OXH_PART(perm, pairs * 4);
    OXH_PART(counts, OXH_MOE_MAX_EXPERTS * 4);
    OXH_PART(offsets, (OXH_MOE_MAX_EXPERTS + 1) * 4);
    OXH_PART(act_x, pairs * oxh_act_bytes(m->qtype_gate_up, m->hidden));
    OXH_PART(gate, pairs * m->ffn * 4);
    OXH_PART(up, pairs * m->ffn * 4);
    OXH_PART(act_h, pairs * oxh_act_bytes(m->qtype_down, m->ffn));
    OXH_PART(y, pairs * m->hidden * 4);
#undef OXH_PART
    l->total = at;
    return OXH_OK;
}

extern "C" int oxh_moe_workspace_bytes(const OxhMoe *m, size_t n_tok, size_t *bytes)
{
    MoeLayout l;
    const int rc = moe_layout(m, n_tok, &l);
    if (rc) return rc;
    if (bytes) *bytes = l.total;
    return OXH_OK;
}

extern "C" int oxh_debug_moe_workspace_parts(const OxhMoe *m, size_t n_tok, size_t parts[12])
{
    MoeLayout l;
    const int rc = moe_layout(m, n_tok, &l);
    if (rc) return rc;
    if (!parts) return arg_fail("oxh_debug_moe_workspace_parts: NULL pointer");
    const size_t v[12] = { l.ids, l.wts, l.slot_pos, l.perm, l.counts, l.offsets, l.act_x, l.gate, l.up, l.act_h,
                           l.y, l.total };
    memcpy(parts, v, sizeof v);
    return OXH_OK;
}

extern "C" int oxh_moe_route(const float *d_logits, size_t n_tok, size_t n_expert, size_t top_k, int renorm,
                             int32_t *d_ids, float *d_weights, uint32_t *d_counts, uint32_t *d_offsets,
                             uint32_t *d_perm, uint32_t *d_slot_pos, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (n_tok == 0) return OXH_OK;
    if (!d_logits || !d_ids || !d_weights || !d_counts || !d_offsets || !d_perm || !d_slot_pos)
        return arg_fail("oxh_moe_route: NULL pointer");
    if (n_expert == 0 || n_expert > OXH_MOE_MAX_EXPERTS) return arg_fail("oxh_moe_route: n_expert must be 1..64");
    if (top_k == 0 || top_k > OXH_MOE_MAX_TOPK || top_k > n_expert)
        return arg_fail("oxh_moe_route: top_k must be 1..8 and at most n_expert");
    if (n_tok > 4096) return arg_fail("oxh_moe_route: at most 4096 tokens per call");
    /* a wave per token in the first phase, per expert in the second: up to 16 waves */
    const size_t waves = n_tok > n_expert ? n_tok : n_expert;
    const uint32_t threads = 64u * (uint32_t)(waves > 16 ? 16 : waves);
    hipLaunchKernelGGL(k_moe_route, dim3(1), dim3(threads), 0, pick_stream(stream),
                       d_logits, (uint32_t)n_tok, (uint32_t)n_expert, (uint32_t)top_k, renorm, d_ids, d_weights,
                       d_counts, d_offsets, d_perm, d_slot_pos);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* one launch of the MFMA tile kernel over all experts, activation runs from device memory */
/* one or more launches of the MFMA tile kernel over all experts, activation runs from device memory.
 * `pairs` = (token, expert) pairs in all; from about two dozen per expert on average on, the 128-row x 64-token tile
 * (eight waves) re-streams an expert's weights four times less often than the 64 x 16 one. */
template <int TC, int WAVES>
static int launch_experts_tiled(uint32_t qtype, const void *const *d_w, float *const *d_out, size_t n_mat,
                                size_t n_expert, size_t rows, size_t cols, const void *d_acts, size_t out_stride,
                                const uint32_t *d_counts, const uint32_t *d_offsets, size_t max_tokens, void *stream)
{
    /* sixteen-token tiles take the token tile from the grid's second dimension: as many as an expert that
     * every token chose would need */
    const uint32_t ny = TC == 1 ? (uint32_t)((max_tokens + 15u) / 16u ? (max_tokens + 15u) / 16u : 1u) : 1u;
    if (ny > 65535u) return arg_fail("moe: too many tokens for the sixteen-token tile");
    const uint32_t tile_major = is_t16(qtype) ? 1u : 0u;
    qtype = t16_base(qtype);
    typedef MmqGeom<TC, 1, WAVES> G;
    typedef Mmq6Geom<TC, 1, WAVES> G6;
    typedef MmqGeom<TC, 1, WAVES, true> G5;
    static_assert(G6::ROWS == G::ROWS && G5::ROWS == G::ROWS, "row tiling is shared by all formats");
    const size_t blocks = cols / OXH_QK_K;
    if (blocks * 292u * 256u > 0xFFFFFFFFull) return arg_fail("moe: cols too large");
    const size_t rb = oxh_row_bytes(qtype, cols);
    const uint8_t *acts = (const uint8_t *)d_acts;
    hipStream_t st = pick_stream(stream);
    const uint32_t nb = (uint32_t)blocks;
#define OXH_EXP_LAUNCH(KERNEL, GEOM, KB, ...)                                                            \
    hipLaunchKernelGGL(KERNEL, dim3(wg, ny), dim3(WAVES * 64), (KB) * GEOM::LDS_BYTES, st, t, nb, acts, out_stride, \
                       d_counts, d_offsets, ##__VA_ARGS__)
    /* one segment per expert and matrix, at most OXH_MAX_SEGS of them per launch */
    const size_t per_launch = OXH_MAX_SEGS / n_mat;
    for (size_t e0 = 0; e0 < n_expert; e0 += per_launch) {
        const size_t e1 = e0 + per_launch < n_expert ? e0 + per_launch : n_expert;
        SegTable t;
        memset(&t, 0, sizeof t);
        uint32_t wg = 0, n = 0;
        for (size_t mtx = 0; mtx < n_mat; mtx++)
            for (size_t e = e0; e < e1; e++) {
                t.s[n].w = (const uint8_t *)d_w[mtx] + e * rows * rb;
                t.s[n].out = d_out[mtx];
                t.s[n].rows = (uint32_t)rows;
                t.s[n].act_first = (uint32_t)e;         /* the expert whose count and offset apply */
                t.s[n].wg_begin = wg;
                wg += (uint32_t)((rows + G::ROWS - 1) / G::ROWS);
                n++;
            }
        t.n = n;
        for (uint32_t i = 1; i < 4 && i < n; i++) t.bound[i - 1] = t.s[i].wg_begin;
        /* super-blocks per stage: one in the large tile (no LDS to spare), two in the 64-row tile when the
         * launch is small, three in the 128-row one (Q4_K only) */
        if constexpr (TC == 1 && WAVES == 8) {
            if (!is_q4k(qtype)) return arg_fail("moe: the 128-row small tile exists for Q4_K only");
            OXH_EXP_LAUNCH((k_mmq_q45_k_experts<1, 1, 8, false, 3>), G, 3, tile_major);
        } else if (TC == 1 && mmq_deep_stages(wg)) {
            if (qtype == OXH_Q6_K) OXH_EXP_LAUNCH((k_mmq_q6_k_experts<TC, 1, WAVES, 2>), G6, 2);
            else if (is_q5k(qtype)) OXH_EXP_LAUNCH((k_mmq_q45_k_experts<TC, 1, WAVES, true, 2>), G5, 2, tile_major);
            else OXH_EXP_LAUNCH((k_mmq_q45_k_experts<TC, 1, WAVES, false, 2>), G, 2, tile_major);
        } else {
            if (qtype == OXH_Q6_K) OXH_EXP_LAUNCH((k_mmq_q6_k_experts<TC, 1, WAVES, 1>), G6, 1);
            else if (is_q5k(qtype)) OXH_EXP_LAUNCH((k_mmq_q45_k_experts<TC, 1, WAVES, true, 1>), G5, 1, tile_major);
            else OXH_EXP_LAUNCH((k_mmq_q45_k_experts<TC, 1, WAVES, false, 1>), G, 1, tile_major);
        }
    }
#undef OXH_EXP_LAUNCH
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

static int launch_experts(uint32_t qtype, const void *const *d_w, float *const *d_out, size_t n_mat,
                          size_t n_expert, size_t rows, size_t cols, const void *d_acts, size_t out_stride,
                          const uint32_t *d_counts, const uint32_t *d_offsets, size_t pairs, size_t max_tokens,
                          void *stream)
{
    static const uint32_t big_from = env_u32("OXH_MOE_BIG_TILE_FROM", 24, 0, 4096);     /* 0 = never */
    const size_t avg_tokens = pairs / n_expert;
    const uint32_t file_type = t16_base(qtype);
    if (big_from && avg_tokens >= big_from)
        return launch_experts_tiled<4, 8>(qtype, d_w, d_out, n_mat, n_expert, rows, cols, d_acts, out_stride,
                                          d_counts, d_offsets, max_tokens, stream);
    /* few rows per expert (a down projection): the 64-row tile gives at most two workgroups per CU; Q4_K
     * can take 128 rows on eight waves with three super-blocks per stage instead, half as much again in
     * flight (OXH_MOE_WIDE_SMALL=1).  Off by default: launched continuously, Mixtral's down projections at
     * 16 tokens run faster on the 64-row tiles with two super-blocks per stage (the layer 163 against 169 us;
     * the wider tile only won when the launches were timed right after an idle period).  Workgroups of
     * experts without a token leave at once, so what counts is the experts that can have one. */
    static const uint32_t wide = env_u32("OXH_MOE_WIDE_SMALL", 0, 0, 1);
    const size_t cus = (size_t)(g_n_cu > 0 ? g_n_cu : 256);
    const size_t live = pairs < n_expert ? (pairs ? pairs : 1) : n_expert;
    if (wide && is_q4k(file_type) && n_mat * n_expert * ((rows + 63) / 64) <= 2u * cus &&
        n_mat * live * ((rows + 127) / 128) >= cus - cus / 8)
        return launch_experts_tiled<1, 8>(qtype, d_w, d_out, n_mat, n_expert, rows, cols, d_acts, out_stride,
                                          d_counts, d_offsets, max_tokens, stream);
    return launch_experts_tiled<1, 4>(qtype, d_w, d_out, n_mat, n_expert, rows, cols, d_acts, out_stride,
                                      d_counts, d_offsets, max_tokens, stream);
}

/* the six launches of a layer over a workspace laid out by moe_layout(); arguments already checked */
static int moe_ffn_run(const OxhMoe *m, const MoeLayout &l, const float *d_logits, const float *d_x, size_t x_stride,
                       size_t n_tok, float *d_out, size_t out_stride, uint8_t *ws, void *stream)
{
    int rc;
    int32_t *ids = (int32_t *)(ws + l.ids);
    float *wts = (float *)(ws + l.wts);
    uint32_t *slot_pos = (uint32_t *)(ws + l.slot_pos), *perm = (uint32_t *)(ws + l.perm);
    uint32_t *counts = (uint32_t *)(ws + l.counts), *offsets = (uint32_t *)(ws + l.offsets);
    float *gate = (float *)(ws + l.gate), *up = (float *)(ws + l.up), *y = (float *)(ws + l.y);
    const size_t pairs = n_tok * m->top_k;

    /* 1. route and group; 2. gather + quantise each pair's token */
    if ((rc = oxh_moe_route(d_logits, n_tok, m->n_expert, m->top_k, m->renorm, ids, wts, counts, offsets, perm,
                            slot_pos, stream))) return rc;
    if ((rc = quantize_q8_k_ex(d_x, x_stride, pairs, m->hidden, ws + l.act_x, perm, nullptr, stream))) return rc;
    /* 3. gate and up of every expert over its own pairs */
    const void *w_gu[2] = { m->d_w_gate, m->d_w_up };
    float *o_gu[2] = { gate, up };
    if ((rc = launch_experts(m->qtype_gate_up, w_gu, o_gu, 2, m->n_expert, m->ffn, m->hidden, ws + l.act_x,
                             m->ffn, counts, offsets, pairs, n_tok, stream))) return rc;
    /* 4. h = silu(gate) * up, quantised; 5. down */
    if ((rc = quantize_q8_k_ex(gate, m->ffn, pairs, m->ffn, ws + l.act_h, nullptr, up, stream))) return rc;
    const void *w_dn[1] = { m->d_w_down };
    float *o_dn[1] = { y };
    if ((rc = launch_experts(m->qtype_down, w_dn, o_dn, 1, m->n_expert, m->hidden, m->ffn, ws + l.act_h,
                             m->hidden, counts, offsets, pairs, n_tok, stream))) return rc;
    /* 6. combine in ascending expert order */
    hipLaunchKernelGGL(k_moe_combine, dim3((uint32_t)((m->hidden + 255u) / 256u), (uint32_t)n_tok), dim3(256), 0,
                       pick_stream(stream), (const float *)y, m->hidden, (const int32_t *)ids, (const float *)wts,
                       (const uint32_t *)slot_pos, (uint32_t)m->top_k, (uint32_t)m->hidden, d_out, out_stride);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_moe_ffn(const OxhMoe *m, const float *d_logits, const float *d_x, size_t x_stride,
                           size_t n_tok, float *d_out, size_t out_stride, void *d_workspace,
                           size_t workspace_bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    MoeLayout l;
    if ((rc = moe_layout(m, n_tok, &l))) return rc;
    if (!d_logits || !d_x || !d_out || !d_workspace || !m->d_w_gate || !m->d_w_up || !m->d_w_down)
        return arg_fail("oxh_moe_ffn: NULL pointer");
    if (workspace_bytes < l.total) return arg_fail("oxh_moe_ffn: workspace too small (see oxh_moe_workspace_bytes)");
    if (x_stride < m->hidden || out_stride < m->hidden) return arg_fail("oxh_moe_ffn: stride < hidden");
    if ((uintptr_t)d_workspace & 255u) return arg_fail("oxh_moe_ffn: workspace must be 256-byte aligned");
    return moe_ffn_run(m, l, d_logits, d_x, x_stride, n_tok, d_out, out_stride, (uint8_t *)d_workspace, stream);
}

/* The workspace of oxh_moe_ffn_static: part of the library's device image, one copy per GPU, held
 * until the process ends.  In host code `scratch` is only a handle for hipGetSymbolAddress; the
 * device address it stands for is looked up once per device in oxh_init and kept in g_scratch. */
static __device__ __align__(256) unsigned char scratch[OXH_MOE_STATIC_WORKSPACE_BYTES];
#define OXH_MAX_DEVICES 64
static uint8_t *g_scratch[OXH_MAX_DEVICES];

static int resolve_scratch(int device)
{
    if (device < 0 || device >= OXH_MAX_DEVICES) return arg_fail("device index beyond the library's table");
    if (g_scratch[device]) return OXH_OK;
    void *p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p || ((uintptr_t)p & 255u)) return arg_fail("the static workspace has no usable device address");
    g_scratch[device] = (uint8_t *)p;
    return OXH_OK;
}

extern "C" int oxh_moe_ffn_static(const OxhMoe *m, const float *d_logits, const float *d_x, size_t x_stride,
                                  size_t n_tok, float *d_out, size_t out_stride, void *stream)
{
    /* nothing here may allocate: no lazy initialisation either */
    const int device = g_device.load(std::memory_order_acquire);
    if (device < 0) return arg_fail("oxh_moe_ffn_static: call oxh_init first (this entry point allocates nothing)");
    MoeLayout l;
    int rc;
    if ((rc = moe_layout(m, n_tok, &l))) return rc;
    if (!d_logits || !d_x || !d_out || !m->d_w_gate || !m->d_w_up || !m->d_w_down)
        return arg_fail("oxh_moe_ffn_static: NULL pointer");
    if (x_stride < m->hidden || out_stride < m->hidden) return arg_fail("oxh_moe_ffn_static: stride < hidden");
    if (l.total > (size_t)OXH_MOE_STATIC_WORKSPACE_BYTES) {
        snprintf(g_err, sizeof g_err, "oxh_moe_ffn_static: this layer needs %zu bytes of workspace, the built-in "
                 "one holds %zu; use oxh_moe_ffn with a workspace of your own", l.total,
                 (size_t)OXH_MOE_STATIC_WORKSPACE_BYTES);
        return OXH_ERR_TOO_WIDE;
    }
    uint8_t *ws = g_scratch[device];
    if (!ws) return arg_fail("oxh_moe_ffn_static: the static workspace was not resolved at oxh_init");
    /* every part of the workspace a launch reads has been written by an earlier launch of the same call,
     * so nothing needs clearing between calls */
    return moe_ffn_run(m, l, d_logits, d_x, x_stride, n_tok, d_out, out_stride, ws, stream);
}

/* ─── memory / stream / event plumbing ────────────────────────────────── */

extern "C" int oxh_host_alloc(void **h_ptr, size_t bytes)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (!h_ptr) return arg_fail("oxh_host_alloc: NULL");
    hipError_t e = hipHostMalloc(h_ptr, bytes ? bytes : 1, hipHostMallocDefault);
    if (e == hipErrorOutOfMemory) {
        snprintf(g_err, sizeof g_err, "out of host memory pinning %zu bytes", bytes);
        (void)hipGetLastError();
        return OXH_ERR_NOMEM;
    }
    if (e != hipSuccess) return hip_fail(e, "hipHostMalloc");
    return OXH_OK;
}

extern "C" int oxh_host_free(void *h_ptr)
{
    if (!h_ptr) return OXH_OK;
    HIP_TRY(hipHostFree(h_ptr));
    return OXH_OK;
}

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

extern "C" int oxh_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    HIP_TRY(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_memcpy2d_h2d(void *d_dst, size_t d_pitch, const void *h_src, size_t h_pitch, size_t width,
                                size_t height, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (width == 0 || height == 0) return OXH_OK;
    if (d_pitch < width || h_pitch < width) return arg_fail("oxh_memcpy2d_h2d: pitch < width");
    HIP_TRY(hipMemcpy2DAsync(d_dst, d_pitch, h_src, h_pitch, width, height, hipMemcpyHostToDevice,
                             pick_stream(stream)));
    return OXH_OK;
}

extern "C" int oxh_memcpy2d_d2h(void *h_dst, size_t h_pitch, const void *d_src, size_t d_pitch, size_t width,
                                size_t height, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (width == 0 || height == 0) return OXH_OK;
    if (d_pitch < width || h_pitch < width) return arg_fail("oxh_memcpy2d_d2h: pitch < width");
    HIP_TRY(hipMemcpy2DAsync(h_dst, h_pitch, d_src, d_pitch, width, height, hipMemcpyDeviceToHost,
                             pick_stream(stream)));
    return OXH_OK;
}

/* Bytes [0, bytes) of dst become `value`: byte stores up to the first 16-byte boundary and after the
 * last, 16-byte stores between.  A kernel rather than hipMemsetAsync so that a caller may record it
 * into a graph. */
__global__ __launch_bounds__(256) void
k_fill(uint8_t *__restrict__ dst, size_t bytes, uint32_t pattern)
{
    const size_t head = min(bytes, (size_t)((16u - ((uintptr_t)dst & 15u)) & 15u));
    const size_t n16 = (bytes - head) / 16u;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    u32x4 *mid = reinterpret_cast<u32x4 *>(dst + head);
    const u32x4 v = { pattern, pattern, pattern, pattern };
    for (size_t i = tid; i < n16; i += stride) mid[i] = v;
    const size_t tail_at = head + n16 * 16u;
    if (tid < head) dst[tid] = (uint8_t)pattern;
    if (tid < bytes - tail_at) dst[tail_at + tid] = (uint8_t)pattern;
}

extern "C" int oxh_memset(void *d_dst, int value, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    if (!d_dst) return arg_fail("oxh_memset: NULL pointer");
    const uint32_t b = (uint32_t)value & 0xFFu, pattern = b * 0x01010101u;
    size_t blocks = (bytes / 16u + 255u) / 256u;
    const size_t cap = (size_t)(g_n_cu > 0 ? g_n_cu : 256) * 8u;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(k_fill, dim3((uint32_t)blocks), dim3(256), 0, pick_stream(stream), (uint8_t *)d_dst, bytes,
                       pattern);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* 16-byte pieces of src to dst, both 16-byte aligned, bytes a multiple of 16.  The host layer uses it
 * to pull a call's input out of page-locked host memory (which the device reads in place) and to push
 * results there: for the few tens of KB of a decode call a launch costs less than a copy through the
 * DMA engines. */
__global__ __launch_bounds__(256) void
k_copy16(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src, size_t n16)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

extern "C" int oxh_internal_copy16(void *dst, const void *src, size_t bytes, void *stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (bytes == 0) return OXH_OK;
    if (!dst || !src || (((uintptr_t)dst | (uintptr_t)src | bytes) & 15u))
        return arg_fail("oxh_internal_copy16: pointers and size must be multiples of 16");
    const size_t n16 = bytes / 16u;
    if (n16 > ((size_t)1 << 31)) return arg_fail("oxh_internal_copy16: too large");
    hipLaunchKernelGGL(k_copy16, dim3((uint32_t)((n16 + 255u) / 256u)), dim3(256), 0, pick_stream(stream),
                       (u32x4 *)dst, (const u32x4 *)src, n16);
    HIP_TRY(hipGetLastError());
    return OXH_OK;
}

/* Wait for the stream by polling it: a blocking wait sleeps on an interrupt and wakes up some
 * microseconds after the work is done, which a decode-sized call notices.  After `spins` polls the
 * blocking wait takes over, so a long batch does not burn a core. */
extern "C" int oxh_internal_stream_sync_spin(void *stream, unsigned spins)
{
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = pick_stream(stream);
    for (unsigned i = 0; i < spins; i++) {
        const hipError_t e = hipStreamQuery(s);
        if (e == hipSuccess) return OXH_OK;
        if (e != hipErrorNotReady) return hip_fail(e, "hipStreamQuery");
    }
    HIP_TRY(hipStreamSynchronize(s));
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

extern "C" int oxh_mem_info(size_t *free_bytes, size_t *total_bytes)
{
    int rc = ensure_init();
    if (rc) return rc;
    size_t f = 0, t = 0;
    HIP_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return OXH_OK;
}

/* The table behind include/oxhip_lab.h. */
extern "C" const OxhLab *oxh_lab(void)
{
    static const OxhLab lab = { oxh_debug_plan_stamps, oxh_debug_plan_phantom, oxh_debug_moe_workspace_parts,
                                oxh_debug_read_probe, oxh_debug_mfma_probe, oxh_debug_subblock_sums };
    return &lab;
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
