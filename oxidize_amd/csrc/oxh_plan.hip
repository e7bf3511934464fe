/*
 * oxh_plan.hip — a whole decode step as ONE launch.
 *
 * A decode step of a dense model is a fixed chain of a hundred-odd matrix-vector
 * products (q/k/v, o, gate/up, down per layer), each a few microseconds long.
 * Launched one by one, every product pays the gap between two kernels, the
 * fetch of its arguments and a cold start of its weight stream; the reference's
 * device path therefore submits the whole token chain at once
 * (oxidize-c/include/oxidize/cuda.h:250-265).  Here the chain is compiled into a
 * table of operations in device memory (an OxhPlan) and walked by one
 * persistent kernel: one 16-wave workgroup per compute unit, every workgroup
 * taking its share of the rows of every operation.
 *
 *   - The arithmetic is the GEMV kernels' (gemv_kernels.inc): same lane split,
 *     same per-block f32 term, same strictly ordered per-row sum, so results
 *     are bit-identical to oxh_gemv_segments_fused launched op by op.
 *   - A wave asks for the first two passes of weights of the NEXT operation
 *     as soon as its registers are free, before it sums its rows: weights do
 *     not depend on activations, so the weight stream does not stop at an
 *     operation boundary.
 *   - An operation that reads what an earlier one wrote waits until every
 *     workgroup has finished that one.  Workgroups announce progress with one
 *     monotonic counter each, stored in eight copies; every workgroup reads
 *     all counters of one copy (plan_wait).  The eight L2 caches of the device are not coherent with each
 *     other and a fence that makes them so costs 35 us here, so there are no
 *     fences: everything one operation hands to another (outputs, residual
 *     sums) is stored and loaded with system-coherent accesses that bypass the
 *     L2s, and so are the counters.
 *   - A plan none of whose operations reads what another one writes (a decode
 *     step's matrices applied to inputs that are all there when the launch
 *     starts) runs on a second kernel, k_plan_ext: each input vector is
 *     normalised and quantised ONCE, by one workgroup, into a staged image in
 *     device memory before the chain starts; after one device-wide wait every
 *     workgroup copies the image of operation i + 1 straight into LDS while it
 *     works on operation i.  An operation boundary then costs the row sums
 *     and one workgroup barrier; no workgroup reads or quantises a vector that
 *     255 others quantise as well.
 *   - Every wait is bounded: after `spin_limit` polls a workgroup raises the
 *     plan's error word and leaves, and every other workgroup leaves at its
 *     next wait, so a launch that cannot make progress (not all workgroups
 *     resident) ends by itself.
 *
 * Wave64, gfx950.  Build flags as oxh_kernels.hip.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "oxhip.h"
#include "oxh_internal.h"

#pragma clang fp contract(off)

#include "oxh_device.inc"
#include "gemv_kernels.inc"

#define PLAN_MAX_SEGS 8             /* segments of a table row */
#define PLAN_OP_SEGS 4              /* segments of an operation as the caller gives it */
#define PLAN_W 16u                  /* waves per workgroup */
#define PLAN_MAX_WG 1024u
#define PLAN_MAX_BLOCKS 64u         /* super-blocks per row: four units per wave staged at once */

#define PLAN_Q4_K 0u
#define PLAN_Q5_K 1u
#define PLAN_Q6_K 2u
#define PLAN_Q6_KG 3u               /* Q6_K regrouped in runs of eight blocks (OXH_Q6_K_G8) */

/* Device addresses travel through the table as integers and become global-memory pointers in the
 * kernel: a pointer merely loaded from memory is a generic one to the compiler, and loads through it
 * are flat_load, counted by lgkmcnt as well as vmcnt, so that every LDS wait would wait for them. */
typedef uint64_t gaddr;

struct PlanSeg {
    gaddr w, w2;                    /* w2: the paired matrix or 0 */
    gaddr out;
    uint32_t rows, wg_begin, rows_q, rows_rem;
    gaddr xq;                       /* k_plan_ext: the staged input this segment multiplies (segments of one
                                     * table row may come from different operations, see plan_merge);
                                     * k_plan: the segment's rows dealt to its workgroups, rows per workgroup
                                     * in the low word, the workgroups that take one more in the high word */
};

struct PlanOp {
    uint32_t kind, pro, n_segs, blocks;
    uint32_t magic, term_stride, rows_cap, n_wg;
    uint32_t wait;                  /* 0, or 1 + index of the operation that must be complete everywhere */
    uint32_t signal;                /* a later operation waits for this one */
    float eps;
    uint32_t pad;
    gaddr x, pro_b, pro_add;
    gaddr pro_sum_out, pro_out;
    gaddr act_out;
    gaddr xq;                       /* where the staged (quantised) input of this operation is kept when the
                                     * plan stages its inputs ahead of the chain; else 0 */
    gaddr reserved;
    PlanSeg s[PLAN_MAX_SEGS];
};

static_assert(sizeof(PlanOp) % 16 == 0, "table rows are copied in 16-byte pieces");

/* progress counters: flags[copy][wg], then go[0] = the minimum workgroup 0 publishes (copies = 0), go[1] = error word */
struct PlanSync {
    uint32_t *flags;
    uint32_t *go;
    uint32_t n_wait;                /* counters gathered: the grid size (one more in the time-out test) */
    uint32_t copies;                /* copies of every counter that every workgroup gathers from, or 0: workgroup 0 gathers */
    uint32_t spin_limit;
    uint64_t *stamps;               /* measurement aid: [op][workgroup][8] clock readings, or NULL */
    uint32_t *host_err;             /* page-locked host word that mirrors go[1], so that the next launch can be refused */
};

#define PLAN_STAMPS 8u

/* wave 0 of a workgroup notes the shader clock at phase `slot` of operation `op` */
/* ON: the kernel variant a plan runs once clock stamps have been asked for (a measurement hook).  The
 * ordinary variants carry none of it: the chained kernel is short of scalar registers, and the stamps' pointer
 * and tests alone cost it five scalars kept in vector lanes and 20 us per 128-operation step. */
template <bool ON>
__device__ __forceinline__ void plan_stamp(const PlanSync &sy, uint32_t op, uint32_t slot, uint32_t lane, uint32_t wave)
{
    if (ON && sy.stamps != nullptr && wave == 0u && lane == 0u)
        sy.stamps[((size_t)op * gridDim.x + blockIdx.x) * PLAN_STAMPS + slot] = __builtin_amdgcn_s_memrealtime();
}

struct PlanLds {
    uint32_t act_bytes;             /* one staged activation (two are kept, used in turn) */
    uint32_t outs_off, red_off, terms_off, terms_per_wave;   /* bytes; terms_per_wave in floats */
    uint32_t table_off;             /* the operation table's copy */
    uint32_t terms_wg;              /* k_plan_ext: floats of one workgroup-wide term table (two are kept) */
};

/* ─── coherent accesses ───────────────────────────────────────────────── */

/* System-scope accesses (sc0 sc1) go past the per-XCD L2s to the memory side, where every XCD sees
 * the same data.  Single words use the atomic builtins; 16-byte pieces use buffer instructions with
 * that cache policy (a volatile generic access would compile to flat_load, which also counts as an
 * LDS operation).  Bit 31 of the policy marks the access volatile for the compiler, so that a poll
 * is not hoisted out of its loop and nothing moves across it. */
#define OXH_SYSTEM_COHERENT ((int)(0x11u | 0x80000000u))

typedef __amdgpu_buffer_rsrc_t CohBuf;

__device__ __forceinline__ CohBuf coh_buf(const void *base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7FFFFFFF, 0x27000);
}
__device__ __forceinline__ u32x4 cload16(CohBuf b, uint32_t byte_off)
{
    return __builtin_amdgcn_raw_buffer_load_b128(b, (int)byte_off, 0, OXH_SYSTEM_COHERENT);
}
__device__ __forceinline__ uint32_t cload(const uint32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void cstore(uint32_t *p, uint32_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void cstore_f32(CohBuf b, uint32_t byte_off, float v)
{
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), b, (int)byte_off, 0, OXH_SYSTEM_COHERENT);
}
__device__ __forceinline__ XRegs cload4(CohBuf b, uint32_t byte_off)
{
    const u32x4 v = cload16(b, byte_off);
    XRegs r;
    r.v0 = __uint_as_float(v.x); r.v1 = __uint_as_float(v.y);
    r.v2 = __uint_as_float(v.z); r.v3 = __uint_as_float(v.w);
    return r;
}
__device__ __forceinline__ void cstore4(CohBuf b, uint32_t byte_off, const XRegs &y)
{
    u32x4 v = { __float_as_uint(y.v0), __float_as_uint(y.v1), __float_as_uint(y.v2), __float_as_uint(y.v3) };
    __builtin_amdgcn_raw_buffer_store_b128(v, b, (int)byte_off, 0, OXH_SYSTEM_COHERENT);
}

/* workgroup barrier that orders LDS only: __syncthreads() may also wait for every
 * global load in flight, and the prefetched weights of the next operation are */
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T>
__device__ __forceinline__ T *gptr(gaddr v)
{
    typedef T __attribute__((address_space(1))) *G;
    return (T *)reinterpret_cast<G>(v);
}

/* The operation table is copied into LDS when the kernel starts: read from global memory, a row costs
 * a trip to HBM (the weight stream flushes it out of every cache between two uses), in the middle of
 * staging.  Fields are the same for every lane; readfirstlane says so to the compiler, and everything
 * computed from them stays in scalar registers. */
__device__ __forceinline__ uint32_t uni(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ gaddr uni(gaddr v)
{
    return (gaddr)uni((uint32_t)v) | ((gaddr)uni((uint32_t)(v >> 32)) << 32);
}
__device__ __forceinline__ float uni(float v) { return __uint_as_float(uni(__float_as_uint(v))); }

/* the per-operation fields staging and the passes use */
struct OpHead {
    uint32_t kind, pro, blocks, magic, term_stride, rows_cap, wait, signal;
    float eps;
    gaddr x, pro_b, pro_add, pro_sum_out, pro_out, act_out;
};

__device__ __forceinline__ OpHead plan_head(const PlanOp *op)
{
    OpHead h;
    h.kind = uni(op->kind); h.pro = uni(op->pro); h.blocks = uni(op->blocks); h.magic = uni(op->magic);
    h.term_stride = uni(op->term_stride); h.rows_cap = uni(op->rows_cap); h.wait = uni(op->wait);
    h.signal = uni(op->signal); h.eps = uni(op->eps);
    h.x = uni(op->x); h.pro_b = uni(op->pro_b); h.pro_add = uni(op->pro_add);
    h.pro_sum_out = uni(op->pro_sum_out); h.pro_out = uni(op->pro_out); h.act_out = uni(op->act_out);
    return h;
}

/* ─── what a wave owns of an operation ───────────────────────────────── */

struct PWork {
    WSrc src;                       /* flat block list: nblk blocks, the first n1 in src.a */
    float *out;                     /* the segment's output vector */
    uint32_t nblk, nrows, row0;
    uint32_t wg_row0, wg_rows;      /* the workgroup's contiguous run of rows */
    uint32_t kind;
    uint32_t paired;                /* 0 / 1 (a whole word: the struct is copied around as scalars) */
    gaddr xq;                       /* the workgroup's segment's staged input (k_plan_ext) */
};

__device__ __forceinline__ uint32_t plan_block_bytes(uint32_t kind)
{
    return kind >= PLAN_Q6_K ? 210u : kind == PLAN_Q5_K ? 176u : 144u;
}

__device__ __forceinline__ PWork plan_work(const PlanOp *op, uint32_t wave)
{
    PWork k;
    const uint32_t wg = blockIdx.x, n = uni(op->n_segs);
    uint32_t si = 0;
#pragma unroll
    for (uint32_t i = 1; i < PLAN_MAX_SEGS; i++)
        if (i < n && wg >= uni(op->s[i].wg_begin)) si = i;
    const PlanSeg *sg = &op->s[si];
    const gaddr w = uni(sg->w), w2 = uni(sg->w2), out = uni(sg->out);
    const uint32_t wg_begin = uni(sg->wg_begin);
    const bool idle = wg >= uni(op->n_wg);
    /* Rows go to the segment's workgroups first and a workgroup's rows to its waves second, both as evenly
     * as whole rows allow.  (Dealt to the waves of all workgroups in one go, 14336 gate/up pairs over 4096
     * waves gave the first 2048 waves four pairs and the others three: half of the workgroups carried a
     * third more than the others, and an operation of a chain ends with its slowest workgroup.  32-layer
     * chain 1.320 -> 1.286 ms.) */
    const gaddr deal = uni(sg->xq);
    const uint32_t per_wg = (uint32_t)deal, more = (uint32_t)(deal >> 32);
    const uint32_t wgi = idle ? 0u : wg - wg_begin;
    k.kind = uni(op->kind);
    k.xq = 0u;
    k.wg_row0 = wgi * per_wg + min(wgi, more);
    k.wg_rows = idle ? 0u : per_wg + (wgi < more ? 1u : 0u);
    const uint32_t q = k.wg_rows / PLAN_W, rem = k.wg_rows % PLAN_W;
    k.row0 = k.wg_row0 + wave * q + min(wave, rem);
    k.nrows = idle ? 0u : q + (wave < rem ? 1u : 0u);
    k.out = gptr<float>(out);
    const uint32_t B = uni(op->blocks);
    const size_t off = (size_t)(k.nrows ? k.row0 : 0u) * B * plan_block_bytes(k.kind);
    k.src.a = gptr<const uint8_t>(w + off);
    k.src.n1 = k.nrows * B;
    k.paired = w2 != 0u ? 1u : 0u;
    k.src.b = gptr<const uint8_t>((k.paired ? w2 : w) + off);
    k.nblk = k.paired ? 2u * k.src.n1 : k.src.n1;
    return k;
}

/* The same rows dealt evenly: the workgroup's rows of the first matrix followed by its rows of the
 * paired one form one list, and wave w takes an equal contiguous run of it (a pair of 56 rows each is
 * seven rows per wave, where dealing pairs gives eight waves four pairs and eight waves three).  A
 * wave's rows of the two matrices are then not the same rows, so the term table is the workgroup's
 * (row0 = the wave's first list row) and rows are summed after a workgroup barrier. */
__device__ __forceinline__ PWork plan_work_flat(const PlanOp *op, uint32_t wave)
{
    PWork k;
    const uint32_t wg = blockIdx.x, n = uni(op->n_segs);
    uint32_t si = 0;
#pragma unroll
    for (uint32_t i = 1; i < PLAN_MAX_SEGS; i++)
        if (i < n && wg >= uni(op->s[i].wg_begin)) si = i;
    const PlanSeg *sg = &op->s[si];
    const gaddr w = uni(sg->w), w2 = uni(sg->w2), out = uni(sg->out);
    const uint32_t wg_begin = uni(sg->wg_begin), sq = uni(sg->rows_q), srem = uni(sg->rows_rem);
    const bool idle = wg >= uni(op->n_wg);
    const uint32_t wi0 = (wg - wg_begin) * PLAN_W;
    k.kind = uni(op->kind);
    k.xq = idle ? (gaddr)0u : uni(sg->xq);
    k.out = gptr<float>(out);
    k.paired = w2 != 0u ? 1u : 0u;
    k.wg_row0 = wi0 * sq + min(wi0, srem);
    k.wg_rows = idle ? 0u : (wi0 + PLAN_W) * sq + min(wi0 + PLAN_W, srem) - k.wg_row0;
    const uint32_t B = uni(op->blocks);
    const gaddr rb = (gaddr)(B * plan_block_bytes(k.kind));
    const uint32_t F = k.paired ? 2u * k.wg_rows : k.wg_rows;
    const uint32_t q = F / PLAN_W, rem = F % PLAN_W;
    const uint32_t f0 = wave * q + min(wave, rem), cnt = q + (wave < rem ? 1u : 0u);
    /* rows of the first matrix in this wave's run, and where its rows of the second one start */
    const uint32_t na = f0 < k.wg_rows ? min(cnt, k.wg_rows - f0) : 0u;
    const uint32_t b0 = f0 < k.wg_rows ? 0u : f0 - k.wg_rows;
    const gaddr first = w + (gaddr)(k.wg_row0 + min(f0, k.wg_rows)) * rb;
    const gaddr second = (k.paired ? w2 : w) + (gaddr)(k.wg_row0 + b0) * rb;
    /* a run that lies wholly in the second matrix is a one-matrix list of that one */
    k.src.a = gptr<const uint8_t>(na != 0u ? first : second);
    k.src.b = gptr<const uint8_t>(second);
    k.src.n1 = (na != 0u ? na : cnt) * B;
    k.row0 = f0;
    k.nrows = cnt;
    k.nblk = cnt * B;
    return k;
}

/* ─── weight register sets, untyped so that they can cross operations ── */

/* named members, not an array: stores to an array from the three format branches get merged into one
 * store at a computed index, and the set then lives in scratch memory instead of registers */
struct WSet { u32x4 a, b, c, d, e; };      /* e: Q5_K only (kernels built without Q5_K never touch it) */

__device__ __forceinline__ u32x4 as_v4(const U32x4u2 &t) { u32x4 v = { t.x, t.y, t.z, t.w }; return v; }
__device__ __forceinline__ U32x4u2 as_u2(const u32x4 &v) { U32x4u2 t; t.x = v.x; t.y = v.y; t.z = v.z; t.w = v.w; return t; }

template <bool HAS_Q5>
__device__ __forceinline__ void wset_load(uint32_t kind, WSet &s, const WSrc &src, uint32_t g, uint32_t lane)
{
    const uint32_t sub = lane & 3u;
    /* the branches produce values, the set is written once after them: stores to different members
     * from different branches would be merged into one store at a computed address */
    u32x4 v0, v1, v2, v3 = s.d, v4 = s.e;
    if (kind == PLAN_Q6_K) {
        Q6kRegs t;
        q6k_load<true>(t, src, g, sub >> 1, sub & 1u);
        v0 = as_v4(t.la); v1 = as_v4(t.lb); v2 = as_v4(t.hh); v3 = as_v4(t.tail);
    } else if (kind == PLAN_Q6_KG) {
        Q6kRegs t;
        q6k_load<true, true>(t, src, g, sub >> 1, sub & 1u);
        v0 = as_v4(t.la); v1 = as_v4(t.lb); v2 = as_v4(t.hh); v3 = as_v4(t.tail);
    } else if (HAS_Q5 && kind == PLAN_Q5_K) {
        Q4kRegs t;
        q4k_load<true, true>(t, src, g, sub);
        v0 = t.hdr; v1 = t.na; v2 = t.nb; v3 = t.ha; v4 = t.hb;
    } else {
        Q4kRegs t;
        q4k_load<false, true>(t, src, g, sub);
        v0 = t.hdr; v1 = t.na; v2 = t.nb;
    }
    s.a = v0; s.b = v1; s.c = v2; s.d = v3;
    if (HAS_Q5) s.e = v4;
}

/* pass `pass` (0 or 1) of an operation into a register set */
template <bool HAS_Q5>
__device__ __forceinline__ void plan_prefetch(const PWork &k, WSet &S, uint32_t pass, uint32_t lane)
{
    if (k.nblk == 0u) return;
    wset_load<HAS_Q5>(k.kind, S, k.src, min(pass * 16u + (lane >> 2), k.nblk - 1u), lane);
}

/* ─── the passes of one operation (sets A and B hold passes 0 and 1) ──── */

template <bool Q5>
__device__ __forceinline__ void
plan_passes_q45(const WSet &A0, const WSet &B0, const PWork &k, const GemvParams &p, const uint8_t *act,
                uint32_t act_lds, float *terms, uint32_t lane)
{
    const uint32_t nblk = k.nblk, B = p.blocks, s = lane & 3u;
    Q4kRegs A, Bq;
    A.hdr = A0.a; A.na = A0.b; A.nb = A0.c;
    Bq.hdr = B0.a; Bq.na = B0.b; Bq.nb = B0.c;
    if (Q5) { A.ha = A0.d; A.hb = A0.e; Bq.ha = B0.d; Bq.hb = B0.e; }
    Q4kLane ln;
    ln.s = s;
    ln.hi = s >= 2u;
    ln.sh = (s & 1u) * 16u;
    ln.mask_a = ln.hi ? 0x0F0F0F0Fu : 0x3F3F3F3Fu;
    ln.mask_b = ln.hi ? 0x30303030u : 0u;
    const uint32_t last = nblk - 1u, npass = (nblk + 15u) / 16u;
    const uint32_t lb = lane >> 2;
    uint32_t i = 0;
    while (i + 3u < npass) {
        q4k_pass<1, false, Q5>(A, ln, p, act, act_lds, 1u, B, i * 16u + lb, nblk, k.row0, terms);
        q4k_load<Q5, true>(A, k.src, min((i + 2u) * 16u + lb, last), s);
        q4k_pass<1, false, Q5>(Bq, ln, p, act, act_lds, 1u, B, (i + 1u) * 16u + lb, nblk, k.row0, terms);
        q4k_load<Q5, true>(Bq, k.src, min((i + 3u) * 16u + lb, last), s);
        i += 2u;
    }
    const uint32_t rem = npass - i;                 /* 1, 2 or 3 */
    q4k_pass<1, false, Q5>(A, ln, p, act, act_lds, 1u, B, i * 16u + lb, nblk, k.row0, terms);
    if (rem == 3u) q4k_load<Q5, true>(A, k.src, min((i + 2u) * 16u + lb, last), s);
    if (rem >= 2u) q4k_pass<1, false, Q5>(Bq, ln, p, act, act_lds, 1u, B, (i + 1u) * 16u + lb, nblk, k.row0, terms);
    if (rem == 3u) q4k_pass<1, false, Q5>(A, ln, p, act, act_lds, 1u, B, (i + 2u) * 16u + lb, nblk, k.row0, terms);
}

template <bool G8>
__device__ __forceinline__ void
plan_passes_q6(const WSet &A0, const WSet &B0, const PWork &k, const GemvParams &p, const uint8_t *act,
               uint32_t act_lds, float *terms, uint32_t lane)
{
    const uint32_t nblk = k.nblk, B = p.blocks, u = lane & 3u, n = u >> 1, lh = u & 1u;
    Q6kRegs A, Bq;
    A.la = as_u2(A0.a); A.lb = as_u2(A0.b); A.hh = as_u2(A0.c); A.tail = as_u2(A0.d);
    Bq.la = as_u2(B0.a); Bq.lb = as_u2(B0.b); Bq.hh = as_u2(B0.c); Bq.tail = as_u2(B0.d);
    const uint32_t last = nblk - 1u, npass = (nblk + 15u) / 16u;
    const uint32_t lb = lane >> 2;
    uint32_t i = 0;
    while (i + 3u < npass) {
        q6k_pass<1, false, G8>(A, u, p, act, act_lds, 1u, B, i * 16u + lb, nblk, k.row0, terms);
        q6k_load<true, G8>(A, k.src, min((i + 2u) * 16u + lb, last), n, lh);
        q6k_pass<1, false, G8>(Bq, u, p, act, act_lds, 1u, B, (i + 1u) * 16u + lb, nblk, k.row0, terms);
        q6k_load<true, G8>(Bq, k.src, min((i + 3u) * 16u + lb, last), n, lh);
        i += 2u;
    }
    const uint32_t rem = npass - i;
    q6k_pass<1, false, G8>(A, u, p, act, act_lds, 1u, B, i * 16u + lb, nblk, k.row0, terms);
    if (rem == 3u) q6k_load<true, G8>(A, k.src, min((i + 2u) * 16u + lb, last), n, lh);
    if (rem >= 2u) q6k_pass<1, false, G8>(Bq, u, p, act, act_lds, 1u, B, (i + 1u) * 16u + lb, nblk, k.row0, terms);
    if (rem == 3u) q6k_pass<1, false, G8>(A, u, p, act, act_lds, 1u, B, (i + 2u) * 16u + lb, nblk, k.row0, terms);
}

/* per-row sums in block order into the workgroup's output staging; a paired operation writes
 * silu(first) * second (the expression of row_sums_paired) */
__device__ __forceinline__ void
plan_row_sums(const float *terms, const PWork &k, uint32_t B, uint32_t term_stride, float *outs, uint32_t lane)
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    for (uint32_t r = lane; r < k.nrows; r += 64u) {
        const float *t = terms + __umul24(r, term_stride);
        float v = row_sum_one<1>(t, B);
        if (k.paired) {
            const float u = row_sum_one<1>(t + __umul24(k.nrows, term_stride), B);
            const float sig = 1.0f / (1.0f + expf(-v));
            v = v * sig * u;
        }
        outs[k.row0 - k.wg_row0 + r] = v;
    }
}

/* ─── activation staging: one f32 vector -> Q8_K in LDS ──────────────── */

/* Staging is split in two so that the loads can be placed where they hurt least in the wave's
 * in-order memory queue: plan_stage_issue asks for this wave's part of the input vector and of whatever
 * the prologue combines it with; plan_stage_finish applies the prologue, quantises and writes LDS.  A
 * vector another workgroup wrote a moment ago is read with coherent loads; inputs nobody in this launch
 * wrote come through the caches.
 *
 * The launches (stage_begin / stage_end) give a wave one 256-value unit at a time, lane l holding
 * values 4l .. 4l+3.  Here a block goes to 16 lanes: lane l of a row holds values 16l .. 16l+15 of
 * block 4 * wave + row.  An instruction costs a 1024-thread workgroup sixteen issue slots whatever its
 * lanes do, so the quantiser's fixed part (maximum, two divisions, slot arithmetic, stores) is paid once
 * per four blocks instead of once per block, and for 4096 values four waves run it while twelve go on
 * to their weight requests.  The bytes are the launches': a maximum and the integer sums do not depend
 * on the order they are taken in, and the sum of squares is added in the launches' order.  There, lane
 * L of wave W adds up its four squares of units W, W + 16, ... in turn, the wave adds its lanes in
 * four exchange steps (neighbour, pair, eight, sixteen) and combines its four rows as (r0 + r1) + (r2 +
 * r3), and the waves' sums are added the same way.  A lane here holds what four neighbouring lanes
 * hold there: row 4w + r of waves 0..3 stands for wave W = 4w + r, walks W's units, does the first two
 * steps in registers, and the same four exchange instructions then perform the launches' last two steps
 * and the combination of the four rows. */
struct XStage {
    XRegs x[4], t[4], b[4];
};

/* Every vector that may have been written in this launch is read with coherent loads, whether it was
 * or not: choosing the instruction per load at run time gives the compiler two definitions of each
 * register to merge, which it does with a move, and a move waits for the load (and for the weights
 * requested before it). */
__device__ __forceinline__ void
plan_stage_issue(const OpHead &op, XStage &xs, uint32_t lane, uint32_t wave)
{
    const uint32_t pro = op.pro;
    const float *b = gptr<const float>(op.pro_b);
    const CohBuf xc = coh_buf(gptr<const float>(op.x)), ac = coh_buf(gptr<const float>(op.pro_add)), bc = coh_buf(b);
    const uint32_t blk = wave * 4u + (lane >> 4);
    if (blk < op.blocks) {
        const uint32_t at0 = blk * 256u + 16u * (lane & 15u);
#pragma unroll
        for (int j = 0; j < 4; j++) xs.x[j] = cload4(xc, (at0 + 4u * (uint32_t)j) * 4u);
        if (pro == GEMV_PRO_ADD_RMSNORM) {
#pragma unroll
            for (int j = 0; j < 4; j++) xs.t[j] = cload4(ac, (at0 + 4u * (uint32_t)j) * 4u);
        }
        if (pro == GEMV_PRO_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j++) xs.b[j] = cload4(bc, (at0 + 4u * (uint32_t)j) * 4u);
        } else if (pro != GEMV_PRO_NONE) {
#pragma unroll
            for (int j = 0; j < 4; j++) xs.b[j] = x_load4(b + at0 + 4u * (uint32_t)j);      /* norm weights: constants */
        }
    }
}

__device__ __forceinline__ int quantize_sum4(const XRegs &y, float inv, uint32_t &packed)
{
    const int q0 = quantize_one(y.v0, inv), q1 = quantize_one(y.v1, inv);
    const int q2 = quantize_one(y.v2, inv), q3 = quantize_one(y.v3, inv);
    packed = (uint32_t)(q0 & 255) | ((uint32_t)(q1 & 255) << 8) | ((uint32_t)(q2 & 255) << 16) |
             ((uint32_t)(q3 & 255) << 24);
    return q0 + q1 + q2 + q3;
}

template <int KIND /* 0 Q4_K/Q5_K layout, 1 Q6_K layout */>
__device__ __forceinline__ void
plan_stage_finish(const OpHead &op, const XStage &xs, uint8_t *base, float *red, bool storer,
                  uint32_t lane, uint32_t wave)
{
    constexpr bool Q6 = KIND == 1;
    const uint32_t B = op.blocks, pro = op.pro;
    const bool rms = pro == GEMV_PRO_RMSNORM || pro == GEMV_PRO_ADD_RMSNORM, add = pro == GEMV_PRO_ADD_RMSNORM;
    const uint32_t blk = wave * 4u + (lane >> 4), l = lane & 15u;
    XRegs xr[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        xr[j] = xs.x[j];
        if (add) { xr[j].v0 += xs.t[j].v0; xr[j].v1 += xs.t[j].v1; xr[j].v2 += xs.t[j].v2; xr[j].v3 += xs.t[j].v3; }
    }
    float inv = 1.0f;
    if (rms) {
        if (wave < PLAN_W / 4u) {
            /* rows beyond the vector hold zeros, the sums of the launches' idle waves */
            float p[4];
#pragma unroll
            for (int j = 0; j < 4; j++)
                p[j] = xr[j].v0 * xr[j].v0 + xr[j].v1 * xr[j].v1 + xr[j].v2 * xr[j].v2 + xr[j].v3 * xr[j].v3;
            /* vectors of more than sixteen blocks: the further units of the wave this row stands for,
             * one round trip each (their values are not kept: the rows that quantise them asked for
             * them already) */
            if (B > PLAN_W) {
                const CohBuf xc = coh_buf(gptr<const float>(op.x)), ac = coh_buf(gptr<const float>(op.pro_add));
                for (uint32_t b2 = blk + PLAN_W; b2 < B; b2 += PLAN_W) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint32_t at = b2 * 256u + 16u * l + 4u * (uint32_t)j;
                        XRegs v = cload4(xc, at * 4u);
                        if (add) {
                            const XRegs t = cload4(ac, at * 4u);
                            v.v0 += t.v0; v.v1 += t.v1; v.v2 += t.v2; v.v3 += t.v3;
                        }
                        p[j] += v.v0 * v.v0 + v.v1 * v.v1 + v.v2 * v.v2 + v.v3 * v.v3;
                    }
                }
            }
            float q = (p[0] + p[1]) + (p[2] + p[3]);
            q += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(q), 0xB1, 0xF, 0xF, false));
            q += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(q), 0x4E, 0xF, 0xF, false));
            q += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(q), 0x141, 0xF, 0xF, false));
            q += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(q), 0x140, 0xF, 0xF, false));
            if (l == 0u) red[blk] = q;
        }
        __syncthreads();
        if (wave * 4u < B) {
            const float tot = wave_sum_f32(lane < PLAN_W ? red[lane] : 0.0f);
            inv = 1.0f / sqrtf(tot / (float)(B * 256u) + op.eps);
        }
    }
    const bool has_sout = add && storer && op.pro_sum_out != 0u;
    const bool has_fout = pro != GEMV_PRO_NONE && storer && op.pro_out != 0u;
    if (blk < B) {
        const CohBuf sout = coh_buf(gptr<float>(op.pro_sum_out)), fout = coh_buf(gptr<float>(op.pro_out));
        const uint32_t at = blk * 256u + 16u * l;
        XRegs y[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (has_sout) cstore4(sout, (at + 4u * (uint32_t)j) * 4u, xr[j]);
            y[j] = xr[j];
            if (rms) y[j] = prologue_apply<GEMV_PRO_RMSNORM>(xr[j], xs.b[j], inv);
            else if (pro == GEMV_PRO_SWIGLU) y[j] = prologue_apply<GEMV_PRO_SWIGLU>(xr[j], xs.b[j], inv);
            if (has_fout) cstore4(fout, (at + 4u * (uint32_t)j) * 4u, y[j]);
        }
        float m = fmaxf(fmaxf(fabsf(y[0].v0), fabsf(y[0].v1)), fmaxf(fabsf(y[0].v2), fabsf(y[0].v3)));
#pragma unroll
        for (int j = 1; j < 4; j++)
            m = fmaxf(m, fmaxf(fmaxf(fabsf(y[j].v0), fabsf(y[j].v1)), fmaxf(fabsf(y[j].v2), fabsf(y[j].v3))));
        m = dpp_max_step(oct_max(m), 3);                /* over the row's sixteen lanes */
        const float d = m / 127.0f;
        const float invd = (d != 0.0f) ? 1.0f / d : 0.0f;
        u32x4 packed;
        uint32_t pk;
        int s16 = quantize_sum4(y[0], invd, pk); packed.x = pk;
        s16 += quantize_sum4(y[1], invd, pk); packed.y = pk;
        s16 += quantize_sum4(y[2], invd, pk); packed.z = pk;
        s16 += quantize_sum4(y[3], invd, pk); packed.w = pk;
        /* value dwords 4l .. 4l+3 of a block are neighbours in both staged layouts */
        *reinterpret_cast<u32x4 *>(reinterpret_cast<uint32_t *>(base) + q8k_slot<Q6>(B, blk, 4u * l)) = packed;
        if (Q6) {
            const uint32_t n = l >> 3, k = (l >> 1) & 3u, lh = l & 1u;
            reinterpret_cast<int32_t *>(base + B * 256u)[(blk * 4u + 2u * n + lh) * 4u + k] = -32 * s16;
        } else {
            const int bj = s16 + __builtin_amdgcn_update_dpp(0, s16, 0xB1, 0xF, 0xF, false);
            if ((l & 1u) == 0u) {
                const uint32_t j = l >> 1;
                reinterpret_cast<int16_t *>(base + B * 256u)[(blk * 4u + (j >> 1)) * 2u + (j & 1u)] = (int16_t)bj;
            }
        }
        if (l == 0u) reinterpret_cast<float *>(base + B * 256u + B * (Q6 ? 64u : 16u))[blk] = d;
        if (storer && op.act_out) {
            uint8_t *dst = gptr<uint8_t>(op.act_out) + (size_t)blk * 292u;
            uint32_t *qs = reinterpret_cast<uint32_t *>(dst + 4) + 4u * l;
            qs[0] = packed.x; qs[1] = packed.y; qs[2] = packed.z; qs[3] = packed.w;
            if (l == 0u) *reinterpret_cast<float *>(dst) = d;
            reinterpret_cast<int16_t *>(dst + 260)[l] = (int16_t)s16;
        }
    }
    /* the side outputs are acknowledged where the trip that follows the passes begins (k_plan), or after
     * the last staged input (k_plan_ext), before the barrier that precedes the announcement: nothing
     * else is in flight there, and here the wait would hold up the workgroup that stores them, which
     * every other workgroup then waits for */
}

/* Vectors of at most sixteen blocks in the chained kernel, staged the launches' own way: wave w takes
 * block w, lane l its values 4l .. 4l+3 (stage_begin / stage_end of the launches, with the loads that may
 * see another workgroup's stores made coherent).  In a chain every wave's weights are already on their
 * way when the vector arrives, so nothing is gained by leaving the vector to four waves of sixteen values
 * a lane: spread over sixteen waves the dependent chain from the vector's arrival to the staged bytes is
 * shorter (32-layer chain 1.317 ms against 1.350 ms).  Same values, same order of the sum of squares,
 * same bytes. */
struct XUnit {
    XRegs x, t, b;
};

__device__ __forceinline__ void
plan_stage_issue_unit(const OpHead &op, XUnit &xu, uint32_t lane, uint32_t wave)
{
    const uint32_t pro = op.pro;
    if (wave < op.blocks) {
        const float *b = gptr<const float>(op.pro_b);
        const uint32_t at = (wave * 256u + 4u * lane) * 4u;
        xu.x = cload4(coh_buf(gptr<const float>(op.x)), at);
        if (pro == GEMV_PRO_ADD_RMSNORM) xu.t = cload4(coh_buf(gptr<const float>(op.pro_add)), at);
        if (pro == GEMV_PRO_SWIGLU) xu.b = cload4(coh_buf(b), at);
        else if (pro != GEMV_PRO_NONE) xu.b = x_load4(b + wave * 256u + 4u * lane);      /* norm weights: constants */
    }
}

template <int KIND /* 0 Q4_K/Q5_K layout, 1 Q6_K layout */>
__device__ __forceinline__ void
plan_stage_finish_unit(const OpHead &op, const XUnit &xu, uint8_t *base, float *red, bool storer,
                       uint32_t lane, uint32_t wave)
{
    const uint32_t B = op.blocks, pro = op.pro;
    const bool rms = pro == GEMV_PRO_RMSNORM || pro == GEMV_PRO_ADD_RMSNORM, add = pro == GEMV_PRO_ADD_RMSNORM;
    XRegs xr = xu.x;
    if (add) { xr.v0 += xu.t.v0; xr.v1 += xu.t.v1; xr.v2 += xu.t.v2; xr.v3 += xu.t.v3; }
    float inv = 1.0f;
    if (rms) {
        float ss = 0.0f;
        if (wave < B) ss += xr.v0 * xr.v0 + xr.v1 * xr.v1 + xr.v2 * xr.v2 + xr.v3 * xr.v3;
        ss = wave_sum_f32(ss);
        if (lane == 0u) red[wave] = ss;
        __syncthreads();
        const float tot = wave_sum_f32(lane < PLAN_W ? red[lane] : 0.0f);
        inv = 1.0f / sqrtf(tot / (float)(B * 256u) + op.eps);
    }
    if (wave < B) {
        const uint32_t at = (wave * 256u + 4u * lane) * 4u;
        if (add && storer && op.pro_sum_out != 0u) cstore4(coh_buf(gptr<float>(op.pro_sum_out)), at, xr);
        XRegs y = xr;
        if (rms) y = prologue_apply<GEMV_PRO_RMSNORM>(xr, xu.b, inv);
        else if (pro == GEMV_PRO_SWIGLU) y = prologue_apply<GEMV_PRO_SWIGLU>(xr, xu.b, inv);
        if (pro != GEMV_PRO_NONE && storer && op.pro_out != 0u) cstore4(coh_buf(gptr<float>(op.pro_out)), at, y);
        q8k_x_finish<KIND == 1>(y, B, wave, base, (storer && op.act_out) ? gptr<uint8_t>(op.act_out) : nullptr, lane);
    }
}

/* ─── waiting for an operation to be complete on every workgroup ──────── */

/* Counters only grow (modulo 2^32): "reached" is a signed difference. */
__device__ __forceinline__ bool reached(uint32_t v, uint32_t target) { return (int32_t)(v - target) >= 0; }

/* Two ways to learn that every workgroup has announced `target`:
 *
 * copies = 0: workgroup 0 gathers the counters and stores their minimum, the others poll that word.  A
 * store then makes four trips through the fabric before everybody has seen it (the store, workgroup
 * 0's poll, its store of the minimum, the others' poll), but a waiting workgroup reads one line.  The
 * pre-staging kernel's single wait is of this kind: half the workgroups have nothing to stage and poll
 * for microseconds while the others work (with everybody gathering, a decode step took 0.745 ms
 * against 0.732 ms).
 *
 * copies = n: every counter exists n times, 4 KiB apart, a workgroup announces by storing all copies
 * (lanes 0..n-1 of one store instruction) and every workgroup gathers for itself, from copy
 * (workgroup % n): two trips instead of four.  With one copy the 256 pollers of the same sixteen lines
 * are slower than the four trips (32-layer chain 1.47 ms against 1.41 ms); with eight, 32 workgroups
 * share a copy: 1.37 ms (4: 1.38, 16: 1.38, 32: 1.39, 64: 1.40).  The chained kernel's waits are of
 * this kind (OXH_PLAN_COPIES, 0 = the first way). */
#define PLAN_COPIES 64u             /* room for */

__device__ __forceinline__ void plan_announce(const PlanSync &sy, uint32_t value, uint32_t lane)
{
    if (lane < max(sy.copies, 1u)) cstore(sy.flags + lane * PLAN_MAX_WG + blockIdx.x, value);
}

__device__ __forceinline__ bool
plan_wait(const PlanSync &sy, uint32_t target, int *s_ok, uint32_t lane, uint32_t wave)
{
    if (wave == 0u) {
        bool ok = true;
        uint32_t spins = 0;
        if (sy.copies != 0u || blockIdx.x == 0u) {
            const CohBuf fb = coh_buf(sy.flags + (sy.copies ? blockIdx.x % sy.copies : 0u) * PLAN_MAX_WG);
            for (;;) {
                bool mine = true;
                const uint32_t err = cload(sy.go + 1);
                for (uint32_t k = 4u * lane; k < sy.n_wait; k += 256u) {
                    const u32x4 f = cload16(fb, k * 4u);
                    mine = mine && reached(f.x, target) && (k + 1u >= sy.n_wait || reached(f.y, target)) &&
                           (k + 2u >= sy.n_wait || reached(f.z, target)) &&
                           (k + 3u >= sy.n_wait || reached(f.w, target));
                }
                if (__all(mine)) break;
                if (++spins > sy.spin_limit || err != 0u) { ok = false; break; }
            }
            if (lane == 0u) {
                if (!ok) { cstore(sy.go + 1, 1u); cstore(sy.host_err, 1u); }
                else if (sy.copies == 0u) cstore(sy.go, target);
            }
        } else {
            const CohBuf gb = coh_buf(sy.go);
            for (;;) {
                const u32x4 g = cload16(gb, 0u);
                if (reached(g.x, target)) break;
                if (g.y != 0u || ++spins > sy.spin_limit) {
                    ok = false;
                    if (lane == 0u) { cstore(sy.go + 1, 1u); cstore(sy.host_err, 1u); }
                    break;
                }
            }
        }
        if (lane == 0u) *s_ok = ok ? 1 : 0;
    }
    __syncthreads();
    return *s_ok != 0;
}

/* ─── the kernel ──────────────────────────────────────────────────────── */

template <bool HAS_Q5, bool STAMPS = false>
__global__ __launch_bounds__(1024) void
k_plan(const PlanOp *__restrict__ ops, uint32_t n_ops, const PlanSync sy, const PlanLds ld)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    /* the wave index in a scalar register: everything a wave owns (rows, pointers, counts) is then
     * scalar too */
    const uint32_t lane = threadIdx.x & 63u, wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    /* every workgroup's counter holds the same value between launches: the end of the last one */
    const uint32_t base = cload(sy.flags + blockIdx.x);
    float *const outs = reinterpret_cast<float *>(lds + ld.outs_off);
    float *const red = reinterpret_cast<float *>(lds + ld.red_off);
    int *const s_ok = reinterpret_cast<int *>(red + 24);      /* the reduction uses slots 0..15 of 32 */
    float *const terms = reinterpret_cast<float *>(lds + ld.terms_off) + (size_t)wave * ld.terms_per_wave;

    /* The loop is cut between an operation's last pass and its row sums: at that point no load is in
     * flight and no weight or input register holds anything, so nothing but scalars crosses the loop
     * boundary.  One trip = (rows, outputs and announcement of operation i - 1), then requests,
     * staging and passes of operation i. */
    /* the operation table, once, into LDS */
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(ops);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds + ld.table_off);
        const uint32_t n16 = n_ops * (uint32_t)(sizeof(PlanOp) / 16u);
        for (uint32_t k = threadIdx.x; k < n16; k += 1024u) dst[k] = src[k];
    }
    __syncthreads();
    const PlanOp *const tab = reinterpret_cast<const PlanOp *>(lds + ld.table_off);
    PWork cur = plan_work(&tab[0], wave);
    PWork prev = cur;
    OpHead po = plan_head(&tab[0]);
    for (uint32_t i = 0;; i++) {
        /* The lane index, made opaque once per trip: everything derived from it (sub-block masks, LDS
         * slots, byte offsets) is then recomputed per operation in a handful of instructions instead of
         * being kept alive across the whole loop, which costs more registers than this kernel has. */
        uint32_t ln = lane;
        asm volatile("" : "+v"(ln));
        if (i > 0u) {
            /* Rows first, then the workgroup's outputs go out, then (below) the requests for the next
             * operation: those queue up in the memory pipeline (a compute unit takes in about 12 bytes
             * per cycle), and anything placed after them in program order waits for that queue. */
            plan_row_sums(terms, prev, po.blocks, po.term_stride, outs, ln);
            /* a prologue's side outputs (stored while staging, by any wave of one workgroup) have to be
             * acknowledged before the workgroup announces the operation: no load is in flight here, so
             * the wait costs nothing unless such a store is still on its way */
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier();
            plan_stamp<STAMPS>(sy, i - 1u, 6, ln, wave);
            if (wave == 0u) {
                const CohBuf dst = coh_buf(prev.out + prev.wg_row0);
                for (uint32_t r = ln; r < prev.wg_rows; r += 64u) cstore_f32(dst, r * 4u, outs[r]);
                if (po.signal != 0u || i == n_ops) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    /* the last operation leaves every counter at base + n_ops + 1, the next launch's base */
                    plan_announce(sy, base + i + (i == n_ops ? 1u : 0u), ln);
                }
            }
            plan_stamp<STAMPS>(sy, i - 1u, 7, ln, wave);
        }
        if (i == n_ops) break;

        const OpHead op = plan_head(&tab[i]);
        uint8_t *act = lds + (size_t)(i & 1u) * ld.act_bytes;
        plan_stamp<STAMPS>(sy, i, 0, ln, wave);
        /* Loads complete in the order a wave issued them, and the compiler waits for ALL of them
         * before the first use of the input vector (its requests sit in conditional code, which it
         * cannot count past).  So the order of the requests is the schedule: one set of weights first
         * (that is what streams in while a dependency is awaited and the vector is on its way), then
         * the vector; the second set goes out once the vector has been quantised, and streams in
         * during the workgroup barrier and the first pass. */
        WSet A, B;
        A.a = A.b = A.c = A.d = A.e = u32x4{ 0u, 0u, 0u, 0u };
        B.a = B.b = B.c = B.d = B.e = A.a;
        XStage xs;
#pragma unroll
        for (int u = 0; u < 4; u++) xs.x[u] = xs.t[u] = xs.b[u] = XRegs{ 0.f, 0.f, 0.f, 0.f };
        XUnit xu;
        xu.x = xu.t = xu.b = XRegs{ 0.f, 0.f, 0.f, 0.f };
        /* vectors of at most sixteen blocks: a block per wave (plan_stage_issue_unit) */
        const bool by_unit = op.blocks <= PLAN_W;
        /* what this wave owns of the next operation: scalar arithmetic, done while nothing waits for it */
        PWork nx = cur;
        if (i + 1u < n_ops) nx = plan_work(&tab[i + 1u], wave);
        if (op.wait == 0u) {
            /* nothing to wait for: the vector goes first and is there in a microsecond */
            if (by_unit) plan_stage_issue_unit(op, xu, ln, wave);
            else         plan_stage_issue(op, xs, ln, wave);
            plan_prefetch<HAS_Q5>(cur, A, 0u, ln);
        } else {
            /* Wave 0 polls, and a poll comes back behind everything the wave asked for before it: its
             * own weights go out after the wait (behind its part of the vector; they are there before
             * the vector is quantised), the other waves' before it.  (Requesting the second set here as
             * well, which the wait would seem to have time for, measured 1.42 ms against 1.35 ms for the
             * 32-layer chain: the requests compete with the passes the slowest workgroups are still
             * streaming.  Two polls in flight instead of one: 1.37 ms; a pause between polls: 1.34 ms
             * and up against 1.32 ms.) */
            if (wave != 0u) plan_prefetch<HAS_Q5>(cur, A, 0u, ln);
            if (!plan_wait(sy, base + op.wait, s_ok, ln, wave)) return;
            if (by_unit) plan_stage_issue_unit(op, xu, ln, wave);
            else         plan_stage_issue(op, xs, ln, wave);
            if (wave == 0u) plan_prefetch<HAS_Q5>(cur, A, 0u, ln);
        }
        plan_stamp<STAMPS>(sy, i, 1, ln, wave);

        /* a prologue's side outputs are one workgroup's work, and not workgroup 0's: that one gathers the
         * counters, and whatever holds it up holds everybody up */
        const bool storer = blockIdx.x == gridDim.x - 1u;
        const uint32_t Bk = op.blocks;
        if (STAMPS && sy.stamps != nullptr) {         /* measurement only: when has the vector arrived? */
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            plan_stamp<STAMPS>(sy, i, 5, ln, wave);
        }
        if (by_unit) {
            if (op.kind >= PLAN_Q6_K) plan_stage_finish_unit<1>(op, xu, act, red, storer, ln, wave);
            else                      plan_stage_finish_unit<0>(op, xu, act, red, storer, ln, wave);
        } else {
            if (op.kind >= PLAN_Q6_K) plan_stage_finish<1>(op, xs, act, red, storer, ln, wave);
            else                      plan_stage_finish<0>(op, xs, act, red, storer, ln, wave);
        }
        plan_prefetch<HAS_Q5>(cur, B, 1u, ln);
        plan_stamp<STAMPS>(sy, i, 2, ln, wave);
        __syncthreads();
        plan_stamp<STAMPS>(sy, i, 3, ln, wave);

        GemvParams gp;
        gp.blocks = Bk;
        gp.magic = op.magic;
        gp.term_stride = op.term_stride;
        gp.rows_cap = op.rows_cap;
        gp.dump = nullptr;
        if (cur.nblk != 0u) {
            if (cur.kind == PLAN_Q6_K)      plan_passes_q6<false>(A, B, cur, gp, act, q8k6_lds_bytes(Bk), terms, ln);
            else if (cur.kind == PLAN_Q6_KG) plan_passes_q6<true>(A, B, cur, gp, act, q8k6_lds_bytes(Bk), terms, ln);
            else if (HAS_Q5 && cur.kind == PLAN_Q5_K) plan_passes_q45<true>(A, B, cur, gp, act, q8k_lds_bytes(Bk), terms, ln);
            else                            plan_passes_q45<false>(A, B, cur, gp, act, q8k_lds_bytes(Bk), terms, ln);
        }
        plan_stamp<STAMPS>(sy, i, 4, ln, wave);
        prev = cur;
        cur = nx;
        po = op;
    }
}

/* ─── plans whose inputs are all there at launch ─────────────────────── */

/* global -> LDS, 16 bytes per lane, past the L2s (the image was written by another workgroup a moment
 * ago, and this XCD's L2 may still hold the previous launch's bytes at the same address): lane l reads
 * base + off, its bytes land at lds_addr + 16*l.  base and lds_addr are wave-uniform. */
__device__ __forceinline__ void plan_dma16(const uint8_t *base, uint32_t off, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "global_load_lds_dwordx4 %1, %2 sc0 sc1"
                 :: "s"(lds_addr), "v"(off), "s"(base) : "memory");
}

__device__ __forceinline__ uint32_t plan_image_bytes(uint32_t kind, uint32_t blocks)
{
    return kind >= PLAN_Q6_K ? q8k6_lds_bytes(blocks) : q8k_lds_bytes(blocks);
}

/* the staged input of an operation into LDS at byte address lds_addr, 1 KB pieces dealt to the waves */
__device__ __forceinline__ void plan_image_fetch(const PlanOp *op, gaddr xq, uint32_t lds_addr, uint32_t lane, uint32_t wave)
{
    if (xq == 0u) return;                       /* a workgroup without rows in this operation */
    const uint32_t bytes = plan_image_bytes(uni(op->kind), uni(op->blocks));
    const uint8_t *img = gptr<const uint8_t>(xq);
    for (uint32_t k = wave * 1024u; k < bytes; k += PLAN_W * 1024u)
        if (k + 16u * lane < bytes) plan_dma16(img + k, 16u * lane, lds_addr + k);
}

template <bool HAS_Q5, bool STAMPS = false>
__global__ __launch_bounds__(1024) void
k_plan_ext(const PlanOp *__restrict__ ins, uint32_t n_ins, const PlanOp *__restrict__ ops, uint32_t n_ops,
           const PlanSync sy, const PlanLds ld)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const uint32_t lane = threadIdx.x & 63u, wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t base = cload(sy.flags + blockIdx.x);
    float *const red = reinterpret_cast<float *>(lds + ld.red_off);
    int *const s_ok = reinterpret_cast<int *>(red + 24);
    float *const terms_wg = reinterpret_cast<float *>(lds + ld.terms_off);
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(ops);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds + ld.table_off);
        const uint32_t n16 = n_ops * (uint32_t)(sizeof(PlanOp) / 16u);
        for (uint32_t k = threadIdx.x; k < n16; k += 1024u) dst[k] = src[k];
    }
    __syncthreads();
    const PlanOp *const tab = reinterpret_cast<const PlanOp *>(lds + ld.table_off);

    /* Inputs first: workgroup g stages the vectors of operations g, g + grid, ... exactly as the chained
     * kernel stages them (prologue, Q8_K quantisation, the layout the passes read) and stores the LDS
     * image with accesses every XCD sees.  The side outputs of a prologue are written here, once. */
    for (uint32_t j = blockIdx.x; j < n_ins; j += gridDim.x) {
        const OpHead op = plan_head(&ins[j]);
        XStage xs;
#pragma unroll
        for (int u = 0; u < 4; u++) xs.x[u] = xs.t[u] = xs.b[u] = XRegs{ 0.f, 0.f, 0.f, 0.f };
        plan_stage_issue(op, xs, lane, wave);
        if (op.kind >= PLAN_Q6_K) plan_stage_finish<1>(op, xs, lds, red, true, lane, wave);
        else                      plan_stage_finish<0>(op, xs, lds, red, true, lane, wave);
        __syncthreads();
        const uint32_t bytes = plan_image_bytes(op.kind, op.blocks);
        const CohBuf img = coh_buf(gptr<uint8_t>(uni(ins[j].xq)));
        for (uint32_t k = threadIdx.x * 16u; k < bytes; k += 16384u)
            __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(lds + k), img, (int)k, 0,
                                                   OXH_SYSTEM_COHERENT);
        __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x < 64u) plan_announce(sy, base + 1u, threadIdx.x);

    /* One trip = requests for operation i, the workgroup barrier, rows and outputs of operation i - 1
     * (summed from the workgroup's term table by the first wg_rows threads while the other waves go
     * on), then the passes of operation i into the other term table.  The weight registers are free
     * when a trip starts, so the two requested sets are not carried around the loop, and the requests go
     * out before the barrier: the weight stream does not stop at an operation boundary.  The staged
     * input of operation i + 1 is fetched into the other LDS buffer during operation i; the wait at
     * the top of a trip finds it (and the output stores) long complete, and the one barrier of a trip
     * both publishes it to the other waves and says that nobody reads the buffer it replaces. */
    PWork cur = plan_work_flat(&tab[0], wave);
    PWork prev = cur;
    uint32_t p_blocks = 0, p_stride = 0;
    for (uint32_t i = 0;; i++) {
        uint32_t ln = lane;
        asm volatile("" : "+v"(ln));
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        plan_stamp<STAMPS>(sy, i < n_ops ? i : n_ops - 1u, i < n_ops ? 0u : 5u, ln, wave);
        WSet A, B;
        A.a = A.b = A.c = A.d = A.e = u32x4{ 0u, 0u, 0u, 0u };
        B.a = B.b = B.c = B.d = B.e = A.a;
        if (i < n_ops) {
            plan_prefetch<HAS_Q5>(cur, A, 0u, ln);
            plan_prefetch<HAS_Q5>(cur, B, 1u, ln);
        }
        if (i > 0u) {
            /* every wave has finished operation i - 1 and has its pieces of this operation's input */
            lds_barrier();
            plan_stamp<STAMPS>(sy, i - 1u, 6, ln, wave);
            const float *tb = terms_wg + (size_t)((i - 1u) & 1u) * ld.terms_wg;
            const CohBuf dst = coh_buf(prev.out + prev.wg_row0);
            for (uint32_t r = threadIdx.x; r < prev.wg_rows; r += 1024u) {
                float v = row_sum_one<1>(tb + __umul24(r, p_stride), p_blocks);
                if (prev.paired) {
                    const float u = row_sum_one<1>(tb + __umul24(prev.wg_rows + r, p_stride), p_blocks);
                    const float sig = 1.0f / (1.0f + expf(-v));
                    v = v * sig * u;
                }
                cstore_f32(dst, r * 4u, v);
            }
        } else {
            /* every input is staged once every workgroup has said so */
            if (!plan_wait(sy, base + 1u, s_ok, ln, wave)) return;
            plan_image_fetch(&tab[0], cur.xq, lds_base, ln, wave);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
        if (i == n_ops) break;
        PWork nx = cur;
        if (i + 1u < n_ops) {
            nx = plan_work_flat(&tab[i + 1u], wave);
            plan_image_fetch(&tab[i + 1u], nx.xq, lds_base + ((i + 1u) & 1u) * ld.act_bytes, ln, wave);
        }
        plan_stamp<STAMPS>(sy, i, 1, ln, wave);

        const PlanOp *const op = &tab[i];
        const uint32_t Bk = uni(op->blocks);
        const uint8_t *act = lds + (size_t)(i & 1u) * ld.act_bytes;
        GemvParams gp;
        gp.blocks = Bk;
        gp.magic = uni(op->magic);
        gp.term_stride = uni(op->term_stride);
        gp.rows_cap = uni(op->rows_cap);
        gp.dump = nullptr;
        float *const terms = terms_wg + (size_t)(i & 1u) * ld.terms_wg + __umul24(cur.row0, gp.term_stride);
        if (cur.nblk != 0u) {
            if (cur.kind == PLAN_Q6_K)      plan_passes_q6<false>(A, B, cur, gp, act, q8k6_lds_bytes(Bk), terms, ln);
            else if (cur.kind == PLAN_Q6_KG) plan_passes_q6<true>(A, B, cur, gp, act, q8k6_lds_bytes(Bk), terms, ln);
            else if (HAS_Q5 && cur.kind == PLAN_Q5_K) plan_passes_q45<true>(A, B, cur, gp, act, q8k_lds_bytes(Bk), terms, ln);
            else                            plan_passes_q45<false>(A, B, cur, gp, act, q8k_lds_bytes(Bk), terms, ln);
        }
        plan_stamp<STAMPS>(sy, i, 4, ln, wave);
        prev = cur;
        cur = nx;
        p_blocks = Bk;
        p_stride = gp.term_stride;
    }
    /* the next launch's base */
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (threadIdx.x < 64u) plan_announce(sy, base + 2u, threadIdx.x);
}

/* ─── host side ───────────────────────────────────────────────────────── */

struct OxhPlan {
    PlanOp *d_ops;
    uint32_t *d_sync;               /* PLAN_COPIES x PLAN_MAX_WG counters, 4 spare words, then go[4] (go[1]: error word) */
    uint32_t n_ops, grid;
    PlanLds ld;
    size_t lds_bytes;
    uint32_t spin_limit, phantom;
    bool has_q5;
    uint64_t *d_stamps;
    uint32_t n_waits;               /* operations that wait (for callers' curiosity) */
    bool ext;                       /* no operation depends on another: inputs are staged ahead (k_plan_ext) */
    uint8_t *d_img;                 /* the staged inputs */
    PlanOp *d_run;                  /* k_plan_ext: the table it walks (d_ops stays the list of inputs) */
    uint32_t n_run;
    void *multi;                    /* a plan over a 32-value format: the table of GEMV launches (oxh_kernels.hip) */
    uint32_t *h_err;                /* page-locked: set by the kernel when a wait gave up, read before every launch */
};

static const void *plan_kernel(const OxhPlan *pl)
{
    /* with clock stamps attached (plans without Q5_K only): the variants that write them */
    if (pl->d_stamps != nullptr && !pl->has_q5)
        return pl->ext ? reinterpret_cast<const void *>(k_plan_ext<false, true>) : reinterpret_cast<const void *>(k_plan<false, true>);
    if (pl->ext)
        return pl->has_q5 ? reinterpret_cast<const void *>(k_plan_ext<true>) : reinterpret_cast<const void *>(k_plan_ext<false>);
    return pl->has_q5 ? reinterpret_cast<const void *>(k_plan<true>) : reinterpret_cast<const void *>(k_plan<false>);
}

#define PLAN_TRY(call)                                                                      \
    do {                                                                                    \
        hipError_t e_ = (call);                                                             \
        if (e_ != hipSuccess)                                                               \
            return oxh_internal_errorf(OXH_ERR_HIP, "HIP error in %s: %s", #call, hipGetErrorString(e_)); \
    } while (0)

static bool plan_kind(uint32_t qtype, uint32_t *kind)
{
    switch (qtype) {
    case OXH_Q4_K_S: case OXH_Q4_K_M: *kind = PLAN_Q4_K; return true;
    case OXH_Q5_K_S: case OXH_Q5_K_M: *kind = PLAN_Q5_K; return true;
    case OXH_Q6_K:                    *kind = PLAN_Q6_K; return true;
    case OXH_Q6_K_G8:                 *kind = PLAN_Q6_KG; return true;
    default: return false;
    }
}

struct Span { const char *p; size_t n; };
static bool spans_meet(const Span &a, const Span &b)
{
    return a.p && b.p && a.n && b.n && a.p < b.p + b.n && b.p < a.p + a.n;
}

/* Rows of an operation dealt to workgroups: in proportion to the segments' rows (a paired segment
 * counts twice), at most `grid` in all, every wave at most GEMV_ROWS_CAP table rows. */
extern "C" int oxh_plan_deal(const size_t *rows, const int *paired, size_t n_segs, uint32_t grid, uint32_t *n_wg,
                             uint32_t *rows_cap)
{
    size_t total_work = 0;
    for (size_t i = 0; i < n_segs; i++) total_work += rows[i] * (paired[i] ? 2u : 1u);
    if (total_work == 0 || grid == 0) return OXH_ERR_ARG;
    uint32_t cap = 1, sum = 0;
    for (size_t i = 0; i < n_segs; i++) {
        const size_t mult = paired[i] ? 2u : 1u;
        size_t share = ((size_t)grid * rows[i] * mult + total_work / 2) / total_work;
        const size_t hi = (rows[i] + PLAN_W - 1) / PLAN_W;
        if (share > hi) share = hi;
        if (share < 1) share = 1;
        n_wg[i] = (uint32_t)share;
        sum += n_wg[i];
    }
    while (sum > grid) {            /* rounding went over: the largest share gives one back */
        size_t big = 0;
        for (size_t i = 1; i < n_segs; i++) if (n_wg[i] > n_wg[big]) big = i;
        if (n_wg[big] <= 1) return OXH_ERR_TOO_WIDE;
        n_wg[big]--;
        sum--;
    }
    for (size_t i = 0; i < n_segs; i++) {
        const size_t mult = paired[i] ? 2u : 1u;
        const size_t waves = (size_t)n_wg[i] * PLAN_W;
        const size_t rpw = (rows[i] + waves - 1) / waves * mult;
        if (rpw > GEMV_ROWS_CAP) return OXH_ERR_TOO_WIDE;
        if (rpw > cap) cap = (uint32_t)rpw;
    }
    *rows_cap = cap;
    return OXH_OK;
}


struct PlanLimits { uint32_t max_wg_rows, max_wg_terms, max_cap_terms; };

/* Deals the rows of d's segments (rows, w2 filled in) to the grid and notes what the row tables must hold. */
static int plan_deal_op(PlanOp &d, uint32_t grid, PlanLimits &lim)
{
    size_t rows[PLAN_MAX_SEGS];
    int paired[PLAN_MAX_SEGS];
    for (uint32_t k = 0; k < d.n_segs; k++) { rows[k] = d.s[k].rows; paired[k] = d.s[k].w2 != 0u; }
    uint32_t n_wg[PLAN_MAX_SEGS], cap = 1;
    const int drc = oxh_plan_deal(rows, paired, d.n_segs, grid, n_wg, &cap);
    if (drc) return drc;
    d.rows_cap = cap;
    uint32_t wg = 0;
    for (uint32_t k = 0; k < d.n_segs; k++) {
        const size_t waves = (size_t)n_wg[k] * PLAN_W;
        d.s[k].wg_begin = wg;
        d.s[k].rows_q = (uint32_t)(rows[k] / waves);
        d.s[k].rows_rem = (uint32_t)(rows[k] % waves);
        const uint32_t per_wg = (uint32_t)((rows[k] / waves + 1) * PLAN_W);
        if (per_wg > lim.max_wg_rows) lim.max_wg_rows = per_wg;
        const uint32_t flat = per_wg * (paired[k] ? 2u : 1u) * d.term_stride;
        if (flat > lim.max_wg_terms) lim.max_wg_terms = flat;
        wg += n_wg[k];
    }
    d.n_wg = wg;
    if (cap * d.term_stride > lim.max_cap_terms) lim.max_cap_terms = cap * d.term_stride;
    return OXH_OK;
}

/* Operations none of which depends on another may run in any order and grouping.  Operations that read
 * the same weight layout over vectors of the same length may share ONE table row: their segments side
 * by side, each with the staged input of the operation it came from.  What is gained is whole passes:
 * a wave takes sixteen blocks per pass and a workgroup is as slow as its busiest wave, so 40 rows of
 * 16 blocks per workgroup (q/k/v + o of a layer: 2.5 rows per wave) cost three passes, the down
 * projection's 3.5 passes cost four, and every row of the table costs a workgroup barrier.  Rows are
 * filled first-fit (an operation joins the latest earlier row of its shape with room), up to
 * `segs` segments and `passes` passes per wave on average; plan_table_cost prices the result and the
 * caller keeps the cheapest of a few limits.  For a Llama-3-8B decode step the winner is eight passes:
 * gate/up of a layer with o of the next (8.0 passes), q/k/v of two layers (3.0), down of two layers
 * (7.0), all whole: 0.720 ms against 0.743 ms with only q/k/v + o of a layer sharing a row.
 * Writes the rows to `run`, dealt to the grid. */
static int plan_merge(const PlanOp *h, size_t n_ops, uint32_t grid, size_t passes, uint32_t max_segs, bool any_row,
                      PlanOp *run, size_t *n_run, PlanLimits &lim)
{
    const size_t limit = (size_t)grid * PLAN_W * 16u * passes;      /* blocks */
    size_t *work = (size_t *)calloc(n_ops, sizeof *work);
    if (!work) return OXH_ERR_NOMEM;
    size_t n = 0;
    for (size_t i = 0; i < n_ops; i++) {
        size_t more = 0;
        for (uint32_t k = 0; k < h[i].n_segs; k++)
            more += (size_t)h[i].s[k].rows * (h[i].s[k].w2 ? 2u : 1u) * h[i].blocks;
        size_t target = n;
        for (size_t r = n; passes != 0 && r-- > 0;) {
            if (run[r].kind == h[i].kind && run[r].blocks == h[i].blocks &&
                run[r].n_segs + h[i].n_segs <= max_segs && work[r] + more <= limit) {
                target = r;
                break;
            }
            if (!any_row) break;                /* neighbours only */
        }
        if (target == n) {
            run[n] = h[i];
            run[n].n_segs = 0;
            work[n] = 0;
            n++;
        }
        PlanOp &g = run[target];
        for (uint32_t k = 0; k < h[i].n_segs; k++) {
            g.s[g.n_segs] = h[i].s[k];
            g.s[g.n_segs].xq = h[i].xq;
            g.n_segs++;
        }
        work[target] += more;
    }
    free(work);
    for (size_t r = 0; r < n; r++) {
        const int drc = plan_deal_op(run[r], grid, lim);
        if (drc) return drc;
    }
    *n_run = n;
    return OXH_OK;
}

/* Pass slots a dealt table takes: per row the passes of the busiest wave of its busiest workgroup
 * (rows of a pair count twice), plus half a pass for the row's barrier and row sums. */
static double plan_table_cost(const PlanOp *run, size_t n_run)
{
    double cost = 0.0;
    for (size_t r = 0; r < n_run; r++) {
        size_t worst = 0;
        for (uint32_t k = 0; k < run[r].n_segs; k++) {
            const PlanSeg &sg = run[r].s[k];
            const size_t wg_rows = (size_t)sg.rows_q * PLAN_W + (sg.rows_rem < PLAN_W ? sg.rows_rem : PLAN_W);
            const size_t flat = wg_rows * (sg.w2 ? 2u : 1u);
            const size_t per_wave = (flat + PLAN_W - 1) / PLAN_W;
            const size_t p = (per_wave * run[r].blocks + 15u) / 16u;
            if (p > worst) worst = p;
        }
        cost += (double)worst + 0.5;
    }
    return cost;
}

/* Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS (and the aliases): the operations of one such format, none of
 * which touches what another writes, become a table of GEMV launches walked by one grid
 * (k_gemv_multi).  No workgroup waits for another there, so a plan with a dependency is declined. */
/* What one operation of such a plan reads and writes: input rows and their quantised blocks over the
 * activations its segments name (one, except in plans over tile-major Q8_0), and per segment the rows of
 * every activation, out_stride floats apart. */
static size_t multi_acts(const OxhPlanOp &o)
{
    size_t n = 1;
    for (size_t k = 0; k < o.n_segs; k++) {
        const size_t end = o.segs[k].act_first + (o.segs[k].n_vec ? o.segs[k].n_vec : 1u);
        if (o.segs[k].rows && end > n) n = end;
    }
    return n;
}

static Span multi_out_span(const OxhPlanOp &o, size_t k)
{
    const size_t nv = o.segs[k].n_vec ? o.segs[k].n_vec : 1u;
    const Span s = { (const char *)o.segs[k].d_out, ((nv - 1u) * o.out_stride + o.segs[k].rows) * sizeof(float) };
    return s;
}

static int plan_create_multi(const OxhPlanOp *ops, size_t n_ops, OxhPlan **out)
{
    for (size_t i = 0; i < n_ops; i++) {
        const OxhPlanOp &o = ops[i];
        if (!o.segs || o.n_segs == 0 || !o.d_x || o.cols == 0 || o.cols % OXH_QK8_0)
            return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu has no segments, no input or "
                                       "cols not a multiple of 32", i);
        for (size_t k = 0; k < o.n_segs; k++)
            if (o.segs[k].act_first > 0xFFFFFFu || o.segs[k].n_vec > 16u || o.segs[k].rows > 0x3FFFFFFFull ||
                o.out_stride > 0xFFFFFFFFull || o.cols > 0xFFFFFFu)
                return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu: a segment's activations, "
                                           "rows or the output stride are out of range", i);
        const size_t acts_i = multi_acts(o);
        const Span xi = { (const char *)o.d_x, acts_i * o.cols * sizeof(float) };
        const Span ai = { (const char *)o.d_act_out, acts_i * (o.cols / OXH_QK8_0) * 34u };
        for (size_t k = 0; k < o.n_segs; k++) {
            const Span wk = multi_out_span(o, k);
            if (spans_meet(wk, xi) || spans_meet(wk, ai) || spans_meet(ai, xi))
                return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu stores over one of its own inputs", i);
        }
        for (size_t j = 0; j < i; j++) {
            const OxhPlanOp &e = ops[j];
            const size_t acts_j = multi_acts(e);
            const Span xj = { (const char *)e.d_x, acts_j * e.cols * sizeof(float) };
            const Span aj = { (const char *)e.d_act_out, acts_j * (e.cols / OXH_QK8_0) * 34u };
            bool hit = spans_meet(ai, xj) || spans_meet(aj, xi) || spans_meet(ai, aj);
            for (size_t k = 0; k < o.n_segs && !hit; k++) {
                const Span wk = multi_out_span(o, k);
                hit = spans_meet(wk, xj) || spans_meet(wk, aj);
                for (size_t m = 0; m < e.n_segs && !hit; m++) hit = spans_meet(wk, multi_out_span(e, m));
            }
            for (size_t m = 0; m < e.n_segs && !hit; m++) {
                const Span wm = multi_out_span(e, m);
                hit = spans_meet(wm, xi) || spans_meet(wm, ai);
            }
            if (hit)
                return oxh_internal_errorf(OXH_DECLINED, "plan: operation %zu depends on operation %zu; plans over the "
                                           "32-value formats run independent operations only", i, j);
        }
    }
    void *multi = nullptr;
    const int rc = oxh_internal_multi_create(ops, n_ops, &multi);
    if (rc) return rc;
    OxhPlan *pl = (OxhPlan *)calloc(1, sizeof *pl);
    if (!pl) {
        (void)oxh_internal_multi_destroy(multi);
        return oxh_internal_errorf(OXH_ERR_NOMEM, "out of host memory building a plan");
    }
    pl->multi = multi;
    pl->n_ops = (uint32_t)n_ops;
    *out = pl;
    return OXH_OK;
}

extern "C" int oxh_plan_create(const OxhPlanOp *ops, size_t n_ops, OxhPlan **out)
{
    if (!out) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_create: NULL");
    *out = nullptr;
    int rc = oxh_init(oxh_internal_device() >= 0 ? oxh_internal_device() : 0);
    if (rc) return rc;
    if (!ops || n_ops == 0 || n_ops > 0xFFFFu)
        return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_create: 1..65535 operations");
    if (oxh_internal_multi_which(ops[0].qtype) >= 0) return plan_create_multi(ops, n_ops, out);
    const uint32_t n_cu = (uint32_t)(oxh_internal_n_cu() > 0 ? oxh_internal_n_cu() : 256);
    const uint32_t grid = n_cu > PLAN_MAX_WG ? PLAN_MAX_WG : n_cu;

    PlanOp *h = (PlanOp *)calloc(n_ops, sizeof *h);
    Span *reads = (Span *)calloc(n_ops * 4, sizeof *reads), *writes = (Span *)calloc(n_ops * 8, sizeof *writes);
    if (!h || !reads || !writes) {
        free(h); free(reads); free(writes);
        return oxh_internal_errorf(OXH_ERR_NOMEM, "out of host memory building a plan");
    }
    uint32_t max_act = 0, n_waits = 0;
    PlanLimits lim = { 0, 0, 0 };
    size_t img_bytes = 0;
    bool has_q5 = false;
    rc = OXH_OK;
    for (size_t i = 0; i < n_ops && !rc; i++) {
        const OxhPlanOp &o = ops[i];
        PlanOp &d = h[i];
        uint32_t kind;
        if (!plan_kind(o.qtype, &kind) || o.cols == 0 || o.cols % OXH_QK_K || o.cols / OXH_QK_K > PLAN_MAX_BLOCKS ||
            (kind == PLAN_Q6_KG && o.cols % (8u * OXH_QK_K))) {
            rc = oxh_internal_errorf(OXH_DECLINED, "plan: operation %zu (qtype %u, cols %zu) is not one a plan runs: "
                                     "Q4_K, Q5_K or Q6_K with cols a multiple of 256 (2048 for the regrouped Q6_K) up to %u", i, o.qtype, o.cols,
                                     PLAN_MAX_BLOCKS * 256u);
            break;
        }
        if (!o.segs || o.n_segs == 0 || !o.d_x) { rc = oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu has no segments or no input", i); break; }
        d.kind = kind;
        if (kind == PLAN_Q5_K) has_q5 = true;
        d.blocks = (uint32_t)(o.cols / OXH_QK_K);
        d.magic = (uint32_t)((0x100000000ull + d.blocks - 1u) / d.blocks);
        d.term_stride = d.blocks + 1u;
        d.x = (gaddr)(uintptr_t)o.d_x;
        d.act_out = (gaddr)(uintptr_t)o.d_act_out;
        d.pro = GEMV_PRO_NONE;
        if (o.pro) {
            const OxhPrologue &p = *o.pro;
            if ((p.kind != OXH_PRO_RMSNORM && p.kind != OXH_PRO_SWIGLU) || !p.d_b ||
                ((p.d_add || p.d_sum_out) && p.kind != OXH_PRO_RMSNORM) || (p.d_sum_out && !p.d_add) ||
                (p.kind == OXH_PRO_RMSNORM && !(p.eps >= 0.0f))) {
                rc = oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu has a malformed prologue", i);
                break;
            }
            d.pro = p.kind == OXH_PRO_SWIGLU ? GEMV_PRO_SWIGLU : p.d_add ? GEMV_PRO_ADD_RMSNORM : GEMV_PRO_RMSNORM;
            d.eps = p.eps;
            d.pro_b = (gaddr)(uintptr_t)p.d_b;
            d.pro_add = (gaddr)(uintptr_t)p.d_add;
            d.pro_sum_out = (gaddr)(uintptr_t)p.d_sum_out;
            d.pro_out = (gaddr)(uintptr_t)p.d_out;
        }
        /* segments with rows, at most four */
        size_t rows[PLAN_MAX_SEGS];
        int paired[PLAN_MAX_SEGS];
        uint32_t ns = 0;
        for (size_t k = 0; k < o.n_segs; k++) {
            const OxhSegment &sg = o.segs[k];
            if (sg.rows == 0) continue;
            if (ns == PLAN_OP_SEGS || !sg.d_w || !sg.d_out || sg.act_first != 0 || sg.n_vec > 1 ||
                sg.rows > 0x3FFFFFFFull / (d.blocks * 16u)) {
                rc = oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu: at most four non-empty "
                                         "segments, each over activation 0 with one vector", i);
                break;
            }
            d.s[ns].w = (gaddr)(uintptr_t)sg.d_w;
            d.s[ns].w2 = (gaddr)(uintptr_t)sg.d_w_pair;
            d.s[ns].out = (gaddr)(uintptr_t)sg.d_out;
            d.s[ns].rows = (uint32_t)sg.rows;
            rows[ns] = sg.rows;
            paired[ns] = sg.d_w_pair != nullptr;
            ns++;
        }
        if (rc) break;
        if (ns == 0) { rc = oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu has no rows", i); break; }
        d.n_segs = ns;
        const int drc = plan_deal_op(d, grid, lim);
        if (drc) { rc = oxh_internal_errorf(drc, "plan: operation %zu has more rows than %u workgroups can own", i, grid); break; }
        const uint32_t act = kind >= PLAN_Q6_K ? q8k6_lds_bytes(d.blocks) : q8k_lds_bytes(d.blocks);
        if (act > max_act) max_act = act;
        d.xq = (gaddr)img_bytes;                    /* offset for now; the base is added once it exists */
        img_bytes += (act + 255u) & ~(size_t)255u;

        /* what the operation reads and writes, for the dependency scan */
        const size_t xb = o.cols * sizeof(float);
        Span *r = reads + i * 4, *w = writes + i * 8;
        r[0] = Span{ (const char *)o.d_x, xb };
        if (o.pro) {
            r[1] = Span{ (const char *)o.pro->d_b, xb };
            r[2] = Span{ (const char *)o.pro->d_add, xb };
            w[0] = Span{ (const char *)o.pro->d_out, xb };
            w[1] = Span{ (const char *)o.pro->d_sum_out, xb };
        }
        w[2] = Span{ (const char *)o.d_act_out, o.cols / OXH_QK_K * OXH_Q8_K_BYTES };
        for (uint32_t k = 0; k < ns; k++) w[3 + k] = Span{ (const char *)(uintptr_t)d.s[k].out, rows[k] * sizeof(float) };
        /* a result stored by this operation over something it reads itself: every workgroup reads
         * while one stores */
        for (int a = 0; a < 8 && !rc; a++)
            for (int b = 0; b < 4; b++)
                if (spans_meet(w[a], r[b])) {
                    rc = oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan: operation %zu stores over one of its own inputs", i);
                    break;
                }
        /* the latest earlier operation this one must not overtake: one that wrote what this reads or
         * writes, or read what this writes */
        uint32_t wait = 0;
        for (size_t j = i; j-- > 0 && !wait;) {
            const Span *rj = reads + j * 4, *wj = writes + j * 8;
            bool hit = false;
            for (int a = 0; a < 8 && !hit; a++) {
                for (int b = 0; b < 4 && !hit; b++) hit = spans_meet(wj[a], r[b]) || spans_meet(w[a], rj[b]);
                for (int b = 0; b < 8 && !hit; b++) hit = spans_meet(wj[a], w[b]);
            }
            if (hit) wait = (uint32_t)j + 1u;
        }
        d.wait = wait;
        if (wait) { h[wait - 1].signal = 1; n_waits++; }
    }
    free(reads);
    free(writes);
    if (rc) { free(h); return rc; }

    OxhPlan *pl = (OxhPlan *)calloc(1, sizeof *pl);
    if (!pl) { free(h); return oxh_internal_errorf(OXH_ERR_NOMEM, "out of host memory building a plan"); }
    pl->n_ops = (uint32_t)n_ops;
    pl->grid = grid;
    pl->n_waits = n_waits;
    pl->has_q5 = has_q5;
    {
        /* OXH_PLAN_PRESTAGE=0 keeps a plan of independent operations on the chained kernel */
        const char *ps = getenv("OXH_PLAN_PRESTAGE");
        pl->ext = n_waits == 0 && !(ps && ps[0] == '0');
    }
    /* the table the kernel walks: the operations themselves, or (independent operations) short
     * neighbours merged into one row (OXH_PLAN_MERGE=0 keeps them apart) */
    PlanOp *run = nullptr;
    size_t n_run = n_ops;
    if (pl->ext) {
        /* OXH_PLAN_MERGE: 0 every operation in a row of its own; 1 neighbours only, four segments, three
         * passes per wave; 2 (default) any earlier row, eight segments, the cheapest of several pass limits
         * (OXH_PLAN_MERGE_PASSES fixes the limit) */
        const char *pm = getenv("OXH_PLAN_MERGE"), *pp = getenv("OXH_PLAN_MERGE_PASSES");
        const int mode = pm && pm[0] >= '0' && pm[0] <= '2' ? pm[0] - '0' : 2;
        run = (PlanOp *)calloc(n_ops, sizeof *run);
        PlanOp *trial = (PlanOp *)calloc(n_ops, sizeof *trial);
        if (!run || !trial) {
            free(h); free(run); free(trial); free(pl);
            return oxh_internal_errorf(OXH_ERR_NOMEM, "out of host memory building a plan");
        }
        const size_t fixed = pp && *pp ? strtoul(pp, nullptr, 10) : 0;
        const size_t first = mode == 0 ? 0 : mode == 1 ? 3 : fixed ? fixed : 3, last = mode == 2 && !fixed ? 10 : first;
        double best = -1.0;
        PlanLimits best_lim = lim;
        int mrc = OXH_OK;
        for (size_t passes = first; passes <= last; passes++) {
            PlanLimits tl = lim;
            size_t tn = 0;
            const int trc = plan_merge(h, n_ops, grid, passes, mode == 2 ? PLAN_MAX_SEGS : PLAN_OP_SEGS, mode == 2, trial, &tn, tl);
            if (trc) { mrc = trc; continue; }
            const double c = plan_table_cost(trial, tn);
            if (best < 0.0 || c < best) {
                best = c;
                best_lim = tl;
                n_run = tn;
                memcpy(run, trial, tn * sizeof *run);
            }
        }
        free(trial);
        if (best < 0.0) {
            free(h); free(run); free(pl);
            return oxh_internal_errorf(mrc, "plan: merged operations have more rows than %u workgroups can own", grid);
        }
        lim = best_lim;
    }
    pl->n_run = (uint32_t)n_run;
    pl->ld.act_bytes = (max_act + 15u) & ~15u;
    pl->ld.outs_off = 2u * pl->ld.act_bytes;
    pl->ld.red_off = pl->ld.outs_off + ((lim.max_wg_rows * 4u + 15u) & ~15u);
    pl->ld.terms_off = pl->ld.red_off + 128u;
    pl->ld.terms_per_wave = lim.max_cap_terms;
    pl->ld.terms_wg = (lim.max_wg_terms + 3u) & ~3u;
    pl->ld.table_off = (pl->ld.terms_off + (pl->ext ? 2u * pl->ld.terms_wg : PLAN_W * lim.max_cap_terms) * 4u + 15u) & ~15u;
    pl->lds_bytes = (size_t)pl->ld.table_off + n_run * sizeof(PlanOp);
    const char *sl = getenv("OXH_PLAN_SPIN_LIMIT");
    pl->spin_limit = sl && *sl ? (uint32_t)strtoul(sl, nullptr, 10) : 4000000u;
    if (pl->lds_bytes > 160u * 1024u) {
        free(h); free(run); free(pl);
        return oxh_internal_errorf(OXH_ERR_TOO_WIDE, "plan: the staged activation, the row tables and the table of %zu operations (%zu bytes each) do not fit 160 KiB of LDS; split the chain into several plans", n_ops, sizeof(PlanOp));
    }
    const void *kernel = plan_kernel(pl);
    {
        hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) { free(h); free(run); free(pl); return oxh_internal_errorf(OXH_ERR_HIP, "HIP error in hipFuncSetAttribute: %s", hipGetErrorString(e)); }
    }
    /* every workgroup must be resident at once: one per compute unit fits by construction when the
     * device can hold one workgroup of this kernel per unit */
    int per_cu = 0;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 1024, pl->lds_bytes);
    if (e != hipSuccess || per_cu < 1) {
        free(h); free(run); free(pl);
        return oxh_internal_errorf(OXH_ERR_HIP, "plan: the device cannot hold one workgroup of the plan kernel per compute unit");
    }
    e = hipMalloc((void **)&pl->d_ops, n_ops * sizeof(PlanOp));
    if (e == hipSuccess && pl->ext) e = hipMalloc((void **)&pl->d_img, img_bytes);
    if (e == hipSuccess && pl->ext) e = hipMalloc((void **)&pl->d_run, n_run * sizeof(PlanOp));
    /* the staged inputs' offsets become addresses */
    for (size_t i = 0; i < n_ops; i++) h[i].xq = pl->ext ? (gaddr)(uintptr_t)pl->d_img + h[i].xq : 0u;
    /* the chained kernel reads its deal of rows to workgroups from the segments' xq (plan_work) */
    for (size_t i = 0; !pl->ext && i < n_ops; i++)
        for (uint32_t k = 0; k < h[i].n_segs; k++) {
            const uint32_t seg_wgs = (k + 1u < h[i].n_segs ? h[i].s[k + 1u].wg_begin : h[i].n_wg) - h[i].s[k].wg_begin;
            h[i].s[k].xq = seg_wgs ? (gaddr)(h[i].s[k].rows / seg_wgs) | ((gaddr)(h[i].s[k].rows % seg_wgs) << 32) : 0u;
        }
    for (size_t i = 0; run && i < n_run; i++)
        for (uint32_t k = 0; k < run[i].n_segs; k++) run[i].s[k].xq += (gaddr)(uintptr_t)pl->d_img;
    if (e == hipSuccess) e = hipMalloc((void **)&pl->d_sync, (PLAN_COPIES * PLAN_MAX_WG + 8u) * sizeof(uint32_t));
    if (e == hipSuccess) e = hipHostMalloc((void **)&pl->h_err, 64, hipHostMallocDefault);
    if (e == hipSuccess) *pl->h_err = 0u;
    if (e == hipSuccess) e = hipMemcpy(pl->d_ops, h, n_ops * sizeof(PlanOp), hipMemcpyHostToDevice);
    if (e == hipSuccess && pl->ext) e = hipMemcpy(pl->d_run, run, n_run * sizeof(PlanOp), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemset(pl->d_sync, 0, (PLAN_COPIES * PLAN_MAX_WG + 8u) * sizeof(uint32_t));
    if (e == hipSuccess) e = hipDeviceSynchronize();
    free(h);
    free(run);
    if (e != hipSuccess) {
        if (pl->d_ops) (void)hipFree(pl->d_ops);
        if (pl->d_run) (void)hipFree(pl->d_run);
        if (pl->d_img) (void)hipFree(pl->d_img);
        if (pl->d_sync) (void)hipFree(pl->d_sync);
        if (pl->h_err) (void)hipHostFree(pl->h_err);
        free(pl);
        return oxh_internal_errorf(e == hipErrorOutOfMemory ? OXH_ERR_NOMEM : OXH_ERR_HIP, "plan: %s", hipGetErrorString(e));
    }
    *out = pl;
    return OXH_OK;
}

extern "C" int oxh_plan_launch(OxhPlan *pl, void *stream)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_launch: NULL plan");
    if (pl->multi) return oxh_internal_multi_launch(pl->multi, stream);
    /* A launch in which a wait gave up leaves the counters unequal: every later launch would leave at its
     * first wait with incomplete outputs.  The kernel notes it in a host word; from then on launches
     * are refused until oxh_plan_status has reported the failure and reset the plan.  (A launch already
     * queued behind the failing one cannot be recalled; oxh_plan_status after it reports the same.) */
    if (*(volatile uint32_t *)pl->h_err != 0u)
        return oxh_internal_errorf(OXH_ERR_TIMEOUT, "plan: an earlier launch gave up at a wait between operations; "
                                   "call oxh_plan_status to reset the plan before launching it again");
    hipStream_t st = stream ? (hipStream_t)stream : (hipStream_t)oxh_internal_stream();
    PlanSync sy;
    sy.flags = pl->d_sync;
    sy.go = pl->d_sync + PLAN_COPIES * PLAN_MAX_WG + 4u;
    sy.n_wait = pl->grid + pl->phantom;
    {
        static int copies = -1;
        if (copies < 0) {
            const char *pc = getenv("OXH_PLAN_COPIES");
            const unsigned long v = pc && *pc ? strtoul(pc, nullptr, 10) : 8ul;
            copies = v > PLAN_COPIES ? (int)PLAN_COPIES : (int)v;
        }
        sy.copies = pl->ext ? 0u : (uint32_t)copies;
    }
    sy.spin_limit = pl->spin_limit;
    sy.stamps = pl->d_stamps;
    sy.host_err = pl->h_err;
#define PLAN_LAUNCH(K)                                                                                  \
    hipLaunchKernelGGL(K, dim3(pl->grid), dim3(1024), pl->lds_bytes, st, (const PlanOp *)pl->d_ops,    \
                       pl->n_ops, sy, pl->ld)
#define PLAN_LAUNCH_EXT(K)                                                                              \
    hipLaunchKernelGGL(K, dim3(pl->grid), dim3(1024), pl->lds_bytes, st, (const PlanOp *)pl->d_ops,    \
                       pl->n_ops, (const PlanOp *)pl->d_run, pl->n_run, sy, pl->ld)
    const bool stamped = pl->d_stamps != nullptr && !pl->has_q5;     /* as plan_kernel() */
    if (pl->ext) {
        if (stamped)         PLAN_LAUNCH_EXT((k_plan_ext<false, true>));
        else if (pl->has_q5) PLAN_LAUNCH_EXT(k_plan_ext<true>);
        else                 PLAN_LAUNCH_EXT(k_plan_ext<false>);
    } else {
        if (stamped)         PLAN_LAUNCH((k_plan<false, true>));
        else if (pl->has_q5) PLAN_LAUNCH(k_plan<true>);
        else                 PLAN_LAUNCH(k_plan<false>);
    }
#undef PLAN_LAUNCH
#undef PLAN_LAUNCH_EXT
    PLAN_TRY(hipGetLastError());
    return OXH_OK;
}

extern "C" int oxh_plan_info(const OxhPlan *pl, size_t *n_ops, size_t *n_waits, size_t *workgroups, size_t *lds_bytes)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_info: NULL plan");
    if (n_ops) *n_ops = pl->n_ops;
    if (n_waits) *n_waits = pl->n_waits;
    if (workgroups) *workgroups = pl->grid;
    if (lds_bytes) *lds_bytes = pl->lds_bytes;
    if (pl->multi) oxh_internal_multi_info(pl->multi, nullptr, workgroups, lds_bytes);
    return OXH_OK;
}

extern "C" int oxh_plan_table_rows(const OxhPlan *pl)
{
    if (!pl) return -1;
    if (pl->multi) {
        size_t items = 0;
        oxh_internal_multi_info(pl->multi, &items, nullptr, nullptr);
        return (int)items;
    }
    return (int)pl->n_run;
}

extern "C" int oxh_plan_prestaged(const OxhPlan *pl)
{
    return pl && pl->ext ? 1 : 0;
}

extern "C" int oxh_plan_set_spin_limit(OxhPlan *pl, uint32_t polls)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_set_spin_limit: NULL plan");
    pl->spin_limit = polls;
    return OXH_OK;
}

extern "C" int oxh_debug_plan_phantom(OxhPlan *pl, int on)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: plan_phantom: NULL plan");
    pl->phantom = on ? 1u : 0u;
    return OXH_OK;
}

extern "C" int oxh_debug_plan_stamps(OxhPlan *pl, uint64_t *d_stamps)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_debug_plan_stamps: NULL plan");
    pl->d_stamps = d_stamps;
    PLAN_TRY(hipFuncSetAttribute(plan_kernel(pl), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    return OXH_OK;
}

extern "C" int oxh_plan_status(OxhPlan *pl, void *stream)
{
    if (!pl) return oxh_internal_errorf(OXH_ERR_ARG, "invalid argument: oxh_plan_status: NULL plan");
    hipStream_t st = stream ? (hipStream_t)stream : (hipStream_t)oxh_internal_stream();
    PLAN_TRY(hipStreamSynchronize(st));
    if (pl->multi) return OXH_OK;              /* nothing waits in such a plan */
    uint32_t go[4] = { 0, 0, 0, 0 };
    PLAN_TRY(hipMemcpy(go, pl->d_sync + PLAN_COPIES * PLAN_MAX_WG + 4u, sizeof go, hipMemcpyDeviceToHost));
    if (go[1] == 0u) return OXH_OK;
    /* a wait ran out: the counters are no longer equal, start them afresh */
    PLAN_TRY(hipMemset(pl->d_sync, 0, (PLAN_COPIES * PLAN_MAX_WG + 8u) * sizeof(uint32_t)));
    PLAN_TRY(hipDeviceSynchronize());
    *(volatile uint32_t *)pl->h_err = 0u;
    return oxh_internal_errorf(OXH_ERR_TIMEOUT, "plan: a wait between operations ran out of polls (not every workgroup "
                               "was resident, or the limit is too small); the launch's outputs are incomplete");
}

extern "C" int oxh_plan_destroy(OxhPlan *pl)
{
    if (!pl) return OXH_OK;
    hipError_t e = hipDeviceSynchronize();
    if (pl->multi) (void)oxh_internal_multi_destroy(pl->multi);
    if (pl->d_ops) (void)hipFree(pl->d_ops);
    if (pl->d_run) (void)hipFree(pl->d_run);
    if (pl->d_img) (void)hipFree(pl->d_img);
    if (pl->d_sync) (void)hipFree(pl->d_sync);
    if (pl->h_err) (void)hipHostFree(pl->h_err);
    free(pl);
    if (e != hipSuccess) return oxh_internal_errorf(OXH_ERR_HIP, "HIP error in hipDeviceSynchronize: %s", hipGetErrorString(e));
    return OXH_OK;
}
