/*
 * oxhip.h — C ABI of liboxhip: MI355X (gfx950) quantized matvec / matmul.
 *
 * Two layers, both plain C (pointers and sizes only):
 *
 *   1. Drop-in host API — same argument lists as the reference's
 *      oxidize-c/include/oxidize/matvec.h.  Host pointers in, host pointers
 *      out; weights are uploaded once (explicitly via oxh_weight_register or
 *      on first sight) and stay resident in HBM.  The oxh_matvec_* functions
 *      return a status; the oc_matvec_* symbols are the reference's own names
 *      and signatures (void) layered on top of them.
 *
 *   2. Device-resident API — asynchronous launches on a caller stream over
 *      device pointers, modelled on the reference's device ABI
 *      (oxidize-c/include/oxidize/cuda_mmq.h:17-20, :57-72, :128-143).
 *
 * There is no CPU fallback anywhere in this library.  A shape the reference's
 * integer path declines (oxidize-c/src/compute/matvec.c:99-127, :961-985)
 * yields OXH_DECLINED so the caller can run its own CPU code; every other
 * failure is an error code plus a message retrievable with oxh_last_error().
 */
#ifndef OXHIP_H
#define OXHIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ─── status ──────────────────────────────────────────────────────────── */

#define OXH_OK            0
#define OXH_DECLINED      1   /* not an integer-path shape/type; nothing was written */
#define OXH_ERR_HIP      (-1) /* a HIP runtime call failed                   */
#define OXH_ERR_ARG      (-2) /* NULL pointer / overflow / bad size          */
#define OXH_ERR_NO_DEVICE (-3)
#define OXH_ERR_TOO_WIDE (-4) /* cols beyond what one workgroup can stage    */
#define OXH_ERR_NOMEM    (-5)
#define OXH_ERR_FORMAT   (-6) /* a model file is malformed or truncated       */
#define OXH_ERR_IO       (-7) /* a model file could not be opened or mapped   */
#define OXH_ERR_TIMEOUT  (-8) /* a bounded wait inside a plan launch ran out  */

/* GGUF quantization type ids handled here; values are ABI
 * (oxidize-c/include/oxidize/quant.h:94-110). */
#define OXH_Q4_0    3u
#define OXH_Q4_1    4u
#define OXH_Q5_0    5u
#define OXH_Q5_1    6u
#define OXH_Q8_0    7u
#define OXH_Q2_K    8u
#define OXH_Q3_K_S  9u     /* ids 9, 10, 11: one Q3_K block layout */
#define OXH_Q3_K_M 10u
#define OXH_Q3_K_L 11u
#define OXH_Q4_K_S 12u
#define OXH_Q4_K_M 13u
#define OXH_Q5_K_S 14u
#define OXH_Q5_K_M 15u
#define OXH_Q6_K   16u
#define OXH_AL5    17u     /* the Q4_0 block layout under its own id (quantization.c:207-214) */
#define OXH_AL5_XS 18u     /* f16 d + thirty-two 3-bit codes (oxk.h:55) */
#define OXH_AL6    19u     /* the Q5_0 layout */
#define OXH_AL8    20u     /* the Q8_0 layout */
#define OXH_IQ3_S  25u     /* codebook format, 3.44 bits per weight (oxk.h:63) */
#define OXH_IQ1_XXXS 36u   /* codebook format, 1.19 bits per weight (quant.h:79) */
/* The two 4-bit codebook formats of the reference's DEQUANTISE path (quant.h:122-123): its CPU API has
 * no integer dot for them, a row is expanded to f32 and dotted with the f32 input (matvec.c:799-831).
 * Here: oxh_gemv_segments_f32 (f32 inputs used as they are, no quantised activations), oxh_get_rows,
 * and, opt-in, the host entry points (OXH_F32_PATH_TYPES=1; declined otherwise, like every other type
 * of that path). */
#define OXH_IQ4_NL 26u     /* 18-byte blocks of 32: f16 d + 16 nibble bytes          */
#define OXH_IQ4_XS 27u     /* 136-byte blocks of 256: f16 d, 8 six-bit scales, nibbles */
#define OXH_QTYPE_UNKNOWN 0xffffffffu

/* Block geometry (oxidize-c/include/oxidize/oxk.h:46-66). */
#define OXH_QK_K         256u
#define OXH_QK8_0         32u
#define OXH_Q4_K_BYTES   144u
#define OXH_Q5_K_BYTES   176u
#define OXH_Q6_K_BYTES   210u
#define OXH_AL5_XS_BYTES  14u
#define OXH_Q2_K_BYTES    84u
#define OXH_Q3_K_BYTES   110u
#define OXH_Q8_0_BYTES    34u
#define OXH_Q4_0_BYTES    18u
#define OXH_Q4_1_BYTES    20u
#define OXH_Q5_0_BYTES    22u
#define OXH_Q5_1_BYTES    24u
#define OXH_Q8_K_BYTES   292u
#define OXH_IQ3_S_BYTES  110u
#define OXH_IQ1_XXXS_BYTES 38u
#define OXH_IQ4_NL_BYTES 18u
#define OXH_IQ4_XS_BYTES 136u

/* Thread-local text of the last failure on this thread ("" if none). */
const char *oxh_last_error(void);

/* ─── layer 2: device-resident, stream-ordered ────────────────────────── */

/* Select the device and create the library's internal stream.  Idempotent.
 * Replaces oc_cuda_init's device selection (oxidize-c/src/backends/cuda.cu:633). */
int oxh_init(int device);
void oxh_shutdown(void);

/* 0 = declined, 1 = pairs with Q8_0 activations, 2 = pairs with Q8_K.
 * Replaces fused_act_kind (oxidize-c/src/compute/matvec.c:99-127) and
 * oc_cuda_mmq_supported (oxidize-c/include/oxidize/cuda_mmq.h:38-42). */
int oxh_act_kind(uint32_t qtype, size_t cols);
/* Packed row size for (qtype, cols), 0 if declined.  Replaces
 * oc_cuda_mmq_row_bytes (cuda_mmq.h:44-48); no padding is ever added, the
 * device layout is the on-disk layout. */
size_t oxh_row_bytes(uint32_t qtype, size_t cols);
/* Row bytes of a type this library runs through f32 inputs instead of an integer dot (OXH_IQ4_NL,
 * OXH_IQ4_XS; cols a whole number of blocks), 0 for every other type or width.  oxh_act_kind and
 * oxh_row_bytes stay 0 for these, as the reference's integer path declines them
 * (oxidize-c/src/compute/matvec.c:99-127). */
size_t oxh_f32_path_row_bytes(uint32_t qtype, size_t cols);
/* Bytes of one quantised activation vector of `cols` values for `qtype`. */
size_t oxh_act_bytes(uint32_t qtype, size_t cols);

/* Activation quantisers.  d_x: n_vec vectors of `cols` floats, `in_stride`
 * floats apart.  d_act: n_vec activations back to back, each in the exact
 * byte format of the reference: Q8_K [f32 d][256 i8][16 i16 sums] per 256
 * values (oxidize-c/src/compute/matvec.c:276-316), Q8_0 [f16 d][32 i8] per 32
 * (matvec.c:130-155).  Replaces oc_cuda_mmq_quantize_x (cuda_mmq.h:128-132). */
int oxh_quantize_q8_k(const float *d_x, size_t in_stride, size_t n_vec,
                      size_t cols, void *d_act, void *stream);
int oxh_quantize_q8_0(const float *d_x, size_t in_stride, size_t n_vec,
                      size_t cols, void *d_act, void *stream);

/* One weight matrix (or expert slice) of a grouped launch. */
typedef struct OxhSegment {
    const void *d_w;      /* packed rows, row stride = oxh_row_bytes()        */
    float      *d_out;    /* output vector 0; vector v at d_out + v*out_stride */
    size_t      rows;
    size_t      act_first;/* index of this segment's first activation in d_acts */
    size_t      n_vec;    /* activations of this segment (1..8); 0 = the launch's n_vec */
    const void *d_w_pair; /* NULL, or a second matrix of the same type and shape: the
                             segment then writes silu(dot(W[r], a)) * dot(W_pair[r], a) */
} OxhSegment;

/* A segment with d_w_pair set computes the gate and up projections of a
 * SwiGLU feed-forward block in one pass and writes only their combination
 * h[r] = silu(gate[r]) * up[r] (f32, the expression of
 * oxidize-c/src/compute/activation.c:92-99 / k_f_swiglu,
 * oxidize-c/src/backends/cuda_fast.cu:477-485): every wave walks its rows of
 * both matrices, so no gate / up vector ever reaches memory.  Paired
 * launches always use the dot-instruction kernels (n_vec <= 8). */

/* Decode GEMV over pre-quantised activations:
 *   out[v][r] = dot(W[r], act[act_first + v])   for v < n_vec (1..8)
 * for every segment, in ONE launch (a segment may override n_vec with its own
 * count: expert e of an MoE layer takes only the m_e tokens routed to it,
 * llama.c:6151-6169).  Covers the reference's row kernels
 * oc_oxk_dot_rows_{q4_k,q5_k,q6_k}_q8_k / _q8_0_q8_0 (oxidize-c/src/compute/oxk.c:
 * 1447-1488) as used by matvec_fused_slice, matvec_fused_multi_slice and
 * matvec_fused_multi_input_slice (matvec.c:640-797) and the small-batch
 * rows path (matvec.c:1079-1102); the device analogue is
 * oc_cuda_mmq_matvec / _matvec_expert (cuda_mmq.h:57-72).  Segments live in
 * HOST memory and are copied into the launch; a launch takes 32 of them, a
 * call with more runs as launches of 32 (over f32 inputs: quantised once for
 * all, which needs d_act_out; no prologue then). */
int oxh_gemv_segments(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                      size_t cols, const void *d_acts, size_t n_vec,
                      size_t out_stride, void *stream);

/* Same launch with the activation quantisation fused into the kernel: d_x
 * holds the f32 input vectors (`x_stride` floats apart, indexed like d_acts),
 * every workgroup quantises the vectors of its segment straight into LDS —
 * one kernel per decode matmul instead of two, which is what
 * oc_matvec_quantized does in one call (matvec.c:860-881).  When d_act_out is
 * not NULL the quantised bytes are also stored there (reference format,
 * oxh_act_bytes() per vector, indexed like d_x; room for every vector up to
 * the largest act_first + n_vec of any segment), and launches of several
 * vectors per weight may then run on the matrix cores (Q4_K, Q5_K, Q6_K from
 * three vectors, the 32-value formats from five), which also lifts the limit
 * on n_vec from 8 to 16. */
int oxh_gemv_segments_f32(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                          size_t cols, const float *d_x, size_t x_stride,
                          void *d_act_out, size_t n_vec, size_t out_stride,
                          void *stream);

/* The same launch with one more step fused in front of the quantiser, so that
 * a decode layer needs no stand-alone normalisation or activation kernel and
 * no f32 round trip between its matmuls:
 *   OXH_PRO_RMSNORM  quantises x[i] * inv_rms * d_b[i] with
 *                    inv_rms = 1/sqrt(mean(x^2) + eps); d_b = the norm weight,
 *                    cols floats shared by all vectors.  Replaces
 *                    oc_rms_norm_f32 (oxidize-c/src/compute/activation.c:16-22)
 *                    / k_f_rmsnorm (oxidize-c/src/backends/cuda_fast.cu:155-168)
 *                    followed by the matvec.  With d_add != NULL the
 *                    vector normalised is x + d_add (laid out like d_x) and,
 *                    when d_sum_out != NULL, that sum is stored there: the
 *                    residual update and the next norm in one step
 *                    (k_f_residual_rms, cuda_fast.cu:171-189).
 *   OXH_PRO_SWIGLU   quantises silu(x[i]) * d_b[v][i]; x = the gate vectors,
 *                    d_b = the up vectors laid out like d_x.  Replaces
 *                    oc_swiglu_inplace_f32 (activation.c:92-99) / k_f_swiglu
 *                    (cuda_fast.cu:477-485) followed by the down projection.
 * d_out (optional, laid out like d_x) receives the f32 result of the
 * prologue.  No stored result may overlap an input or the other stored
 * result: every workgroup reads the inputs while one per segment stores.  pro == NULL is oxh_gemv_segments_f32.
 * These are float operations: the normalised / activated values agree with
 * the reference's to rounding (its own SIMD variants differ from one another
 * in summation order), and everything after them, quantised bytes included,
 * is the exact integer path applied to those values.  Launches with a
 * prologue always use the dot-instruction kernels (n_vec <= 8). */
#define OXH_PRO_RMSNORM 1u
#define OXH_PRO_SWIGLU  2u
typedef struct OxhPrologue {
    uint32_t     kind;
    float        eps;     /* RMSNORM */
    const float *d_b;
    float       *d_out;
    const float *d_add;     /* RMSNORM only, optional */
    float       *d_sum_out; /* RMSNORM with d_add only, optional */
} OxhPrologue;
int oxh_gemv_segments_fused(uint32_t qtype, const OxhSegment *segs, size_t n_segs,
                            size_t cols, const float *d_x, size_t x_stride,
                            const OxhPrologue *pro, void *d_act_out, size_t n_vec,
                            size_t out_stride, void *stream);

/* A chain of decode matmuls as ONE launch.  The reference's device path
 * submits the whole token chain and replays it at about one launch per token
 * (oxidize-c/include/oxidize/cuda.h:250-265, cuda_fast.cu); here the chain is
 * compiled into a table in device memory and walked by one persistent kernel
 * (a 16-wave workgroup per compute unit), which takes the launch gap, the
 * argument fetch and the cold start of the weight stream out of every matmul:
 * a wave requests the next operation's first weights before it has summed the
 * rows of the current one.
 *
 * An operation is what one oxh_gemv_segments_fused call describes: up to four
 * non-empty segments (each over activation 0, one vector; d_w_pair allowed),
 * the f32 input, an optional prologue, an optional store of the quantised
 * bytes.  Types: Q4_K, Q5_K, Q6_K; cols a multiple of 256 up to 16384 (the
 * 32-value formats: see below).  Anything else makes oxh_plan_create return
 * OXH_DECLINED (launch those matmuls one by one).  Results are bit-identical to the same calls made one
 * after the other.
 *
 * Dependencies are found from the addresses: an operation that reads or
 * overwrites what an earlier operation wrote (or overwrites what it read)
 * waits until every workgroup has finished that earlier one; operations
 * without such a conflict run back to back without waiting.  Buffers that
 * pass between operations may be ordinary oxh_malloc memory.  An operation
 * must not store a result over one of its own inputs.
 *
 * A plan in which NO operation conflicts with an earlier one (every input is
 * there when the launch starts) stages its inputs ahead of the chain: each
 * vector is normalised and quantised once, by one workgroup, into device
 * memory the plan owns (about 1.3 bytes per input value), all workgroups meet
 * once, and from then on an operation's quantised input is copied into LDS
 * while the previous operation runs.  The operations of such a plan may run
 * in any order and grouping: those that read one weight layout over vectors
 * of one length are walked as one table row with several inputs while the row
 * stays within eight segments and eight passes per wave (q/k/v and o of two
 * layers: five rows per wave where one layer's are 2.5, i.e. three passes for
 * half the waves and two for the rest; the down projections of two layers).
 * Same results; oxh_plan_prestaged says whether a plan runs this way and
 * oxh_plan_table_rows how many rows it walks (at creation, in the
 * environment: OXH_PLAN_PRESTAGE=0 keeps such a plan on the chained kernel,
 * OXH_PLAN_MERGE=0 keeps every operation on its own, OXH_PLAN_MERGE=1 merges
 * neighbours only, within four segments and three passes per wave).
 *
 * Plans over the 32-value formats: when the first operation's type is Q8_0,
 * Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS or one of their aliases, every operation must
 * be of that same type (cols a multiple of 32), without prologue and unpaired,
 * any number of segments, and NO operation may touch what another writes
 * (OXH_DECLINED otherwise: nothing waits in such a launch).  The rows of all
 * operations are cut into runs and dealt to the workgroups so that each streams
 * the same number of bytes; a workgroup walks its runs with the GEMV kernel's
 * own steps.  Same bits as the calls one by one.  oxh_plan_table_rows gives
 * the number of runs; nothing of the residency rule below applies.
 *
 * Plans over tile-major Q8_0 (OXH_Q8_0_T16, see oxh_tile16): every operation
 * of that form (cols a multiple of 128), independent of each other as above,
 * without prologue and unpaired; a segment may carry up to sixteen activations
 * (its n_vec, from row act_first of d_x on, the rows cols floats apart; d_act_out,
 * when given, receives the Q8_0 blocks of the same rows), activation v's rows
 * going out_stride floats after activation v - 1's.  The matrices are cut into
 * runs of whole 16-row groups and dealt so that every workgroup streams the
 * same amount; same bits as oxh_gemv_segments_f32 segment by segment.  (The
 * independence check takes a segment's outputs as one span from its first
 * activation's first row to its last one's last row: outputs of different
 * operations interleaved in one buffer are declined.)  This
 * is how many small matrices are batched: a Qwen2.5-0.5B-shaped step of 97
 * matmuls at eight activations each is one launch.
 *
 * All workgroups must be resident together (one per compute unit; the kernel
 * needs the whole device, so do not run other kernels beside a plan launch).
 * Every wait is bounded: after `polls` unsuccessful polls (about a microsecond
 * each; default 4 000 000, OXH_PLAN_SPIN_LIMIT) the launch gives up, every
 * workgroup leaves, and oxh_plan_status reports OXH_ERR_TIMEOUT.  A plan keeps
 * progress counters in device memory between launches: launches of one plan
 * must not overlap (one stream, or ordered by events); a graph may replay it. */
typedef struct OxhPlanOp {
    uint32_t           qtype;
    const OxhSegment  *segs;
    size_t             n_segs;
    size_t             cols;
    const float       *d_x;
    const OxhPrologue *pro;         /* NULL: quantise d_x as it is */
    void              *d_act_out;   /* NULL, or where the quantised bytes are also stored */
    size_t             out_stride;  /* floats from one activation's outputs to the next one's (tile-major
                                       plans with several activations per segment); otherwise unused, 0 */
} OxhPlanOp;
typedef struct OxhPlan OxhPlan;
int oxh_plan_create(const OxhPlanOp *ops, size_t n_ops, OxhPlan **plan);
int oxh_plan_launch(OxhPlan *plan, void *stream);
/* Waits for `stream`, then OXH_OK, or OXH_ERR_TIMEOUT when a launch since the
 * last call gave up (the plan is reset and may be launched again). */
int oxh_plan_status(OxhPlan *plan, void *stream);
/* Operations, how many of them wait for an earlier one, workgroups, LDS bytes
 * per workgroup.  Any pointer may be NULL. */
int oxh_plan_info(const OxhPlan *plan, size_t *n_ops, size_t *n_waits, size_t *workgroups, size_t *lds_bytes);
/* 1 when the plan stages its inputs ahead of the chain (see above), else 0. */
int oxh_plan_prestaged(const OxhPlan *plan);
/* Rows of the table a launch walks: the operations, or fewer where independent
 * operations share rows.  Negative for a NULL plan. */
int oxh_plan_table_rows(const OxhPlan *plan);
/* The poll limit of every wait (default 4 000 000, or OXH_PLAN_SPIN_LIMIT). */
int oxh_plan_set_spin_limit(OxhPlan *plan, uint32_t polls);
int oxh_plan_destroy(OxhPlan *plan);
/* How a plan deals the rows of one operation's segments to `grid` workgroups of
 * sixteen waves (pure host arithmetic): workgroups per segment and the most
 * table rows any wave owns (a paired segment counts two per row). */
int oxh_plan_deal(const size_t *rows, const int *paired, size_t n_segs, uint32_t grid, uint32_t *n_wg,
                  uint32_t *rows_cap);

/* Prefill matmul on int8 MFMA: out[v*out_stride + r] = dot(W[r], act[v]) for
 * v < n_vec (any count), Q8_K activations, Q4_K / Q5_K / Q6_K weights.
 * Replaces the prepared-row batch kernels oc_oxk_q4_k_prep_row (and
 * oc_oxk_q5_k_prep_row, oc_oxk_q6_k_prep_row) + oc_oxk_dot_q4_k_prepped_multi
 * (oxidize-c/src/compute/oxk.c:316-366, :372-373, :787-836) driven by
 * matvec_batch_prep_slice (matvec.c:1198-1228).
 *
 * The 32-value formats (Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS and the ids that
 * share their layouts) are taken too, against Q8_0 activations: tiles of 128
 * rows x 64 activations, a 16x16x32 MFMA per block and 16-token chunk, the
 * per-block float step and the block-sequential sum of oxk.c:88-241, so every
 * output is the single-vector dot bit for bit and the matrix is streamed once
 * per 64 activations (the reference walks such a batch four activations at a
 * time, matvec.c:1263-1488).  Rows must be at least 16 bytes long. */
int oxh_mmq(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
            const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
            void *stream);

/* oxh_mmq with options.  OXH_MMQ_RELAXED: the per-block float step of the
 * Q4_K and Q5_K prefill tiles (256 or 128 rows x 128 tokens and 128 x 64,
 * which a launch gets when it fills the device with them) is evaluated as dq * (dw * pos - dmin * min) with fused multiply-adds, five
 * operations per output and block instead of the eight the reference's order
 * takes ((dw*dq)*pos - (dmin*dq)*min, oxk.c:316-366).  The integers are the
 * same and every block term is within an ulp or two of the exact one, so an
 * output differs from the exact one by at most 1e-5 * |exact| + 2e-6 * r, r
 * the root mean square of the launch's outputs (measured: 1.3e-6 * r at
 * worst over 14336 x 4096 x 512; for outputs of unit scale that is well
 * inside the 1e-4 + 1e-5 * |ref| the reference's own tests allow between its
 * kernels), but it is no longer bit-identical to the CPU path.  Off unless asked for: flags = 0
 * is oxh_mmq.  Other types and launches on the smaller tiles ignore the flag.  The host
 * layer passes it when OXH_MMQ_RELAXED=1 is in the environment. */
#define OXH_MMQ_RELAXED 1u
int oxh_mmq_ex(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
               const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
               uint32_t flags, void *stream);

/* oxh_mmq for launches of few tiles over many columns (a 4096 x 14336 down projection under 5-64
 * activations): a tile's workgroup walks all super-blocks of its rows at about a microsecond each, so
 * with fewer than half a 64 x 16 tile per compute unit the launch is paced by that walk.  Here several
 * workgroups share a tile's columns, every super-block's terms go to a workspace of
 * cols/256 x n_vec x out_stride floats and a second launch adds them up in block order: the order the
 * single workgroup adds them in, so the same bits.  oxh_mmq_split_workspace returns the bytes needed, or 0
 * for a launch that would not be split (types other than Q4_K, Q5_K, Q6_K and OXH_Q2_K_WIDE, more tiles,
 * fewer than eight super-blocks, more than 64 activations); oxh_mmq_split with a smaller workspace, or
 * none, is oxh_mmq.
 * The reference has no counterpart (its batch kernel gives every worker whole rows, oxk.c:787-836). */
size_t oxh_mmq_split_workspace(uint32_t qtype, size_t rows, size_t cols, size_t n_vec, size_t out_stride);
int oxh_mmq_split(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                  const void *d_acts, size_t n_vec, float *d_out, size_t out_stride,
                  void *d_workspace, size_t workspace_bytes, void *stream);

/* The tile (weight rows x activations per workgroup) oxh_mmq picks for a launch
 * on a device of n_cu compute units: the largest of 256 x 128 (128 x 128 for
 * Q5_K, Q6_K and widened Q2_K), 64 x 128 (Q6_K only), 128 x 64, 64 x 32, 64 x 16
 * that still gives nearly every compute unit a workgroup; 128 x 64 always for
 * the 32-value formats.  Pure host arithmetic (no device needed); OXH_DECLINED
 * for a type without a matrix-core kernel.
 * The reference has no counterpart: its batch kernel takes four activations
 * per weight row regardless of the shape (oxk.c:787-836). */
int oxh_mmq_tile(uint32_t qtype, size_t rows, size_t n_vec, size_t n_cu, uint32_t *tile_rows,
                 uint32_t *tile_tokens);

/* A Q3_K matrix rewritten as a Q6_K matrix that gives bit-identical results:
 * Q3_K's d * (sc - 32) * (code - 4) is Q6_K's d * sc6 * (code6 - 32) with
 * code6 = code + 28 and sc6 = sc - 32, over the same groups in the same
 * element order, and the two block terms (oxidize-c/src/compute/oxk.c:624-652,
 * :913-964) are the same float of the same integer.  The reference prepares
 * Q3_K rows into its Q6_K batch layout the same way (oxk.c:734-745).  Lets a
 * prefill over Q3_K weights run on oxh_mmq(OXH_Q6_K, ...); d_q6k must hold
 * rows * (cols/256) * 210 bytes. */
int oxh_q3_k_as_q6_k(const void *d_w, size_t rows, size_t cols, void *d_q6k, void *stream);

/* A Q2_K matrix widened for the matrix cores: 210-byte blocks whose 6-bit
 * fields hold scale * code (at most 45), followed by the sixteen group minima
 * as nibbles, dmin and d (oxk.c:592-622 gives the arithmetic: the block term
 * dq * (d * sum sc*code*q - dmin * sum m*bsum), which the tile kernel
 * reproduces to the bit).  The result is not a GGUF type: oxh_mmq accepts it
 * under OXH_Q2_K_WIDE and nothing else does.  d_wide must hold
 * rows * (cols/256) * 210 bytes. */
#define OXH_Q2_K_WIDE 0x1008u
int oxh_q2_k_widen(const void *d_w, size_t rows, size_t cols, void *d_wide, void *stream);

/* Q6_K regrouped for decode: the same bytes, permuted inside every run of eight
 * consecutive blocks (1680 bytes) so that the 16-byte pieces the lanes of a
 * GEMV pass load lie next to each other and aligned:
 *   [0..511] pieces ql[64n+16lh ..] of (block j, lane u = 2n+lh) at 16*(4j+u),
 *   [512..1023] pieces ql[64n+32+16lh ..], [1024..1535] pieces qh[32n+16lh ..],
 *   [1536..1663] the sixteen scales of block j at 16*j, [1664..1679] the f16 d
 *   of block j at 2*j.
 * The plain 210-byte blocks are only 2-byte aligned and every load instruction
 * of a pass touches all 27 cache lines of the pass's span; regrouped, the same
 * pass touches a third as many (decode kernels are paced by exactly that).
 * Size and row order are unchanged; cols must be a multiple of 2048, otherwise
 * OXH_DECLINED.  The result is a weight matrix only oxh_gemv_segments*,
 * oxh_gemv, oxh_matvec* and plans accept, under OXH_Q6_K_G8; oxh_mmq,
 * oxh_get_rows and the expert layer read the file layout.  The host layer keeps
 * this form next to a registered Q6_K range by itself.  d_g8 != d_w, 16-byte
 * aligned, rows * cols / 256 * 210 bytes.  No counterpart in the reference
 * (its CPU kernels read the file layout, oxk.c:913-964). */
#define OXH_Q6_K_G8 0x1009u
int oxh_q6_k_group(const void *d_w, size_t rows, size_t cols, void *d_g8, void *stream);

/* Q4_K / Q5_K stored tile-major for the matrix-core tile kernels: the rows are
 * taken in groups of sixteen, and inside a group the sixteen blocks that share
 * a block index lie next to each other, rows ascending:
 *   block (row r, index b) at ((r / 16) * B + b) * 16 + r % 16   blocks,
 * B = cols / 256.  A wave of the tile kernel fetches exactly such a run per
 * super-block: in the file layout it is sixteen pieces of 144 (176) bytes a row
 * apart, each straddling cache lines it shares with nothing else the wave
 * wants; tile-major it is 2304 (2816) contiguous bytes, 18 (22) whole lines.
 * The memory pipeline charges per line touched, so an expert launch with few
 * tokens per expert runs 10-20 % faster from this form (Mixtral's gate/up at
 * four tokens per expert: 59 -> 53 us per 264 MB).  The blocks themselves are
 * unchanged and so is every result, to the bit.
 *   The last group of a matrix whose rows are not a multiple of sixteen is
 * padded with zero blocks: oxh_tile16_bytes() gives the size (0 for a type or
 * width without this form).  Accepted under OXH_Q4_K_T16 / OXH_Q5_K_T16 by
 * oxh_gemv_segments and oxh_gemv_segments_f32 with d_act_out (1 to 16
 * activations per segment, every segment starting at a group boundary; such a
 * launch always runs on the matrix cores) and by the expert layer (OxhMoe's
 * qtype_gate_up / qtype_down; rows per expert in whole sixteens); everything
 * else reads the file layout and declines these ids.  d_t16 != d_w, both 16-byte
 * aligned.  No counterpart in the reference (its kernels read the file layout,
 * oxk.c:812-897). */
#define OXH_Q4_K_T16 0x100Au
#define OXH_Q5_K_T16 0x100Bu
/* Q8_0 has a tile-major form too (oxh_tile16 with OXH_Q8_0; cols in whole
 * runs of four blocks, i.e. a multiple of 128): per 16-row group and run of
 * four blocks one 2176-byte unit, seventeen whole cache lines,
 *   [0..1023]    blocks 4c, 4c+1 as the matrix cores' operand wants them: the
 *                16-byte piece at 16 * (16q + r) holds row r's values 8q..8q+7
 *                of block 4c (bytes 0-7) and of block 4c+1 (bytes 8-15),
 *   [1024..2047] blocks 4c+2, 4c+3 likewise,
 *   [2048..2175] the f16 scales, row r's four at 2048 + 8r,
 * units in the order (group, run).  A wave fetches a unit with two aligned
 * 16-byte loads per lane and one 8-byte load, straight into the operand
 * registers, where the file layout's 34-byte blocks (2-byte aligned, a row
 * apart) have to be carried through LDS and shifted into place; launches with
 * 2 to 16 activations per weight then stream a large matrix at about the rate
 * of the single-activation kernel.  Accepted under OXH_Q8_0_T16 by
 * oxh_gemv_segments (Q8_0 activations) and oxh_gemv_segments_f32 (the
 * workgroups quantise the f32 inputs themselves; d_act_out may be NULL), 1 to
 * 16 activations per segment, segments starting at group boundaries; results
 * bit-identical to OXH_Q8_0.  A wave walks all of a row group's
 * blocks by itself, so the form pays for matrices with many rows (a
 * vocabulary head) and not for a few hundred long ones. */
#define OXH_Q8_0_T16 0x100Cu
size_t oxh_tile16_bytes(uint32_t qtype, size_t rows, size_t cols);
int oxh_tile16(uint32_t qtype, const void *d_w, size_t rows, size_t cols, void *d_t16, void *stream);

/* Embedding lookup: out[t*out_stride ..] = row d_ids[t] of a packed matrix,
 * expanded to f32 in the reference's dequantisation arithmetic (bit-identical
 * to oc_quant_dequant_row, oxidize-c/src/compute/quantization.c:2781-2795), so
 * the token-embedding table stays quantized in HBM and the ids never leave
 * the device.  Replaces oc_cuda_mmq_get_row / _get_row_dev / _get_row_batch
 * (oxidize-c/include/oxidize/cuda_mmq.h:74-93).  Every type the matvec entry
 * points take (Q2_K ... Q6_K, Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, the AL aliases);
 * d_ids is device memory (at most 65535 per call); an id >= rows gives a row
 * of zeros; d_out and out_stride*4 must be multiples of 16 bytes. */
int oxh_get_rows(uint32_t qtype, const void *d_w, size_t rows, size_t cols,
                 const uint32_t *d_ids, size_t n_ids, float *d_out, size_t out_stride,
                 void *stream);

/* Mixture-of-experts feed-forward with the routing on the device.  For n_tok
 * tokens (router logits [n_tok][n_expert], inputs [n_tok][hidden]):
 *   route    softmax, the top_k experts per token, gate weights (renormalised
 *            over the selected experts when `renorm`)
 *   group    (token, expert) pairs sorted by expert, token order kept
 *   experts  per expert and only for its own tokens: gate, up, silu(gate)*up,
 *            down -- int8 MFMA over Q8_K activations
 *   combine  out[token] = sum, in ascending expert order, of weight * down
 * as oxidize-c/src/model/llama.c:5965-6160 does it on the host; the device
 * analogues are k_moe_route (oxidize-c/src/backends/cuda.cu:495) and
 * oc_cuda_mmq_matvec_expert (oxidize-c/include/oxidize/cuda_mmq.h:64-72).
 * Nothing returns to the host between the steps and the launch sizes depend
 * only on n_tok, so a layer is a fixed sequence that may be captured in a
 * graph.  Expert matrices are stacked expert-major (expert e of gate/up at
 * rows [e*ffn, (e+1)*ffn), of down at rows [e*hidden, (e+1)*hidden)); types
 * Q4_K, Q5_K or Q6_K; at most 64 experts (the expert launches carry up to 32
 * matrices each and repeat beyond that), top_k <= 8, n_tok <= 4096.
 * Expert ids and the grouping are exact; gate weights and silu(gate)*up are
 * float steps that agree with the reference to rounding; everything the
 * integer path computes from them is exact. */
typedef struct OxhMoe {
    uint32_t    qtype_gate_up, qtype_down;
    const void *d_w_gate, *d_w_up, *d_w_down;
    size_t      n_expert, top_k, hidden, ffn;
    int         renorm;
} OxhMoe;
int oxh_moe_workspace_bytes(const OxhMoe *m, size_t n_tok, size_t *bytes);
/* d_workspace: oxh_moe_workspace_bytes() of device memory, 256-byte aligned,
 * overwritten by every call. */
int oxh_moe_ffn(const OxhMoe *m, const float *d_logits, const float *d_x, size_t x_stride,
                size_t n_tok, float *d_out, size_t out_stride, void *d_workspace,
                size_t workspace_bytes, void *stream);
/* oxh_moe_ffn for callers that cannot allocate or pass a workspace (code under
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * workspace is a built-in device array of OXH_MOE_STATIC_WORKSPACE_BYTES per
 * GPU, held until the process ends.  No counterpart in the reference.  The
 * call allocates nothing and initialises nothing: oxh_init must have run.  A
 * layer whose oxh_moe_workspace_bytes() exceeds the built-in array is refused
 * with OXH_ERR_TOO_WIDE.  All calls on a GPU share the one array: calls that
 * overlap in time (two streams, two threads) race; calls on one stream are
 * ordered and safe.  Results are those of oxh_moe_ffn, bit for bit. */
#define OXH_MOE_STATIC_WORKSPACE_BYTES (8u << 20)
int oxh_moe_ffn_static(const OxhMoe *m, const float *d_logits, const float *d_x, size_t x_stride,
                       size_t n_tok, float *d_out, size_t out_stride, void *stream);
/* The routing and grouping step alone (n_expert <= 64).  ids, weights,
 * slot_pos: n_tok*top_k entries, pair (t, j) at t*top_k + j; counts,
 * offsets: per expert (offsets has n_expert + 1 entries); perm: the token of
 * each sorted pair; slot_pos: where pair (t, j) landed in that order. */
int oxh_moe_route(const float *d_logits, size_t n_tok, size_t n_expert, size_t top_k, int renorm,
                  int32_t *d_ids, float *d_weights, uint32_t *d_counts, uint32_t *d_offsets,
                  uint32_t *d_perm, uint32_t *d_slot_pos, void *stream);

/* Device memory / stream / event plumbing so that C callers never include
 * HIP headers (as cuda_mmq.h does with its void* stream). */
int  oxh_malloc(void **d_ptr, size_t bytes);
/* Page-locked host memory (hipHostMalloc): copies to and from it are true
 * asynchronous DMA.  The host-pointer entry points stage their small inputs
 * and outputs through such buffers. */
int  oxh_host_alloc(void **h_ptr, size_t bytes);
int  oxh_host_free(void *h_ptr);
int  oxh_free(void *d_ptr);
int  oxh_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes, void *stream);
int  oxh_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes, void *stream);
int  oxh_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes, void *stream);
/* Rows of `width` bytes between a host matrix with `h_pitch` bytes per row and a device matrix with
 * `d_pitch`: a padded batch travels in one copy (oc_matvec_quantized_batch's in_stride / out_stride). */
int  oxh_memcpy2d_h2d(void *d_dst, size_t d_pitch, const void *h_src, size_t h_pitch, size_t width,
                      size_t height, void *stream);
int  oxh_memcpy2d_d2h(void *h_dst, size_t h_pitch, const void *d_src, size_t d_pitch, size_t width,
                      size_t height, void *stream);
/* A fill kernel, not a memset node: safe between oxh_graph_begin and oxh_graph_end. */
int  oxh_memset(void *d_dst, int value, size_t bytes, void *stream);
int  oxh_stream_create(void **stream);
int  oxh_stream_destroy(void *stream);
int  oxh_stream_sync(void *stream);   /* NULL = the library's internal stream */
int  oxh_event_create(void **event);
int  oxh_event_destroy(void *event);
int  oxh_event_record(void *event, void *stream);
int  oxh_event_sync(void *event);
int  oxh_event_elapsed_ms(void *start, void *stop, float *ms);
/* Capture everything launched on `stream` between begin and end into a HIP
 * graph and replay it with one call: a decode step is a few hundred short
 * launches whose submission cost would otherwise dominate.  The device
 * functions above record no memset nodes.  The reference's counterpart is the
 * graph-replay decode of oxidize-c/src/backends/cuda_fast.cu (cuda.h:250-265). */
int  oxh_graph_begin(void *stream);
int  oxh_graph_end(void *stream, void **graph_exec);
int  oxh_graph_launch(void *graph_exec, void *stream);
int  oxh_graph_destroy(void *graph_exec);
/* name (<=255 chars), compute units, clock MHz, memory bytes. */
int  oxh_device_info(char *name, size_t name_len, int *n_cu, int *clock_mhz,
                     size_t *mem_bytes);
/* Device memory free right now and in all (hipMemGetInfo); either may be NULL. */
int  oxh_mem_info(size_t *free_bytes, size_t *total_bytes);

/* ─── model files ─────────────────────────────────────────────────────── */

/* GGUF v2 / v3 files: the tensor table as weight views for the entry points
 * below, and the upload of every tensor this library has kernels for.
 * Replaces oc_gguf_map_open / oc_gguf_map_tensor_get / oc_gguf_map_tensor_data
 * (oxidize-c/include/oxidize/gguf.h:262-331, parser oxidize-c/src/format/
 * gguf.c:322-505, same acceptance rules), view_from_info
 * (oxidize-c/src/model/llama.c:108-127) and oc_cuda_init's upload loop
 * (oxidize-c/src/backends/cuda.cu:633-712).  The file is mapped read-only and
 * never copied on the host; a malformed file is OXH_ERR_FORMAT, never a crash. */
#define OXH_GGUF_MAX_DIMS 8u

typedef struct OxhGguf OxhGguf;

typedef struct OxhTensor {
    const char *name;       /* NUL-terminated, owned by the OxhGguf                     */
    uint32_t    qtype;      /* type id as the matvec entry points take it (oxidize-c/
                               include/oxidize/quant.h:92-140), OXH_QTYPE_UNKNOWN if the
                               on-disk id is not one the reference maps                 */
    uint32_t    ggml_type;  /* the on-disk id                                           */
    uint32_t    n_dims;
    uint64_t    dims[OXH_GGUF_MAX_DIMS];    /* dims[0] is the innermost                 */
    uint64_t    offset;     /* from the start of the data section                       */
    const void *data;       /* inside the mapping                                       */
    size_t      nbytes;     /* 0 when the type has no fixed block layout here           */
    size_t      rows;       /* product of dims[1..]: a stacked expert tensor is all its
                               experts' rows, expert e at rows [e*dims[1], (e+1)*dims[1]) */
    size_t      cols;       /* dims[0]                                                  */
    size_t      row_bytes;  /* packed bytes of one row, 0 if cols is not whole blocks   */
    int         resident;   /* made resident by oxh_gguf_register_all                   */
} OxhTensor;

int  oxh_gguf_open(const char *path, OxhGguf **out);
/* Unregisters what oxh_gguf_register_all made resident and unmaps the file. */
void oxh_gguf_close(OxhGguf *g);
/* Any of the out pointers may be NULL. */
int  oxh_gguf_info(const OxhGguf *g, uint32_t *version, uint64_t *alignment, uint64_t *data_start,
                   size_t *n_tensors, size_t *n_metadata);
int  oxh_gguf_tensor_at(const OxhGguf *g, size_t index, OxhTensor *out);
/* OXH_DECLINED when there is no tensor of that name. */
int  oxh_gguf_tensor_find(const OxhGguf *g, const char *name, OxhTensor *out);
/* Metadata by key: OXH_DECLINED when the key is absent or of another kind
 * (u64: any integer or bool that is not negative; f64: F32 or F64; str: the
 * bytes inside the mapping, not NUL-terminated). */
int  oxh_gguf_meta_u64(const OxhGguf *g, const char *key, uint64_t *out);
int  oxh_gguf_meta_f64(const OxhGguf *g, const char *key, double *out);
int  oxh_gguf_meta_str(const OxhGguf *g, const char *key, const char **data, size_t *len);
/* Makes every matrix (2 or more dimensions) whose type and width have an
 * integer path here resident in HBM, whole, so that later matvec calls on
 * the tensor or on an expert slice of it find it there. */
int  oxh_gguf_register_all(OxhGguf *g, size_t *n_registered, size_t *bytes);
/* On-disk type id -> type id of the matvec entry points
 * (oc_quant_type_from_ggml_id, oxidize-c/src/compute/quantization.c:2980-2988). */
uint32_t oxh_qtype_from_ggml_id(uint32_t ggml_id);

/* ─── layer 1: drop-in host API ───────────────────────────────────────── */

/* Make the bytes at [h_data, h_data+bytes) resident in HBM and remember the
 * mapping, so later calls that pass any pointer inside that range (a whole
 * tensor or an expert slice of a stacked tensor) run without an upload and
 * without looking at the host bytes.  Modelled on oc_cuda_init's weight upload
 * (oxidize-c/src/backends/cuda.cu:633-712).  Registered weights are taken to
 * be immutable, as there: unregister before reusing the memory.
 *
 * Weights the caller never registered keep the reference's contract, under
 * which the host bytes are the input of every call (oxidize-c/include/oxidize/
 * matvec.h:45-52), with ONE STATED LIMIT.  The device copy made on first sight
 * serves only the exact (pointer, byte count) it was made for, and every later
 * call re-checks the host bytes before using it (a few microseconds):
 *   - the length, the first and last 4 KiB and 128 strided 64-byte samples:
 *     a freed model replaced by another at the same addresses, a buffer
 *     refilled, a matrix that overlaps older cached ones: seen on that call;
 *   - two 16 KiB slices, hashed whole against the hashes taken of every slice
 *     at upload, the slices taking turns from call to call: an edit of ANY
 *     size ANYWHERE in the matrix is seen after at most
 *     ceil(bytes / 32 KiB) calls over that matrix (1008 for 33 MB).
 * THE LIMIT: a few bytes patched in place, between the samples, may be served
 * from the old device copy until the rotating slices reach them.  A caller
 * that edits weights in place and needs the very next call to see the edit
 * calls oxh_weight_unregister(ptr) after the edit (it drops cached copies as
 * well), or runs with OXH_WEIGHT_CACHE=full (every byte hashed on every call)
 * or =off (uploaded on every call).  Registered ranges are never looked at.
 * OXH_WEIGHT_CACHE_MB bounds the bytes cached this way and their rewritten
 * forms (default: half of the device memory free when the first one is made);
 * the least recently used go first, also when the device itself runs out. */
int oxh_weight_register(const void *h_data, size_t bytes);
/* Drops every range, registered or cached, that contains h_data. */
int oxh_weight_unregister(const void *h_data);
/* Drop every range (the host memory may then be reused or freed). */
int oxh_weight_clear(void);
/* Device address backing a host pointer inside a registered or cached range, or NULL. */
const void *oxh_weight_device_ptr(const void *h_data);
/* Counts of registered and cached ranges, the bytes cached, and how many times
 * a cached copy was refreshed because its host bytes had changed.  Any pointer
 * may be NULL. */
int oxh_weight_stats(size_t *n_registered, size_t *n_cached, size_t *cached_bytes, size_t *refreshes);
/* Cached ranges given up so far for the budget or for want of device memory. */
size_t oxh_weight_evictions(void);

/* Same arguments and results as oc_matvec_quantized
 * (oxidize-c/include/oxidize/matvec.h:50-52; matvec.c:833-907): output[r] =
 * dot(W[r], Q8(input)); `temp` (>= cols floats) receives the quantised
 * activation bytes exactly as the reference leaves them there, for Q4_0 and
 * AL5 followed (from the next multiple of four bytes) by the int32 sum of
 * every 32-value block (matvec.c:198-227, :866-877). */
int oxh_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp);
/* oc_matvec_quantized_fused (matvec.h:62-66; matvec.c:1525-1594). */
int oxh_matvec_quantized_fused(const uint32_t *qtypes,
                               const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input,
                               float *const *outs, float *temp);
/* oc_matvec_quantized_multi_input (matvec.h:72-76; matvec.c:1597-1680). */
int oxh_matvec_quantized_multi_input(const uint32_t *qtypes,
                                     const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs,
                                     float *const *outs, float *temp);
/* oc_matvec_quantized_batch (matvec.h:118-124; matvec.c:1263-1488).
 * `act_scratch`/`act_bytes` keep the reference's meaning for eligibility
 * (NULL or too small for one activation => OXH_DECLINED); the quantised
 * activations themselves stay on the device. */
int oxh_matvec_quantized_batch(uint32_t qtype, const uint8_t *data,
                               size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec,
                               float *temp, uint8_t *act_scratch,
                               size_t act_bytes);

/* The reference's own symbols (matvec.h:50-52, :62-66, :72-76, :118-124,
 * :132, :146-147, :81-88).  They call the oxh_ functions above.  Because they
 * return void, a call that comes back declined or failed is handed on, with
 * its original arguments, to the CPU functions installed with
 * oxh_set_cpu_fallback(); failing that to the symbols oc_ref_matvec_quantized,
 * _fused, _multi_input and _batch when the program defines them (weak
 * references: the reference's own functions under another name); failing that
 * the handler of oxh_set_decline_handler() is told; and with none of the three
 * the process prints the error and aborts.  This library never computes on
 * the CPU itself. */
typedef struct {
    size_t activation_quantizations;
    size_t parallel_dispatches;
    size_t fallback_calls;
} OcMatvecFusedTestStats;

void oc_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp);
void oc_matvec_quantized_fused(const uint32_t *qtypes,
                               const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input,
                               float *const *outs, float *temp);
void oc_matvec_quantized_multi_input(const uint32_t *qtypes,
                                     const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs,
                                     float *const *outs, float *temp);
void oc_matvec_quantized_batch(uint32_t qtype, const uint8_t *data,
                               size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec,
                               float *temp, uint8_t *act_scratch,
                               size_t act_bytes);
size_t oc_matvec_batch_scratch_bytes(size_t max_cols);
void oc_matvec_set_fused(bool enabled);
bool oc_matvec_fused_enabled(void);
void oc_matvec_fused_test_reset(void);
OcMatvecFusedTestStats oc_matvec_fused_test_stats(void);

/* The caller's CPU implementations of the four entry points (the reference's
 * own oc_matvec_quantized* under whatever names the build gives them); a NULL
 * member falls through to the weak oc_ref_* symbol of that entry.  NULL clears
 * the table.  Set before the first matvec call; not synchronised with calls in
 * flight. */
typedef struct OxhCpuFallback {
    void (*matvec_quantized)(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                             const float *input, float *output, float *temp);
    void (*matvec_quantized_fused)(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                                   size_t cols, const size_t *row_bytes, size_t n_outs, const float *input,
                                   float *const *outs, float *temp);
    void (*matvec_quantized_multi_input)(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                                         size_t cols, const size_t *row_bytes, size_t n_outs,
                                         const float *const *inputs, float *const *outs, float *temp);
    void (*matvec_quantized_batch)(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols,
                                   size_t row_bytes, const float *inputs, size_t in_stride, float *outputs,
                                   size_t out_stride, size_t n_vec, float *temp, uint8_t *act_scratch,
                                   size_t act_bytes);
} OxhCpuFallback;
void oxh_set_cpu_fallback(const OxhCpuFallback *fb);
/* Calls handed on to a CPU fallback so far. */
size_t oxh_cpu_fallback_calls(void);

/* Called by the void oc_matvec_* symbols when the oxh_ call did not return
 * OXH_OK and no CPU fallback exists for that entry.  `which` is 0 single,
 * 1 fused, 2 multi_input, 3 batch; `status` is the oxh_ status. */
typedef void (*OxhDeclineHandler)(int which, int status, void *user);
void oxh_set_decline_handler(OxhDeclineHandler fn, void *user);

#ifdef __cplusplus
}
#endif
#endif /* OXHIP_H */
