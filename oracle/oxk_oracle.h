/*
 * oxk_oracle.h — CPU restatement of oxidize-c's quantized-matvec arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * Every function restates one reference function (cited below, paths relative
 * to the reference checkout, oxidize-c/...) in plain scalar C, compiled with
 * -ffp-contract=off exactly like the reference (oxidize-c/Makefile:20-21).
 * Unlike the reference, the dot functions can also hand back the per-sub-block
 * int32 sums, which are the quantities the GPU path must reproduce bit for bit.
 *
 * Pinning status (what each function was checked against):
 *   oxo_f16_to_f32        all 65536 inputs vs numpy float16 and vs the compiled
 *                         reference; KATs of tests/test_oxk.c:8-47
 *   oxo_f32_to_f16_bits   dense sample + ties/subnormals vs compiled reference
 *   oxo_scale_min_k4      KATs tests/test_oxk.c:72-103; exhaustive byte triples
 *                         vs compiled reference
 *   oxo_quantize_q8_k/0   compiled reference through oc_matvec_quantized (the
 *                         activation is left in `temp`); invariants (bsums);
 *                         rounding ties, largest floats, subnormal scales.
 *                         Not pinned, because the reference has no single
 *                         answer there: blocks whose 1/d overflows (largest
 *                         magnitude below 3.7e-37) and non-finite inputs
 *   oxo_dot_*             compiled reference scalar + dispatched kernels on the
 *                         raw-block generator of tests/test_oxk_avx2_parity.c,
 *                         closed forms, dequantised double-precision cross-check
 *   oxo_matvec_*          compiled reference entry points, float bits
 *   oxo_dequant_row       compiled reference oc_quant_dequant_row, float bits
 *   oxo_rms_norm_f32,     compiled reference (oc_rms_norm_f32, oc_swiglu_inplace_f32)
 *   oxo_swiglu_f32        to 1e-6 relative, double-precision numpy, closed
 *                         forms (constant vector, silu(0) = 0, large |g|)
 *   oxo_moe_route         brute force (argsort of a double-precision softmax)
 *   oxo_moe_ffn           composition of the functions above; against a numpy
 *                         restatement built from per-expert dense products of
 *                         the dequantised matrices (loose tolerance: pins the
 *                         routing, grouping, expert indexing and combination,
 *                         not the rounding, which the parts pin)
 * No function is "parity unpinned".
 */
#ifndef OXK_ORACLE_H
#define OXK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF type ids used on this path (include/oxidize/quant.h:94-110). */
enum {
    OXO_Q4_0   = 3,
    OXO_Q4_1   = 4,
    OXO_Q5_0   = 5,
    OXO_Q5_1   = 6,
    OXO_Q8_0   = 7,
    OXO_Q2_K   = 8,
    OXO_Q3_K_S = 9,
    OXO_Q3_K_M = 10,
    OXO_Q3_K_L = 11,
    OXO_Q4_K_S = 12,
    OXO_Q4_K_M = 13,
    OXO_Q5_K_S = 14,
    OXO_Q5_K_M = 15,
    OXO_Q6_K   = 16,
    OXO_AL5    = 17,    /* Q4_0 layout */
    OXO_AL5_XS = 18,    /* f16 d + 32 three-bit codes in 12 bytes */
    OXO_AL6    = 19,    /* Q5_0 layout */
    OXO_AL8    = 20,    /* Q8_0 layout */
    OXO_IQ4_NL = 26,    /* f16 d + 16 nibble bytes per 32 values (dequantise path only) */
    OXO_IQ4_XS = 27,    /* f16 d + u16 scale high bits + 4 scale nibble bytes + 128 nibble bytes per 256 */
    OXO_IQ3_S  = 25,    /* f16 d + 64 grid codes + 8 ninth bits + 32 sign bytes + 4 scale bytes */
    OXO_IQ1_XXXS = 36,  /* f16 d + 32 codebook indices + 4 scale|sign bytes */
};

#define OXO_QK_K        256u
#define OXO_QK8_0       32u
#define OXO_AL5_XS_BYTES 14u
#define OXO_Q2_K_BYTES  84u
#define OXO_Q3_K_BYTES  110u
#define OXO_Q4_K_BYTES  144u
#define OXO_Q5_K_BYTES  176u
#define OXO_Q6_K_BYTES  210u
#define OXO_Q8_0_BYTES  34u
#define OXO_Q8_K_BYTES  292u
#define OXO_IQ3_S_BYTES 110u
#define OXO_IQ1_XXXS_BYTES 38u

/* src/compute/oxk.c:26-56 */
float    oxo_f16_to_f32(uint16_t h);
/* src/compute/flash_attention.c:149-185 (round-half-up, not RNE) */
uint16_t oxo_f32_to_f16_bits(float v);
/* src/compute/oxk.c:60-75 */
void     oxo_scale_min_k4(unsigned j, const uint8_t scales[12],
                          uint8_t *sc, uint8_t *mn);

/* src/compute/matvec.c:276-316 — n must be a multiple of 256. */
void oxo_quantize_q8_k(const float *x, size_t n, uint8_t *out);
/* src/compute/matvec.c:130-155 — n must be a multiple of 32. */
void oxo_quantize_q8_0(const float *x, size_t n, uint8_t *out);

/* src/compute/oxk.c:243-297.  `sub` (optional) receives 8 int32 per block:
 * S_j = sum over sub-block j of nibble * q8.  `posmin` (optional) receives
 * 2 int32 per block: {sum_j sc_j*S_j, sum_j m_j*B_j}. */
float oxo_dot_q4_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *sub, int32_t *posmin);
/* src/compute/oxk.c:849-911 (same scale/min decode and f32 expression as
 * Q4_K; the fifth bit of element 32j + l is bit j of byte l of the 32-byte
 * plane at block offset 16).  `sub` and `posmin` as for Q4_K. */
float oxo_dot_q5_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *sub, int32_t *posmin);
/* src/compute/oxk.c:913-964.  `grp` (optional) receives 16 int32 per block. */
float oxo_dot_q6_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *grp);
/* src/compute/oxk.c:592-622 (Q2_K: 16 bytes of 4-bit scale | 4-bit min, 64
 * bytes of 2-bit codes, f16 d, f16 dmin; the block term is
 * dq*(d*pos - dmin*min)) and :624-652 (Q3_K: 32 bytes of third bits, 64 bytes
 * of 2-bit codes, sixteen 6-bit scales in 12 bytes, f16 d; codes 0..7 with a
 * uniform offset of 4: d*dq*(pos - 4*off)).  `grp` (optional) receives the 16
 * int32 group sums per block. */
/* src/compute/oxk.c:1052-1116: IQ3_S.  Each 32-value sub-block: eight 9-bit codes (8 bits in qs, the
 * ninth in qh) into a codebook of four magnitudes each, a sign bit per value, an odd scale 2*s+1 from a
 * nibble.  The f32 part is NOT one term per block: eight float lanes, lane j taking the positions
 * 4j..4j+3 of every sub-block, acc[j] = acc[j] + d*(float)lane[j] per block, reduced at the end as
 * ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)).  `lanes` (optional) receives the 8 int32 per block.
 * Pinned: tests/golden/iq_types.npz (compiled reference, scalar and dispatched forms) and live;
 * a one-hot construction that isolates every (sub-block, position) pair. */
float oxo_dot_iq3_s_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *lanes);
/* src/compute/quantization.c:941-1015 (scalar branch): IQ1_XXXS.  Each group of 8 values is one byte
 * into a codebook of {-1,0,+1}^8; per 32 values an odd scale 2*(n&7)+1 and a sign of the common offset
 * 0.125: block term dw*da*((float)main + 0.125f*(float)delta), summed in block order.  `sums`
 * (optional) receives {main, delta} per block.  Pinned like IQ3_S. */
float oxo_dot_iq1_xxxs_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *sums);
float oxo_dot_q2_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *grp);
float oxo_dot_q3_k_q8_k(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *grp);
/* src/compute/oxk.c:224-241 (block-sequential scalar chain).  `isum`
 * (optional) receives one int32 per block. */
float oxo_dot_q8_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act,
                        int32_t *isum);

/* src/compute/oxk.c:88-113, :115-139, :141-165, :167-191 (scalar forms, the
 * block-sequential f32 chain).  `isum` (optional): one int32 per block, the
 * offset-corrected dot for Q4_0 / Q5_0, the plain code dot for Q4_1 / Q5_1. */
float oxo_dot_q4_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum);
float oxo_dot_q4_1_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum);
float oxo_dot_q5_0_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum);
float oxo_dot_q5_1_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum);
/* src/compute/oxk.c:195-222: codes 0..7 with an offset of 4, (dw*dq) * (float)isum per block */
float oxo_dot_al5_xs_q8_0(const uint8_t *row, size_t blocks, const uint8_t *act, int32_t *isum);

/* 0 = not eligible for the integer path, 1 = Q8_0 activation, 2 = Q8_K
 * (src/compute/matvec.c:99-127 restricted to the types above) and the stride
 * rule of src/compute/matvec.c:961-985. */
int oxo_act_kind(uint32_t qtype, size_t cols);
int oxo_stride_ok(uint32_t qtype, size_t cols, size_t row_bytes);

/* src/compute/matvec.c:833-907 (integer path only).  Returns 0 when handled,
 * 1 when the reference would have taken its dequantise-to-f32 path (which
 * this oracle does not restate).  `temp` receives the quantised activation. */
int oxo_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp);
/* src/compute/matvec.c:1525-1594 */
int oxo_matvec_quantized_fused(const uint32_t *qtypes,
                               const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input,
                               float *const *outs, float *temp);
/* src/compute/matvec.c:1597-1680 */
int oxo_matvec_quantized_multi_input(const uint32_t *qtypes,
                                     const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs,
                                     float *const *outs, float *temp);
/* src/compute/matvec.c:1263-1488 (integer path; every output is the same
 * single-vector dot, so no tiling is restated). */
int oxo_matvec_quantized_batch(uint32_t qtype, const uint8_t *data,
                               size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec,
                               uint8_t *act_scratch, size_t act_bytes);
/* src/compute/matvec.c:997-1014 with the default 4 MiB tile. */
size_t oxo_matvec_batch_scratch_bytes(size_t max_cols);

/* MoE routing as the prefill caller does it (src/model/llama.c:5965-6031):
 * softmax over n_expert logits, top-k by repeated strict-greater scan (ties
 * keep the lower index), optional renormalisation.  ids/weights: n_tok*k. */
void oxo_moe_route(const float *logits, size_t n_tok, size_t n_expert,
                   size_t k, int renorm, int32_t *ids, float *weights);

/* One MoE feed-forward layer over n_tok tokens as src/model/llama.c:5965-6160
 * runs it (quantised expert matrices, no shared or zero experts): route, then
 * experts in ascending order, each over its tokens in token order: gate, up,
 * SwiGLU, down, out[token] += weight * down.  Expert matrices stacked
 * expert-major.  Returns 0 when every matvec took the integer path. */
int oxo_moe_ffn(uint32_t qtype_gate_up, uint32_t qtype_down, const uint8_t *w_gate,
                const uint8_t *w_up, const uint8_t *w_down, size_t n_expert, size_t k,
                size_t hidden, size_t ffn, int renorm, const float *logits,
                const float *x, size_t n_tok, float *out);

/* The float steps a decode layer runs in front of the quantiser, scalar forms:
 * RMSNorm (src/compute/activation.c:16-22 with the scalar dot and apply of
 * src/compute/attn_kernels.c:6-11, :28-33) and SwiGLU
 * (src/compute/activation.c:92-99).  The reference's x86 builds sum the
 * squares in SIMD lanes and use a polynomial exp, so they agree with these
 * to rounding, not to the bit. */
void oxo_rms_norm_f32(const float *x, const float *weight, float *out, size_t n,
                      float eps);
void oxo_swiglu_f32(const float *gate, const float *up, float *out, size_t n);

/* Dequantise one row to f32 (src/compute/quantization.c:486-503, :633-670,
 * :672-721, :723-766): the checker of the embedding lookup, and an independent
 * cross-check of the layouts behind the dot functions. */
int oxo_dequant_row(uint32_t qtype, const uint8_t *row, size_t cols, float *out);
/* The types without an integer dot (IQ4_NL, IQ4_XS) go through the reference's dequantise loop,
 * src/compute/matvec.c:799-831: a row expanded to f32 (src/compute/quantization.c:1401-1459, restated
 * in oxo_dequant_row and pinned to the compiled reference's bits), then dotted with the f32 input.
 * The reference's dot runs in SIMD lanes whose order depends on the host, so this restatement sums in
 * double: out[r] is the exact-order-free value, mag[r] = sum |w*x| the scale a tolerance goes by.
 * Pinned against the compiled reference's oc_matvec_quantized within 4e-6 * mag (f32 lane sums).
 * Returns 1 for any other type or a width that is not a whole number of blocks. */
int oxo_matvec_dequant(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                       const float *x, double *out, double *mag);
size_t oxo_dequant_path_row_bytes(uint32_t qtype, size_t cols);

#ifdef __cplusplus
}
#endif
#endif
