/* oxhip_lab.h — test hooks and measurement aids of liboxhip.
 *
 * None of these has a counterpart in the reference and none belongs to the
 * drop-in surface: the shared library exports exactly the functions that
 * include/oxhip.h declares plus the one accessor below, and everything here is
 * reached through the table it returns.  The parity tests use the hooks to
 * read intermediates (sub-block sums, the expert layer's workspace), the
 * benchmark uses the probes to measure what the device itself can do.
 */
#ifndef OXHIP_LAB_H
#define OXHIP_LAB_H

#include "oxhip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct OxhLab {
    /* With d_stamps set (n_ops * workgroups * 8 uint64 of device memory, or
     * NULL to switch it off) wave 0 of every workgroup of a plan launch stores
     * the shader clock at eight points of every operation: start, dependency
     * met, activation staged, workgroup barrier passed, passes done, rows
     * summed, barrier passed, outputs stored and announced. */
    int (*plan_stamps)(OxhPlan *plan, uint64_t *d_stamps);
    /* With `on` set the waits of a plan also expect a workgroup that does not
     * exist, so every wait runs into the poll limit: the way to test the
     * give-up path from the host without hanging anything. */
    int (*plan_phantom)(OxhPlan *plan, int on);
    /* Byte offsets inside oxh_moe_ffn's workspace of, in this order, ids,
     * weights, slot_pos, perm, counts, offsets, the gathered Q8_K activations,
     * gate, up (f32 [pair][ffn]), the Q8_K form of silu(gate)*up, the down
     * outputs (f32 [pair][hidden]), and the total size.  After a call the
     * parity tests read every intermediate from there. */
    int (*moe_workspace_parts)(const OxhMoe *m, size_t n_tok, size_t parts[12]);
    /* One launch that only reads `bytes` of device memory (a workgroup per CU,
     * 16-byte loads, nothing computed); d_sink may be NULL.  Timed on a buffer
     * the size of a weight matrix it gives the ceiling any kernel streaming
     * that matrix once can reach on the device, launch cost included. */
    int (*read_probe)(const void *d_buf, size_t bytes, uint32_t *d_sink, void *stream);
    /* The int8 matrix-core rate of the whole device (POP/s) when every
     * v_mfma_i32_16x16x64_i8 is followed by `valu_per_mfma` (0, 1, 2 or 4)
     * independent f32 vector instructions, with 1..4 waves per SIMD.
     * Synchronous (two launches, the second timed with events). */
    int (*mfma_probe)(int valu_per_mfma, int waves_per_simd, double *pops);
    /* The integer sub-block sums the GEMV kernel forms, written by the same
     * device code path.  Q4_K and Q5_K: 8 int32 per super-block (S_j), Q6_K: 16
     * per super-block, Q8_0: 1 per block; layout [row][block][j].  The values
     * are the intermediates of oxidize-c/src/compute/oxk.c:263-283, :870-886,
     * :932-954, :234-237, which the reference's API does not expose. */
    int (*subblock_sums)(uint32_t qtype, const void *d_w, size_t rows, size_t cols, const void *d_act,
                         int32_t *d_sums, void *stream);
} OxhLab;

const OxhLab *oxh_lab(void);

#ifdef __cplusplus
}
#endif
#endif
