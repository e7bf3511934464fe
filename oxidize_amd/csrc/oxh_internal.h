/* oxh_internal.h — symbols shared between the HIP translation unit and the C
 * host layer of liboxhip; not part of the public ABI: the library's export list is
 * made from the public headers, so nothing declared here is visible outside it. */
#ifndef OXH_INTERNAL_H
#define OXH_INTERNAL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* printf-style with exactly two %s slots (either may be NULL). */
void oxh_set_error(const char *fmt, const char *a, const char *b);
/* The stream created by oxh_init(). */
void *oxh_internal_stream(void);
/* Largest n_vec (1..8) one GEMV launch can stage for (qtype, cols); 0 when
 * even a single activation does not fit. */
size_t oxh_gemv_max_nvec(uint32_t qtype, size_t cols);
/* The same for a launch that passes a buffer for the quantised activations
 * (up to 16 for Q8_0 weights, which then run on the matrix cores). */
size_t oxh_gemv_max_nvec_buffered(uint32_t qtype, size_t cols);

/* Sets the thread's error text (printf-style) and returns `status`. */
int oxh_internal_errorf(int status, const char *fmt, ...);
/* Compute units and index of the device oxh_init() chose (0 / -1 before it ran). */
int oxh_internal_n_cu(void);
int oxh_internal_device(void);
/* Host layer: drop the weight registry and the staging buffers (oxh_shutdown). */
void oxh_internal_host_reset(void);

/* Plans over the 32-value formats: a table of plain GEMV launches walked by one grid (oxh_kernels.hip).
 * `ops` is an array of OxhPlanOp; which = -1 for a type without such a launch. */
struct OxhPlanOp;
int oxh_internal_multi_which(uint32_t qtype);
int oxh_internal_multi_create(const struct OxhPlanOp *ops, size_t n_ops, void **handle);
int oxh_internal_multi_launch(void *handle, void *stream);
void oxh_internal_multi_info(const void *handle, size_t *n_items, size_t *workgroups, size_t *lds_bytes);
int oxh_internal_multi_destroy(void *handle);
/* 16-byte-granular copy by a kernel (either side may be page-locked host memory). */
int oxh_internal_copy16(void *dst, const void *src, size_t bytes, void *stream);
/* Wait for a stream by polling it `spins` times before blocking. */
int oxh_internal_stream_sync_spin(void *stream, unsigned spins);


/* The functions behind include/oxhip_lab.h's table (not exported by name). */
struct OxhPlan;
struct OxhMoe;
int oxh_debug_plan_stamps(struct OxhPlan *plan, uint64_t *d_stamps);
int oxh_debug_plan_phantom(struct OxhPlan *plan, int on);
int oxh_debug_moe_workspace_parts(const struct OxhMoe *m, size_t n_tok, size_t parts[12]);
int oxh_debug_read_probe(const void *d_buf, size_t bytes, uint32_t *d_sink, void *stream);
int oxh_debug_mfma_probe(int valu_per_mfma, int waves_per_simd, double *pops);
int oxh_debug_subblock_sums(uint32_t qtype, const void *d_w, size_t rows, size_t cols, const void *d_act,
                            int32_t *d_sums, void *stream);

#ifdef __cplusplus
}
#endif
#endif
