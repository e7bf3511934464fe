/*
 * oc_matvec.c — host side of liboxhip: the drop-in for oxidize-c's quantized
 * matvec API (oxidize-c/include/oxidize/matvec.h), written against the thin
 * device layer in oxh_kernels.hip.  Plain C11; never includes a HIP header.
 *
 * What is mirrored from oxidize-c/src/compute/matvec.c:
 *   eligibility        fused_act_kind :99-127, fused_stride_ok :961-985,
 *                      the global on/off switch and OC_NO_FUSED :67-86
 *   oc_matvec_quantized          :833-907   quantise once, every row one dot,
 *                                           activation bytes left in `temp`
 *   oc_matvec_quantized_fused    :1525-1594 one quantisation + one launch when
 *                                           all matrices share an eligible type
 *   oc_matvec_quantized_multi_input :1597-1680
 *   oc_matvec_quantized_batch    :1263-1488
 *   dispatch counters            :55-65, :1571-1572, :1584-1592
 *
 * What is NOT here on purpose: the reference's dequantise-to-f32 path.  When
 * the integer path is not eligible the functions return OXH_DECLINED and
 * touch nothing; there is no CPU arithmetic in this library.
 */
#include "oxhip.h"
#include "oxh_internal.h"

#include <pthread.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ─── fused switch + counters ─────────────────────────────────────────── */

static atomic_bool g_fused = true;
static atomic_bool g_env_seen = false;
static _Thread_local OcMatvecFusedTestStats g_stats;

void oc_matvec_fused_test_reset(void) { memset(&g_stats, 0, sizeof g_stats); }
OcMatvecFusedTestStats oc_matvec_fused_test_stats(void) { return g_stats; }

void oc_matvec_set_fused(bool enabled)
{
    atomic_store(&g_fused, enabled);
    atomic_store(&g_env_seen, true);
}

bool oc_matvec_fused_enabled(void)
{
    if (!atomic_load(&g_env_seen)) {
        const char *e = getenv("OC_NO_FUSED");
        if (e && e[0] && e[0] != '0') atomic_store(&g_fused, false);
        atomic_store(&g_env_seen, true);
    }
    return atomic_load(&g_fused);
}

size_t oc_matvec_batch_scratch_bytes(size_t max_cols)
{
    /* Same bound as the reference (matvec.c:997-1014): the larger of one
     * activation (Q8_K, or Q8_0 plus its 4-byte-per-block scale tail) and the
     * 4 MiB activation tile. */
    const size_t nbk = max_cols / OXH_QK_K, nb0 = max_cols / OXH_QK8_0;
    if (nbk > SIZE_MAX / OXH_Q8_K_BYTES || nb0 > (SIZE_MAX - 3u) / 38u) return SIZE_MAX;
    const size_t q8k = nbk * OXH_Q8_K_BYTES;
    const size_t q80 = ((nb0 * OXH_Q8_0_BYTES + 3u) & ~(size_t)3u) + nb0 * 4u;
    const size_t one = q8k > q80 ? q8k : q80;
    const size_t tile = (size_t)4u << 20;
    return one > tile ? one : tile;
}

/* ─── weight registry: host range -> device copy ──────────────────────── */

typedef struct {
    const uint8_t *h;
    size_t bytes;
    uint8_t *d;
} Resident;

static pthread_mutex_t g_lock = PTHREAD_MUTEX_INITIALIZER;
/* Held for the whole of a matvec call, and by the calls that free device weights (taken before g_lock):
 * the staging buffers and the library's stream are shared by every call, so concurrent callers are
 * serialised (the reference's worker pool is one process-global resource too, include/oxidize/parallel.h:13-19). */
static pthread_mutex_t g_call = PTHREAD_MUTEX_INITIALIZER;
static Resident *g_res = NULL;
static size_t g_nres = 0, g_cap = 0;

static Resident *find_range(const uint8_t *p, size_t bytes)
{
    for (size_t i = 0; i < g_nres; i++) {
        const Resident *r = &g_res[i];
        /* p must lie inside the range: the end of one tensor is the start of the
         * next in a mapped model file */
        if (p >= r->h && (size_t)(p - r->h) < r->bytes &&
            bytes <= r->bytes - (size_t)(p - r->h))
            return &g_res[i];
    }
    return NULL;
}

static int register_locked(const uint8_t *h, size_t bytes, Resident **out)
{
    if (g_nres == g_cap) {
        const size_t nc = g_cap ? g_cap * 2 : 64;
        Resident *n = (Resident *)realloc(g_res, nc * sizeof *n);
        if (!n) {
            oxh_set_error("out of host memory growing the weight registry%s%s", NULL, NULL);
            return OXH_ERR_NOMEM;
        }
        g_res = n;
        g_cap = nc;
    }
    void *d = NULL;
    int rc = oxh_malloc(&d, bytes);
    if (rc) return rc;
    rc = oxh_memcpy_h2d(d, h, bytes, NULL);
    if (!rc) rc = oxh_stream_sync(NULL);
    if (rc) {
        oxh_free(d);
        return rc;
    }
    g_res[g_nres].h = h;
    g_res[g_nres].bytes = bytes;
    g_res[g_nres].d = (uint8_t *)d;
    if (out) *out = &g_res[g_nres];
    g_nres++;
    return OXH_OK;
}

int oxh_weight_register(const void *h_data, size_t bytes)
{
    if (!h_data || bytes == 0) {
        oxh_set_error("invalid argument: %s%s", "oxh_weight_register: empty range", NULL);
        return OXH_ERR_ARG;
    }
    pthread_mutex_lock(&g_lock);
    int rc = OXH_OK;
    if (!find_range((const uint8_t *)h_data, bytes))
        rc = register_locked((const uint8_t *)h_data, bytes, NULL);
    pthread_mutex_unlock(&g_lock);
    return rc;
}

int oxh_weight_unregister(const void *h_data)
{
    int rc = OXH_OK;
    pthread_mutex_lock(&g_call);
    pthread_mutex_lock(&g_lock);
    for (size_t i = 0; i < g_nres; i++) {
        if (g_res[i].h == (const uint8_t *)h_data) {
            rc = oxh_stream_sync(NULL);
            if (!rc) rc = oxh_free(g_res[i].d);
            g_res[i] = g_res[g_nres - 1];
            g_nres--;
            break;
        }
    }
    pthread_mutex_unlock(&g_lock);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_weight_clear(void)
{
    pthread_mutex_lock(&g_call);
    pthread_mutex_lock(&g_lock);
    int rc = g_nres ? oxh_stream_sync(NULL) : OXH_OK;
    for (size_t i = 0; i < g_nres; i++) {
        const int r = oxh_free(g_res[i].d);
        if (!rc) rc = r;
    }
    g_nres = 0;
    pthread_mutex_unlock(&g_lock);
    pthread_mutex_unlock(&g_call);
    return rc;
}

const void *oxh_weight_device_ptr(const void *h_data)
{
    pthread_mutex_lock(&g_lock);
    const Resident *r = find_range((const uint8_t *)h_data, 0);
    const void *d = r ? r->d + ((const uint8_t *)h_data - r->h) : NULL;
    pthread_mutex_unlock(&g_lock);
    return d;
}

/* Device address of `bytes` of weights starting at host pointer p, uploading
 * them first if no registered range covers them. */
static int resident_ptr(const uint8_t *p, size_t bytes, const uint8_t **d)
{
    pthread_mutex_lock(&g_lock);
    Resident *r = find_range(p, bytes);
    int rc = OXH_OK;
    if (!r) rc = register_locked(p, bytes, &r);
    if (!rc) *d = r->d + (p - r->h);
    pthread_mutex_unlock(&g_lock);
    return rc;
}

/* ─── device staging buffers (inputs, activations, outputs) ───────────── */

typedef struct {
    void *p;
    size_t bytes;
} DevBuf;

static DevBuf g_dx, g_dact, g_dout, g_dprep;

/* Page-locked host staging for the decode-sized entry points: the caller's
 * vectors are ordinary pageable memory, and a copy between pageable memory and
 * the device is a synchronous two-step affair inside the runtime (about 12 us
 * each, three per call).  Staged through pinned buffers a call is one DMA in,
 * the launch, one DMA out (output and quantised activation together). */
typedef struct {
    void *p;
    size_t bytes;
} HostBuf;

static HostBuf g_hin, g_hout;

static int reserve_host(HostBuf *b, size_t bytes)
{
    if (b->bytes >= bytes) return OXH_OK;
    int rc = oxh_stream_sync(NULL);
    if (rc) return rc;
    if (b->p) {
        rc = oxh_host_free(b->p);
        b->p = NULL;
        b->bytes = 0;
        if (rc) return rc;
    }
    size_t want = bytes < (1u << 18) ? (1u << 18) : bytes + bytes / 4;
    rc = oxh_host_alloc(&b->p, want);
    if (rc) return rc;
    b->bytes = want;
    return OXH_OK;
}

static size_t align16(size_t n) { return (n + 15u) & ~(size_t)15u; }

static int reserve(DevBuf *b, size_t bytes)
{
    if (b->bytes >= bytes) return OXH_OK;
    int rc = oxh_stream_sync(NULL);
    if (rc) return rc;
    if (b->p) {
        rc = oxh_free(b->p);
        b->p = NULL;
        b->bytes = 0;
        if (rc) return rc;
    }
    size_t want = bytes < (1u << 20) ? (1u << 20) : bytes + bytes / 4;
    rc = oxh_malloc(&b->p, want);
    if (rc) return rc;
    b->bytes = want;
    return OXH_OK;
}

static bool mul_ok(size_t a, size_t b, size_t *out)
{
    if (a != 0 && b > SIZE_MAX / a) return false;
    *out = a * b;
    return true;
}

static int bad_arg(const char *what)
{
    oxh_set_error("invalid argument: %s%s", what, NULL);
    return OXH_ERR_ARG;
}

static int declined(const char *why)
{
    oxh_set_error("declined: %s%s", why, NULL);
    return OXH_DECLINED;
}

/* Integer-path eligibility of one matrix: 0 = declined, else activation kind. */
static int eligible(uint32_t qtype, size_t cols, size_t row_bytes)
{
    if (!oc_matvec_fused_enabled()) return 0;
    const int kind = oxh_act_kind(qtype, cols);
    if (!kind) return 0;
    const size_t expect = oxh_row_bytes(qtype, cols);
    if (expect == 0 || row_bytes != expect) return 0;
    return kind;
}

static int quantize(int kind, const float *d_x, size_t in_stride, size_t n_vec,
                    size_t cols, void *d_act)
{
    return kind == 2 ? oxh_quantize_q8_k(d_x, in_stride, n_vec, cols, d_act, NULL)
                     : oxh_quantize_q8_0(d_x, in_stride, n_vec, cols, d_act, NULL);
}

/* ─── oc_matvec_quantized ─────────────────────────────────────────────── */

static int mv_one(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp)
{
    const int kind = eligible(qtype, cols, row_bytes);
    if (!kind) return declined("type/shape/stride has no integer path (or it is switched off)");
    if (temp == NULL) return declined("temp is NULL");      /* matvec.c:865 */
    if (rows == 0) return OXH_OK;
    if (!data || !input || !output) return bad_arg("oxh_matvec_quantized: NULL pointer");
    size_t wbytes, obytes;
    if (!mul_ok(rows, row_bytes, &wbytes) || !mul_ok(rows, sizeof(float), &obytes) ||
        cols > SIZE_MAX / sizeof(float))
        return bad_arg("oxh_matvec_quantized: size overflow");
    const size_t abytes = oxh_act_bytes(qtype, cols);

    int rc = oxh_init(0);
    if (rc) return rc;
    const uint8_t *d_w;
    if ((rc = resident_ptr(data, wbytes, &d_w))) return rc;
    /* device and pinned-host images: [output rows][quantised activation] */
    const size_t act_off = align16(obytes);
    if ((rc = reserve(&g_dx, cols * sizeof(float)))) return rc;
    if ((rc = reserve(&g_dout, act_off + abytes))) return rc;
    if ((rc = reserve_host(&g_hin, cols * sizeof(float)))) return rc;
    if ((rc = reserve_host(&g_hout, act_off + abytes))) return rc;

    memcpy(g_hin.p, input, cols * sizeof(float));
    if ((rc = oxh_memcpy_h2d(g_dx.p, g_hin.p, cols * sizeof(float), NULL))) return rc;
    /* one launch: quantise the activation inside the GEMV kernel */
    OxhSegment seg = { d_w, (float *)g_dout.p, rows, 0, 0, NULL };
    if ((rc = oxh_gemv_segments_f32(qtype, &seg, 1, cols, (const float *)g_dx.p, cols,
                                    (uint8_t *)g_dout.p + act_off, 1, rows, NULL)))
        return rc;
    if ((rc = oxh_memcpy_d2h(g_hout.p, g_dout.p, act_off + abytes, NULL))) return rc;
    if ((rc = oxh_stream_sync(NULL))) return rc;
    memcpy(output, g_hout.p, obytes);
    memcpy(temp, (const uint8_t *)g_hout.p + act_off, abytes);
    return OXH_OK;
}

/* ─── grouped launches (fused / multi-input) ──────────────────────────── */

/* Shared body: n_outs matrices of one eligible type.  `inputs` has either one
 * vector (shared) or n_outs vectors. */
static int grouped(uint32_t qtype, const uint8_t *const *datas,
                   const size_t *rows, size_t cols, const size_t *row_bytes,
                   size_t n_outs, const float *const *inputs, size_t n_inputs,
                   float *const *outs)
{
    const size_t abytes = oxh_act_bytes(qtype, cols);
    size_t total_rows = 0;
    for (size_t k = 0; k < n_outs; k++) {
        if (rows[k] > SIZE_MAX / sizeof(float) - total_rows) return bad_arg("grouped: row overflow");
        total_rows += rows[k];
    }
    size_t xbytes, actbytes;
    if (!mul_ok(n_inputs, cols * sizeof(float), &xbytes) || !mul_ok(n_inputs, abytes, &actbytes))
        return bad_arg("grouped: size overflow");

    int rc = oxh_init(0);
    if (rc) return rc;
    if ((rc = reserve(&g_dx, xbytes))) return rc;
    if ((rc = reserve(&g_dact, actbytes))) return rc;
    if ((rc = reserve(&g_dout, total_rows * sizeof(float)))) return rc;
    if ((rc = reserve_host(&g_hin, xbytes))) return rc;
    if ((rc = reserve_host(&g_hout, total_rows * sizeof(float)))) return rc;

    for (size_t i = 0; i < n_inputs; i++) {
        if (!inputs[i]) return bad_arg("grouped: NULL input");
        memcpy((float *)g_hin.p + i * cols, inputs[i], cols * sizeof(float));
    }
    if ((rc = oxh_memcpy_h2d(g_dx.p, g_hin.p, xbytes, NULL))) return rc;
    enum { CHUNK = 32 };
    OxhSegment segs[CHUNK];
    size_t done_rows = 0;
    for (size_t k0 = 0; k0 < n_outs; k0 += CHUNK) {
        const size_t n = n_outs - k0 < CHUNK ? n_outs - k0 : CHUNK;
        for (size_t i = 0; i < n; i++) {
            const size_t k = k0 + i;
            size_t wbytes;
            if (!mul_ok(rows[k], row_bytes[k], &wbytes)) return bad_arg("grouped: size overflow");
            const uint8_t *d_w = NULL;
            if (rows[k]) {
                if (!datas[k] || !outs[k]) return bad_arg("grouped: NULL matrix pointer");
                if ((rc = resident_ptr(datas[k], wbytes, &d_w))) return rc;
            }
            segs[i].d_w = d_w;
            segs[i].d_out = (float *)g_dout.p + done_rows;
            segs[i].rows = rows[k];
            segs[i].act_first = n_inputs == 1 ? 0 : k;
            segs[i].n_vec = 0;
            segs[i].d_w_pair = NULL;
            done_rows += rows[k];
        }
        if ((rc = oxh_gemv_segments_f32(qtype, segs, n, cols, (const float *)g_dx.p, cols, NULL, 1, 0,
                                        NULL)))
            return rc;
    }
    if ((rc = oxh_memcpy_d2h(g_hout.p, g_dout.p, total_rows * sizeof(float), NULL))) return rc;
    if ((rc = oxh_stream_sync(NULL))) return rc;
    size_t off = 0;
    for (size_t k = 0; k < n_outs; k++) {
        if (rows[k]) memcpy(outs[k], (const float *)g_hout.p + off, rows[k] * sizeof(float));
        off += rows[k];
    }
    return OXH_OK;
}

static int mv_fused(const uint32_t *qtypes, const uint8_t *const *datas,
                               const size_t *rows, size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input, float *const *outs,
                               float *temp)
{
    if (n_outs == 0) return OXH_OK;
    if (!qtypes || !datas || !rows || !row_bytes || !outs || !input)
        return bad_arg("oxh_matvec_quantized_fused: NULL pointer");
    /* Every matrix must be runnable here, otherwise nothing is touched. */
    bool same = true;
    size_t total_rows = 0;
    for (size_t k = 0; k < n_outs; k++) {
        if (!eligible(qtypes[k], cols, row_bytes[k]))
            return declined("a matrix of the group has no integer path");
        if (qtypes[k] != qtypes[0]) same = false;
        total_rows += rows[k];
    }
    if (same && total_rows != 0) {
        /* matvec.c:1571-1573 */
        g_stats.activation_quantizations++;
        g_stats.parallel_dispatches++;
        return grouped(qtypes[0], datas, rows, cols, row_bytes, n_outs, &input, 1, outs);
    }
    /* mixed types (or an all-empty group): one call per matrix, matvec.c:1579-1593 */
    if (temp == NULL) return declined("temp is NULL");
    for (size_t k = 0; k < n_outs; k++) {
        int rc = mv_one(qtypes[k], datas[k], rows[k], cols, row_bytes[k],
                                      input, outs[k], temp);
        if (rc) return rc;
        g_stats.activation_quantizations++;
        g_stats.parallel_dispatches++;
        g_stats.fallback_calls++;
    }
    return OXH_OK;
}

static int mv_multi_input(const uint32_t *qtypes, const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs, float *const *outs,
                                     float *temp)
{
    if (n_outs == 0) return OXH_OK;
    if (!qtypes || !datas || !rows || !row_bytes || !outs || !inputs)
        return bad_arg("oxh_matvec_quantized_multi_input: NULL pointer");
    bool same = true;
    size_t total_rows = 0;
    for (size_t k = 0; k < n_outs; k++) {
        if (!eligible(qtypes[k], cols, row_bytes[k]))
            return declined("a matrix of the group has no integer path");
        if (qtypes[k] != qtypes[0]) same = false;
        total_rows += rows[k];
    }
    if (same && total_rows != 0) {
        /* matvec.c:1661-1662 */
        g_stats.activation_quantizations += n_outs;
        g_stats.parallel_dispatches++;
        return grouped(qtypes[0], datas, rows, cols, row_bytes, n_outs, inputs, n_outs, outs);
    }
    if (temp == NULL) return declined("temp is NULL");
    for (size_t k = 0; k < n_outs; k++) {
        int rc = mv_one(qtypes[k], datas[k], rows[k], cols, row_bytes[k],
                                      inputs[k], outs[k], temp);
        if (rc) return rc;
        g_stats.activation_quantizations++;
        g_stats.parallel_dispatches++;
        g_stats.fallback_calls++;
    }
    return OXH_OK;
}

/* ─── oc_matvec_quantized_batch ───────────────────────────────────────── */

static int mv_batch(uint32_t qtype, const uint8_t *data, size_t rows,
                               size_t cols, size_t row_bytes, const float *inputs,
                               size_t in_stride, float *outputs, size_t out_stride,
                               size_t n_vec, float *temp, uint8_t *act_scratch,
                               size_t act_bytes)
{
    (void)temp;
    if (n_vec == 0 || rows == 0) return OXH_OK;             /* matvec.c:1271 */
    const int kind = eligible(qtype, cols, row_bytes);
    if (!kind) return declined("type/shape/stride has no integer path (or it is switched off)");
    const size_t abytes = oxh_act_bytes(qtype, cols);
    /* matvec.c:1290-1292: no scratch, or not even one activation fits */
    if (act_scratch == NULL || abytes == 0 || act_bytes < abytes)
        return declined("activation scratch missing or smaller than one activation");
    if (!data || !inputs || !outputs) return bad_arg("oxh_matvec_quantized_batch: NULL pointer");
    if (in_stride < cols || out_stride < rows) return bad_arg("oxh_matvec_quantized_batch: stride < length");
    size_t wbytes, in_span, out_span, act_total;
    if (!mul_ok(rows, row_bytes, &wbytes) || !mul_ok(n_vec - 1, in_stride, &in_span) ||
        !mul_ok(n_vec - 1, out_stride, &out_span) || !mul_ok(n_vec, abytes, &act_total) ||
        in_span > SIZE_MAX / 4 - cols || out_span > SIZE_MAX / 4 - rows)
        return bad_arg("oxh_matvec_quantized_batch: size overflow");
    in_span += cols;
    out_span += rows;

    int rc = oxh_init(0);
    if (rc) return rc;
    const uint8_t *d_w;
    if ((rc = resident_ptr(data, wbytes, &d_w))) return rc;
    /* Inputs travel with their host stride; outputs come back packed
     * [n_vec][rows] and are scattered on the host so that nothing between
     * `rows` and `out_stride` is written (tests/test_matvec_batch.c:226-230). */
    size_t packed_out;
    if (!mul_ok(n_vec, rows * sizeof(float), &packed_out)) return bad_arg("batch: size overflow");
    if ((rc = reserve(&g_dx, in_span * sizeof(float)))) return rc;
    if ((rc = reserve(&g_dact, act_total))) return rc;
    if ((rc = reserve(&g_dout, packed_out))) return rc;
    if (in_stride == cols) {
        if ((rc = oxh_memcpy_h2d(g_dx.p, inputs, in_span * sizeof(float), NULL))) return rc;
    } else {
        for (size_t v = 0; v < n_vec; v++)
            if ((rc = oxh_memcpy_h2d((float *)g_dx.p + v * in_stride, inputs + v * in_stride,
                                     cols * sizeof(float), NULL)))
                return rc;
    }
    /* More vectors than the GEMV kernel keeps in flight: Q4_K, Q5_K and Q6_K go to the
     * int8-MFMA kernel behind a stand-alone quantiser launch; everything else
     * walks the batch in GEMV-sized slices with the quantisation fused in
     * (every output is the same dot either way). */
    if (n_vec > 8 && (qtype == OXH_Q4_K_S || qtype == OXH_Q4_K_M || qtype == OXH_Q5_K_S ||
                      qtype == OXH_Q5_K_M || qtype == OXH_Q6_K)) {
        if ((rc = quantize(kind, (const float *)g_dx.p, in_stride, n_vec, cols, g_dact.p))) return rc;
        if ((rc = oxh_mmq(qtype, d_w, rows, cols, g_dact.p, n_vec, (float *)g_dout.p, rows, NULL)))
            return rc;
    } else if (n_vec > 8 && (qtype == OXH_Q2_K || qtype == OXH_Q3_K_S || qtype == OXH_Q3_K_M ||
                             qtype == OXH_Q3_K_L)) {
        /* No MFMA kernel reads these blocks as they are.  Q3_K is exactly a Q6_K matrix in other bytes
         * and Q2_K widens to 210-byte blocks with scale * code in the 6-bit fields: rewrite the matrix
         * for this call, as the reference prepares its batch rows (oxk.c:734-745), and use that kernel */
        size_t prep_bytes;
        if (!mul_ok(rows, cols / OXH_QK_K * OXH_Q6_K_BYTES, &prep_bytes)) return bad_arg("batch: size overflow");
        if ((rc = reserve(&g_dprep, prep_bytes))) return rc;
        if (qtype == OXH_Q2_K) rc = oxh_q2_k_widen(d_w, rows, cols, g_dprep.p, NULL);
        else                   rc = oxh_q3_k_as_q6_k(d_w, rows, cols, g_dprep.p, NULL);
        if (rc) return rc;
        if ((rc = quantize(kind, (const float *)g_dx.p, in_stride, n_vec, cols, g_dact.p))) return rc;
        if ((rc = oxh_mmq(qtype == OXH_Q2_K ? OXH_Q2_K_WIDE : OXH_Q6_K, g_dprep.p, rows, cols, g_dact.p, n_vec,
                          (float *)g_dout.p, rows, NULL)))
            return rc;
    } else {
        size_t step = oxh_gemv_max_nvec_buffered(qtype, cols);
        if (step == 0) {
            oxh_set_error("batch: cols too wide for one workgroup%s%s", NULL, NULL);
            return OXH_ERR_TOO_WIDE;
        }
        for (size_t v0 = 0; v0 < n_vec; v0 += step) {
            const size_t m = n_vec - v0 < step ? n_vec - v0 : step;
            OxhSegment seg = { d_w, (float *)g_dout.p + v0 * rows, rows, v0, 0, NULL };
            /* with room for the quantised activations a slice of several vectors may run on
             * the matrix cores (same results; the library decides) */
            if ((rc = oxh_gemv_segments_f32(qtype, &seg, 1, cols, (const float *)g_dx.p, in_stride,
                                            g_dact.p, m, rows, NULL)))
                return rc;
        }
    }
    if (out_stride == rows) {
        if ((rc = oxh_memcpy_d2h(outputs, g_dout.p, packed_out, NULL))) return rc;
    } else {
        for (size_t v = 0; v < n_vec; v++)
            if ((rc = oxh_memcpy_d2h(outputs + v * out_stride, (float *)g_dout.p + v * rows,
                                     rows * sizeof(float), NULL)))
                return rc;
    }
    return oxh_stream_sync(NULL);
}

/* ─── public entry points: one call at a time ─────────────────────────── */

int oxh_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                         const float *input, float *output, float *temp)
{
    pthread_mutex_lock(&g_call);
    const int rc = mv_one(qtype, data, rows, cols, row_bytes, input, output, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_fused(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes, size_t n_outs, const float *input,
                               float *const *outs, float *temp)
{
    pthread_mutex_lock(&g_call);
    const int rc = mv_fused(qtypes, datas, rows, cols, row_bytes, n_outs, input, outs, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_multi_input(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                                     size_t cols, const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs, float *const *outs, float *temp)
{
    pthread_mutex_lock(&g_call);
    const int rc = mv_multi_input(qtypes, datas, rows, cols, row_bytes, n_outs, inputs, outs, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_batch(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride, float *outputs, size_t out_stride,
                               size_t n_vec, float *temp, uint8_t *act_scratch, size_t act_bytes)
{
    pthread_mutex_lock(&g_call);
    const int rc = mv_batch(qtype, data, rows, cols, row_bytes, inputs, in_stride, outputs, out_stride, n_vec,
                            temp, act_scratch, act_bytes);
    pthread_mutex_unlock(&g_call);
    return rc;
}

/* ─── the reference's own symbols ─────────────────────────────────────── */

static OxhDeclineHandler g_handler = NULL;
static void *g_handler_user = NULL;

void oxh_set_decline_handler(OxhDeclineHandler fn, void *user)
{
    g_handler = fn;
    g_handler_user = user;
}

static void not_ok(int which, int status)
{
    if (g_handler) {
        g_handler(which, status, g_handler_user);
        return;
    }
    fprintf(stderr, "liboxhip: oc_matvec entry %d failed with status %d: %s\n", which, status,
            oxh_last_error());
    abort();
}

void oc_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols,
                         size_t row_bytes, const float *input, float *output, float *temp)
{
    const int rc = oxh_matvec_quantized(qtype, data, rows, cols, row_bytes, input, output, temp);
    if (rc) not_ok(0, rc);
}

void oc_matvec_quantized_fused(const uint32_t *qtypes, const uint8_t *const *datas,
                               const size_t *rows, size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input, float *const *outs,
                               float *temp)
{
    const int rc = oxh_matvec_quantized_fused(qtypes, datas, rows, cols, row_bytes, n_outs,
                                              input, outs, temp);
    if (rc) not_ok(1, rc);
}

void oc_matvec_quantized_multi_input(const uint32_t *qtypes, const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs, float *const *outs,
                                     float *temp)
{
    const int rc = oxh_matvec_quantized_multi_input(qtypes, datas, rows, cols, row_bytes,
                                                    n_outs, inputs, outs, temp);
    if (rc) not_ok(2, rc);
}

void oc_matvec_quantized_batch(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols,
                               size_t row_bytes, const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec, float *temp,
                               uint8_t *act_scratch, size_t act_bytes)
{
    const int rc = oxh_matvec_quantized_batch(qtype, data, rows, cols, row_bytes, inputs,
                                              in_stride, outputs, out_stride, n_vec, temp,
                                              act_scratch, act_bytes);
    if (rc) not_ok(3, rc);
}
