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

/* Two kinds of entry.
 *   explicit  made by oxh_weight_register (and oxh_gguf_register_all): the caller promises the bytes do
 *             not change while registered; any pointer inside the range resolves (expert slices).
 *   automatic made on first sight of an unregistered matrix.  The reference reads the caller's host bytes
 *             on every call (oxidize-c/include/oxidize/matvec.h:45-52), so an address alone proves
 *             nothing: the heap hands the same address to the next model.  An automatic entry matches
 *             only the exact (pointer, byte count) it was made for, and every hit re-checks a
 *             fingerprint of the host bytes; on a mismatch the device copy is refreshed in place.  A new
 *             range that overlaps automatic entries replaces them.  Least recently used entries go once
 *             the cached bytes pass a budget.
 * OXH_WEIGHT_CACHE = sample (default), full (hash of every byte on every call), off (upload on every call).
 * What `sample` checks on every call over an automatic entry:
 *   - the length, the first and last 4 KiB and 128 strided 64-byte samples (a reused buffer, a model
 *     loaded over another: caught on the next call);
 *   - SLICES_PER_CALL slices of SLICE_BYTES, hashed whole and compared with the hash the slice had when
 *     the range was uploaded (every slice is hashed then), the slices taking turns from call to call.
 *     An edit of any size anywhere in the range is therefore caught after at most
 *     ceil(bytes / SLICE_BYTES / SLICES_PER_CALL) calls over that matrix, whatever it misses before.
 * A caller that patches weights in place and needs the very next call to see it calls
 * oxh_weight_unregister(ptr) (it drops automatic entries too), registers the range, or runs with `full`. */
#define SLICE_BYTES ((size_t)16384u)
#define SLICES_PER_CALL 2u
typedef struct {
    size_t off, rows, cols;     /* which sub-matrix of the range, and its shape */
    uint32_t form;              /* OXH_PREP_* */
    uint8_t *d;
    size_t bytes;
} Prepared;

typedef struct {
    const uint8_t *h;
    size_t bytes;
    uint8_t *d;
    bool automatic;
    uint64_t print;             /* automatic entries: fingerprint of the host bytes at upload */
    uint64_t *slice;            /* automatic entries in `sample` mode: hash of every SLICE_BYTES slice */
    size_t n_slice, cursor;     /* their count; the slice the next call re-checks first */
    uint64_t tick;              /* last use */
    Prepared *prep;             /* device-side rewrites of (parts of) this range, made on demand */
    size_t n_prep;
} Resident;

static pthread_mutex_t g_lock = PTHREAD_MUTEX_INITIALIZER;
/* Held for the whole of a matvec call, and by the calls that add or free device weights (taken before g_lock):
 * the staging buffers and the library's stream are shared by every call, so concurrent callers are
 * serialised (the reference's worker pool is one process-global resource too, include/oxidize/parallel.h:13-19). */
static pthread_mutex_t g_call = PTHREAD_MUTEX_INITIALIZER;
static Resident *g_res = NULL;
static size_t g_nres = 0, g_cap = 0;
static uint64_t g_tick = 0;
/* g_tick when the running call began: entries used since then back a launch of this call and must
 * stay where they are until it has finished */
static uint64_t g_call_tick = 0;
static size_t g_auto_bytes = 0;       /* automatic entries and their rewritten forms */
static size_t g_evictions = 0;

enum { CACHE_SAMPLE = 0, CACHE_FULL = 1, CACHE_OFF = 2 };

static int cache_mode(void)
{
    static int mode = -1;
    if (mode < 0) {
        const char *e = getenv("OXH_WEIGHT_CACHE");
        mode = CACHE_SAMPLE;
        if (e && !strcmp(e, "full")) mode = CACHE_FULL;
        else if (e && !strcmp(e, "off")) mode = CACHE_OFF;
    }
    return mode;
}

/* Budget for automatic entries and the rewritten forms kept with them: OXH_WEIGHT_CACHE_MB, else half of
 * the device memory that is free when the first automatic entry is made (other processes and the
 * caller's own buffers are then already counted out), and never less than 256 MiB. */
static size_t cache_budget(void)
{
    static size_t budget = 0;
    if (!budget) {
        const char *e = getenv("OXH_WEIGHT_CACHE_MB");
        unsigned long long mb = e && *e ? strtoull(e, NULL, 10) : 0ull;
        if (mb != 0ull && mb <= (1ull << 24)) {
            budget = (size_t)mb << 20;
        } else {
            size_t free_b = 0, total_b = 0;
            if (oxh_mem_info(&free_b, &total_b) != OXH_OK || free_b == 0) free_b = (size_t)128u << 30;
            budget = free_b / 2u;
            if (budget < ((size_t)256u << 20)) budget = (size_t)256u << 20;
        }
    }
    return budget;
}

static uint64_t mix64(uint64_t h, uint64_t v)
{
    h ^= v;
    h *= 0x9E3779B97F4A7C15ull;
    return h ^ (h >> 29);
}

/* Four chains side by side (a multiply's latency apart each), folded at the end: the fingerprint is
 * taken on every call over unregistered weights, and one chain alone runs at a fifth of this rate. */
static uint64_t hash_bytes(uint64_t h, const uint8_t *p, size_t n)
{
    size_t i = 0;
    if (n >= 64) {
        uint64_t a = h, b = h ^ 0xA5A5A5A5A5A5A5A5ull, c = h + 0x1234567ull, d = ~h;
        for (; i + 32 <= n; i += 32) {
            uint64_t v[4];
            memcpy(v, p + i, 32);
            a = mix64(a, v[0]);
            b = mix64(b, v[1]);
            c = mix64(c, v[2]);
            d = mix64(d, v[3]);
        }
        h = mix64(mix64(mix64(a, b), c), d);
    }
    for (; i + 8 <= n; i += 8) {
        uint64_t v;
        memcpy(&v, p + i, 8);
        h = mix64(h, v);
    }
    if (i < n) {
        uint64_t v = 0;
        memcpy(&v, p + i, n - i);
        h = mix64(h, v);
    }
    return h;
}

static uint64_t host_print(const uint8_t *p, size_t bytes)
{
    uint64_t h = mix64(0x6F78685F77746673ull, (uint64_t)bytes);
    if (cache_mode() == CACHE_FULL || bytes <= 16384u) return hash_bytes(h, p, bytes);
    h = hash_bytes(h, p, 4096u);
    h = hash_bytes(h, p + bytes - 4096u, 4096u);
    const size_t span = bytes - 8192u - 64u, n = 128u;
    for (size_t i = 0; i < n; i++)
        h = hash_bytes(h, p + 4096u + (size_t)(((unsigned __int128)span * i) / (n - 1u)), 64u);
    return h;
}

/* Hash of slice i of the range (the last one may be short). */
static uint64_t slice_print(const uint8_t *p, size_t bytes, size_t i)
{
    const size_t at = i * SLICE_BYTES, n = bytes - at < SLICE_BYTES ? bytes - at : SLICE_BYTES;
    return hash_bytes(mix64(0x736C696365ull, (uint64_t)i), p + at, n);
}

/* The per-slice hashes of an automatic entry, taken when its bytes go to the device (`sample` mode and
 * ranges the fingerprint does not cover whole).  Without memory for the table the entry simply has none. */
static void slices_take(Resident *r)
{
    free(r->slice);
    r->slice = NULL;
    r->n_slice = r->cursor = 0;
    if (!r->automatic || cache_mode() != CACHE_SAMPLE || r->bytes <= 16384u) return;
    const size_t n = (r->bytes + SLICE_BYTES - 1u) / SLICE_BYTES;
    r->slice = (uint64_t *)malloc(n * sizeof *r->slice);
    if (!r->slice) return;
    for (size_t i = 0; i < n; i++) r->slice[i] = slice_print(r->h, r->bytes, i);
    r->n_slice = n;
}

/* This call's turn of the rotating check: true when every slice looked at still has its hash. */
static bool slices_hold(Resident *r)
{
    for (unsigned k = 0; k < SLICES_PER_CALL && r->n_slice; k++) {
        const size_t i = r->cursor;
        r->cursor = (i + 1u) % r->n_slice;
        if (slice_print(r->h, r->bytes, i) != r->slice[i]) return false;
    }
    return true;
}

static void drop_prepared(Resident *r)
{
    for (size_t i = 0; i < r->n_prep; i++) {
        if (r->automatic) g_auto_bytes -= r->prep[i].bytes;
        (void)oxh_free(r->prep[i].d);
    }
    free(r->prep);
    r->prep = NULL;
    r->n_prep = 0;
}

/* caller holds g_lock and has synchronised the library's stream */
static int drop_entry(size_t i)
{
    Resident *r = &g_res[i];
    drop_prepared(r);
    if (r->automatic) g_auto_bytes -= r->bytes;
    free(r->slice);
    const int rc = oxh_free(r->d);
    g_res[i] = g_res[g_nres - 1];
    g_nres--;
    return rc;
}

static bool overlaps(const Resident *r, const uint8_t *p, size_t bytes)
{
    return p < r->h + r->bytes && r->h < p + bytes;
}

/* explicit entries: p .. p+bytes lies inside the range (the end of one tensor is the start of the next
 * in a mapped model file, so p itself must be inside) */
static Resident *find_explicit(const uint8_t *p, size_t bytes)
{
    for (size_t i = 0; i < g_nres; i++) {
        Resident *r = &g_res[i];
        if (!r->automatic && p >= r->h && (size_t)(p - r->h) < r->bytes &&
            bytes <= r->bytes - (size_t)(p - r->h))
            return r;
    }
    return NULL;
}

static Resident *find_automatic(const uint8_t *p, size_t bytes)
{
    for (size_t i = 0; i < g_nres; i++)
        if (g_res[i].automatic && g_res[i].h == p && g_res[i].bytes == bytes) return &g_res[i];
    return NULL;
}

static int upload(uint8_t *d, const uint8_t *h, size_t bytes)
{
    int rc = oxh_memcpy_h2d(d, h, bytes, NULL);
    if (!rc) rc = oxh_stream_sync(NULL);
    return rc;
}

/* Drops the least recently used automatic entry that the running call does not use (and is not `keep`).
 * False when there is none.  The caller holds g_lock. */
static bool evict_one(const Resident *keep, bool *synced)
{
    size_t lru = g_nres;
    for (size_t i = 0; i < g_nres; i++)
        if (g_res[i].automatic && &g_res[i] != keep && g_res[i].tick <= g_call_tick &&
            (lru == g_nres || g_res[i].tick < g_res[lru].tick)) lru = i;
    if (lru == g_nres) return false;
    if (!*synced) {
        if (oxh_stream_sync(NULL) != OXH_OK) return false;
        *synced = true;
    }
    (void)drop_entry(lru);
    return true;
}

/* Device memory for the registry.  The budget is a guess about what the device has left for us; when
 * the allocation itself fails, automatic entries are given up, least recently used first, until it
 * succeeds or none is left.  drop_entry moves the last entry into the freed slot, so `keep` (an entry
 * the caller goes on using) is passed by address and re-found by the caller if it needs to. */
static int alloc_evicting(void **d, size_t bytes, const uint8_t *keep_h, bool *synced)
{
    int rc = oxh_malloc(d, bytes);
    while (rc == OXH_ERR_NOMEM) {
        const Resident *keep = NULL;
        for (size_t i = 0; i < g_nres && keep_h; i++)
            if (g_res[i].h == keep_h) keep = &g_res[i];
        if (!evict_one(keep, synced)) break;
        g_evictions++;
        rc = oxh_malloc(d, bytes);
    }
    return rc;
}

static int register_locked(const uint8_t *h, size_t bytes, bool automatic, Resident **out)
{
    /* whatever automatic entry shares bytes with the new range describes memory that now holds
     * something else */
    bool synced = false;
    for (size_t i = 0; i < g_nres;) {
        if (g_res[i].automatic && overlaps(&g_res[i], h, bytes)) {
            if (g_res[i].tick > g_call_tick) {
                oxh_set_error("invalid argument: %s%s", "two matrices of one call overlap in host memory", NULL);
                return OXH_ERR_ARG;
            }
            if (!synced) { int rc = oxh_stream_sync(NULL); if (rc) return rc; synced = true; }
            (void)drop_entry(i);
        } else {
            i++;
        }
    }
    if (automatic) {
        while (g_auto_bytes && g_auto_bytes + bytes > cache_budget()) {
            if (!evict_one(NULL, &synced)) break;
            g_evictions++;
        }
    }
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
    int rc = alloc_evicting(&d, bytes, NULL, &synced);
    if (rc) return rc;
    const uint64_t print = automatic ? host_print(h, bytes) : 0u;
    if ((rc = upload((uint8_t *)d, h, bytes))) {
        oxh_free(d);
        return rc;
    }
    Resident *r = &g_res[g_nres++];
    memset(r, 0, sizeof *r);
    r->h = h;
    r->bytes = bytes;
    r->d = (uint8_t *)d;
    r->automatic = automatic;
    r->print = print;
    r->tick = ++g_tick;
    if (automatic) g_auto_bytes += bytes;
    slices_take(r);
    if (out) *out = r;
    return OXH_OK;
}

int oxh_weight_register(const void *h_data, size_t bytes)
{
    if (!h_data || bytes == 0) {
        oxh_set_error("invalid argument: %s%s", "oxh_weight_register: empty range", NULL);
        return OXH_ERR_ARG;
    }
    int rc = oxh_init(0);
    if (rc) return rc;
    pthread_mutex_lock(&g_call);
    g_call_tick = g_tick;
    pthread_mutex_lock(&g_lock);
    if (!find_explicit((const uint8_t *)h_data, bytes))
        rc = register_locked((const uint8_t *)h_data, bytes, false, NULL);
    pthread_mutex_unlock(&g_lock);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_weight_unregister(const void *h_data)
{
    int rc = OXH_OK;
    const uint8_t *p = (const uint8_t *)h_data;
    pthread_mutex_lock(&g_call);
    pthread_mutex_lock(&g_lock);
    bool synced = false;
    for (size_t i = 0; i < g_nres;) {
        const Resident *r = &g_res[i];
        if (p >= r->h && (size_t)(p - r->h) < r->bytes) {
            if (!synced) { rc = oxh_stream_sync(NULL); synced = true; }
            const int r2 = drop_entry(i);
            if (!rc) rc = r2;
        } else {
            i++;
        }
    }
    pthread_mutex_unlock(&g_lock);
    pthread_mutex_unlock(&g_call);
    return rc;
}

static int clear_locked(void)
{
    int rc = g_nres ? oxh_stream_sync(NULL) : OXH_OK;
    while (g_nres) {
        const int r = drop_entry(g_nres - 1);
        if (!rc) rc = r;
    }
    g_auto_bytes = 0;
    return rc;
}

int oxh_weight_clear(void)
{
    pthread_mutex_lock(&g_call);
    pthread_mutex_lock(&g_lock);
    const int rc = clear_locked();
    pthread_mutex_unlock(&g_lock);
    pthread_mutex_unlock(&g_call);
    return rc;
}

const void *oxh_weight_device_ptr(const void *h_data)
{
    const uint8_t *p = (const uint8_t *)h_data;
    pthread_mutex_lock(&g_lock);
    const Resident *r = find_explicit(p, 0);
    if (!r)
        for (size_t i = 0; i < g_nres && !r; i++)
            if (g_res[i].automatic && p >= g_res[i].h && (size_t)(p - g_res[i].h) < g_res[i].bytes) r = &g_res[i];
    const void *d = r ? r->d + (p - r->h) : NULL;
    pthread_mutex_unlock(&g_lock);
    return d;
}

int oxh_weight_stats(size_t *n_explicit, size_t *n_automatic, size_t *automatic_bytes, size_t *refreshes);
static size_t g_refreshes = 0;

int oxh_weight_stats(size_t *n_explicit, size_t *n_automatic, size_t *automatic_bytes, size_t *refreshes)
{
    pthread_mutex_lock(&g_lock);
    size_t ne = 0, na = 0;
    for (size_t i = 0; i < g_nres; i++) {
        if (g_res[i].automatic) na++;
        else ne++;
    }
    if (n_explicit) *n_explicit = ne;
    if (n_automatic) *n_automatic = na;
    if (automatic_bytes) *automatic_bytes = g_auto_bytes;
    if (refreshes) *refreshes = g_refreshes;
    pthread_mutex_unlock(&g_lock);
    return OXH_OK;
}

size_t oxh_weight_evictions(void)
{
    pthread_mutex_lock(&g_lock);
    const size_t n = g_evictions;
    pthread_mutex_unlock(&g_lock);
    return n;
}

/* Device address of `bytes` of weights starting at host pointer p.  Registered ranges resolve without
 * looking at the host bytes; anything else is uploaded on first sight and re-validated on every later
 * call (see the registry's header; with OXH_WEIGHT_CACHE=off every hit counts as changed and is uploaded
 * again).  The caller holds g_call.  `entry`, when not NULL, receives the registry entry. */
static int resident_ptr(const uint8_t *p, size_t bytes, const uint8_t **d, Resident **entry)
{
    pthread_mutex_lock(&g_lock);
    int rc = OXH_OK;
    if (entry) *entry = NULL;
    Resident *r = find_explicit(p, bytes);
    if (!r) {
        r = find_automatic(p, bytes);
        if (r && r->tick <= g_call_tick) {         /* validated once per call is enough */
            const uint64_t now = cache_mode() == CACHE_OFF ? ~r->print : host_print(p, bytes);
            if (now != r->print || !slices_hold(r)) {
                /* same address and size, other contents: the caller reused or patched the memory */
                drop_prepared(r);
                rc = oxh_stream_sync(NULL);
                if (!rc) rc = upload(r->d, p, bytes);
                /* a copy that did not arrive must not pass for the new contents on the next call */
                r->print = (rc || cache_mode() == CACHE_OFF) ? ~now : now;
                if (!rc) slices_take(r);
                g_refreshes++;
            }
        } else if (!r) {
            rc = register_locked(p, bytes, true, &r);
        }
    }
    if (!rc) {
        r->tick = ++g_tick;
        *d = r->d + (p - r->h);
        if (entry) *entry = r;
    }
    pthread_mutex_unlock(&g_lock);
    return rc;
}

static bool mul_ok(size_t a, size_t b, size_t *out);
static int bad_arg(const char *what);

/* Forms a resident matrix can be rewritten into, once, on the device. */
#define OXH_PREP_Q3K_AS_Q6K 1u      /* oxh_q3_k_as_q6_k */
#define OXH_PREP_Q2K_WIDE   2u      /* oxh_q2_k_widen   */
#define OXH_PREP_Q6K_G8     3u      /* oxh_q6_k_group   */
#define OXH_PREP_Q80_T16    4u      /* oxh_tile16 of a Q8_0 matrix */

/* The rewritten form of the rows x cols matrix at host pointer p inside registry entry r, made on first
 * use and kept with the entry (the reference prepares its batch rows once per matrix as well,
 * oxidize-c/src/compute/oxk.c:316-366, :734-745).  It goes when the entry goes or is refreshed.  The
 * caller holds g_call. */
static int prepared_ptr(Resident *r, const uint8_t *p, size_t rows, size_t cols, uint32_t form,
                        const uint8_t **d)
{
    const size_t off = (size_t)(p - r->h);
    for (size_t i = 0; i < r->n_prep; i++) {
        const Prepared *q = &r->prep[i];
        if (q->off == off && q->rows == rows && q->cols == cols && q->form == form) {
            *d = q->d;
            return OXH_OK;
        }
    }
    size_t bytes;
    if (form == OXH_PREP_Q80_T16) {
        bytes = oxh_tile16_bytes(OXH_Q8_0, rows, cols);
        if (!bytes) return bad_arg("prepared form: no tile-major form of this width");
    } else if (!mul_ok(rows, cols / OXH_QK_K * OXH_Q6_K_BYTES, &bytes))
        return bad_arg("prepared form: size overflow");
    Prepared *np = (Prepared *)realloc(r->prep, (r->n_prep + 1) * sizeof *np);
    if (!np) {
        oxh_set_error("out of host memory growing the weight registry%s%s", NULL, NULL);
        return OXH_ERR_NOMEM;
    }
    r->prep = np;
    void *nd = NULL;
    /* Giving up other entries for the memory may move this one inside the table (never drop it: the
     * running call uses it), so it is looked up again by its range. */
    const uint8_t *const rh = r->h;
    const size_t rbytes = r->bytes;
    const bool rauto = r->automatic;
    pthread_mutex_lock(&g_lock);
    bool synced = false;
    if (rauto)
        while (g_auto_bytes + bytes > cache_budget() && evict_one(r, &synced)) {
            g_evictions++;
            for (size_t i = 0; i < g_nres; i++)
                if (g_res[i].h == rh && g_res[i].bytes == rbytes && g_res[i].automatic == rauto) r = &g_res[i];
        }
    int rc = alloc_evicting(&nd, bytes, rh, &synced);
    for (size_t i = 0; i < g_nres; i++)
        if (g_res[i].h == rh && g_res[i].bytes == rbytes && g_res[i].automatic == rauto) r = &g_res[i];
    pthread_mutex_unlock(&g_lock);
    if (rc) return rc;
    if (form == OXH_PREP_Q80_T16)     rc = oxh_tile16(OXH_Q8_0, r->d + off, rows, cols, nd, NULL);
    else if (form == OXH_PREP_Q2K_WIDE) rc = oxh_q2_k_widen(r->d + off, rows, cols, nd, NULL);
    else if (form == OXH_PREP_Q6K_G8) rc = oxh_q6_k_group(r->d + off, rows, cols, nd, NULL);
    else                              rc = oxh_q3_k_as_q6_k(r->d + off, rows, cols, nd, NULL);
    if (rc) {
        (void)oxh_free(nd);
        return rc;
    }
    Prepared *q = &r->prep[r->n_prep++];
    q->off = off; q->rows = rows; q->cols = cols; q->form = form; q->d = (uint8_t *)nd; q->bytes = bytes;
    if (r->automatic) g_auto_bytes += bytes;
    *d = q->d;
    return OXH_OK;
}

/* Q6_K for the decode kernels: the regrouped copy (oxh_q6_k_group), made the first time a GEMV runs over
 * the matrix and kept with its registry entry next to the file layout, which the matrix-core kernel and
 * the row lookup go on reading.  OXH_Q6K_GROUPED=0 switches it off; a matrix whose cols are not a
 * multiple of 2048, or for which there is no memory left, stays on the file layout, and so do
 * unregistered weights under OXH_WEIGHT_CACHE=off. */
static int q6k_grouped_enabled(void)
{
    static int cached = -1;
    if (cached < 0) {
        const char *e = getenv("OXH_Q6K_GROUPED");
        cached = (e && e[0] == '0') ? 0 : 1;
    }
    return cached;
}

static void decode_form(uint32_t *qtype, Resident *entry, const uint8_t *data, size_t rows, size_t cols,
                        const uint8_t **d_w)
{
    if (*qtype != OXH_Q6_K || !entry || rows == 0 || cols % (8u * OXH_QK_K) || !q6k_grouped_enabled()) return;
    /* a cache that uploads the bytes again on every call would regroup them on every call as well */
    if (entry->automatic && cache_mode() == CACHE_OFF) return;
    const uint8_t *d;
    if (prepared_ptr(entry, data, rows, cols, OXH_PREP_Q6K_G8, &d) != OXH_OK) return;
    *d_w = d;
    *qtype = OXH_Q6_K_G8;
}

/* Q8_0 for batches of 2 to 16: the tile-major copy (oxh_tile16), made the first time such a batch runs
 * over a matrix with enough rows to fill the device one 16-row group per wave (sixteen groups per compute
 * unit; a vocabulary head) and kept with its registry entry next to the file layout, which single
 * vectors and longer batches go on reading.  OXH_Q80_TILED=0 switches it off; no memory left, a width
 * that is not a multiple of 128, or OXH_WEIGHT_CACHE=off leave the call on the file layout. */
static int q80_tiled_enabled(void)
{
    static int cached = -1;
    if (cached < 0) {
        const char *e = getenv("OXH_Q80_TILED");
        cached = (e && e[0] == '0') ? 0 : 1;
    }
    return cached;
}

static void batch_form(uint32_t *qtype, Resident *entry, const uint8_t *data, size_t rows, size_t cols, size_t n_vec,
                       const uint8_t **d_w)
{
    const int n_cu = oxh_internal_n_cu();
    if (*qtype != OXH_Q8_0 || !entry || n_vec < 2 || n_vec > 16 || cols % (4u * OXH_QK8_0) || !q80_tiled_enabled() ||
        n_cu <= 0 || rows / 16u < 16u * (size_t)n_cu || cols / OXH_QK8_0 * 576u > 160u * 1024u)
        return;                                     /* the last: what the tile-major kernel's workgroup holds in LDS */
    if (entry->automatic && cache_mode() == CACHE_OFF) return;
    const uint8_t *d;
    if (prepared_ptr(entry, data, rows, cols, OXH_PREP_Q80_T16, &d) != OXH_OK) return;
    *d_w = d;
    *qtype = OXH_Q8_0_T16;
}

/* ─── device staging buffers (inputs, activations, outputs) ───────────── */

typedef struct {
    void *p;
    size_t bytes;
} DevBuf;

static DevBuf g_dx, g_dact, g_dout, g_dsplit;

/* Page-locked host staging for the decode-sized entry points: the caller's
 * vectors are ordinary pageable memory, and a copy between pageable memory and
 * the device is a synchronous two-step affair inside the runtime (about 12 us
 * each, three per call).  Page-locked memory the device reads and writes in
 * place, so up to HOST_DIRECT_MAX bytes a call's input is pulled out of it by a
 * copy kernel ahead of the GEMV launch, and the GEMV kernel stores its rows (and
 * the quantised activation) straight into it: two launches and a wait, where a
 * DMA each way costs 7-8 us more per call than the 5-15 us the kernel runs.
 * (Letting the GEMV read its input in place would not do: every workgroup
 * reads the whole vector, 256 trips over the bus.)  Larger transfers keep the
 * DMA engines. */
#define HOST_DIRECT_MAX ((size_t)1 << 20)
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

/* oxh_shutdown: forget every device and pinned buffer made under the state that is going away. */
void oxh_internal_host_reset(void)
{
    pthread_mutex_lock(&g_call);
    pthread_mutex_lock(&g_lock);
    (void)clear_locked();
    pthread_mutex_unlock(&g_lock);
    DevBuf *dv[] = { &g_dx, &g_dact, &g_dout, &g_dsplit };
    for (size_t i = 0; i < sizeof dv / sizeof dv[0]; i++) {
        if (dv[i]->p) (void)oxh_free(dv[i]->p);
        dv[i]->p = NULL;
        dv[i]->bytes = 0;
    }
    HostBuf *hv[] = { &g_hin, &g_hout };
    for (size_t i = 0; i < sizeof hv / sizeof hv[0]; i++) {
        if (hv[i]->p) (void)oxh_host_free(hv[i]->p);
        hv[i]->p = NULL;
        hv[i]->bytes = 0;
    }
    pthread_mutex_unlock(&g_call);
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

/* The first `bytes` of the pinned input image to the device input buffer. */
static int push_input(size_t bytes)
{
    if (bytes <= HOST_DIRECT_MAX) return oxh_internal_copy16(g_dx.p, g_hin.p, align16(bytes), NULL);
    return oxh_memcpy_h2d(g_dx.p, g_hin.p, bytes, NULL);
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

/* OXH_MMQ_RELAXED=1: prefill batches take the five-operation float step (within 1e-5*|exact| + 2e-6 of the
 * outputs' root mean square of the exact outputs, no longer bit-identical to the CPU path); off by default */
static int mmq_relaxed_enabled(void)
{
    static int cached = -1;
    if (cached < 0) {
        const char *e = getenv("OXH_MMQ_RELAXED");
        cached = (e && e[0] == '1') ? 1 : 0;
    }
    return cached;
}

/* OXH_MMQ_SPLIT_MIN_NV: activations from which a batch over few rows and many columns shares its tiles'
 * columns between workgroups (7; 0 = never) */
static size_t mmq_split_min_nv(void)
{
    static long cached = -1;
    if (cached < 0) {
        const char *e = getenv("OXH_MMQ_SPLIT_MIN_NV");
        char *end = NULL;
        const long v = (e && *e) ? strtol(e, &end, 10) : 7;
        cached = (e && *e && (end == e || v < 0 || v > 64)) ? 7 : v;
    }
    return cached == 0 ? SIZE_MAX : (size_t)cached;
}

static int quantize(int kind, const float *d_x, size_t in_stride, size_t n_vec,
                    size_t cols, void *d_act)
{
    return kind == 2 ? oxh_quantize_q8_k(d_x, in_stride, n_vec, cols, d_act, NULL)
                     : oxh_quantize_q8_0(d_x, in_stride, n_vec, cols, d_act, NULL);
}

/* ─── oc_matvec_quantized ─────────────────────────────────────────────── */

/* OXH_F32_PATH_TYPES=1: oc_matvec_quantized over IQ4_NL / IQ4_XS runs on the device (weights expanded
 * against the f32 input, oxh_gemv_segments_f32).  Off by default: the reference's CPU code takes these
 * types through its dequantise loop (matvec.c:886-907), whose results this path matches to f32 rounding,
 * not to the bit, so the default hands them back like every other type of that loop. */
static int f32_path_enabled(void)
{
    static int cached = -1;
    if (cached < 0) {
        const char *e = getenv("OXH_F32_PATH_TYPES");
        cached = (e && e[0] && e[0] != '0') ? 1 : 0;
    }
    return cached;
}

static int mv_one_f32_path(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                           const float *input, float *output)
{
    if (rows == 0) return OXH_OK;
    if (!data || !input || !output) return bad_arg("oxh_matvec_quantized: NULL pointer");
    size_t wbytes, obytes;
    if (!mul_ok(rows, row_bytes, &wbytes) || !mul_ok(rows, sizeof(float), &obytes) || cols > SIZE_MAX / sizeof(float))
        return bad_arg("oxh_matvec_quantized: size overflow");
    int rc = oxh_init(0);
    if (rc) return rc;
    const uint8_t *d_w;
    if ((rc = resident_ptr(data, wbytes, &d_w, NULL))) return rc;
    if ((rc = reserve(&g_dx, cols * sizeof(float)))) return rc;
    if ((rc = reserve(&g_dout, obytes))) return rc;
    if ((rc = reserve_host(&g_hin, cols * sizeof(float)))) return rc;
    if ((rc = reserve_host(&g_hout, obytes))) return rc;
    memcpy(g_hin.p, input, cols * sizeof(float));
    if ((rc = push_input(cols * sizeof(float)))) return rc;
    const bool direct = obytes <= HOST_DIRECT_MAX;
    OxhSegment seg = { d_w, (float *)(direct ? g_hout.p : g_dout.p), rows, 0, 0, NULL };
    if ((rc = oxh_gemv_segments_f32(qtype, &seg, 1, cols, (const float *)g_dx.p, cols, NULL, 1, rows, NULL)))
        return rc;
    if (!direct && (rc = oxh_memcpy_d2h(g_hout.p, g_dout.p, obytes, NULL))) return rc;
    if ((rc = oxh_stream_sync(NULL))) return rc;
    memcpy(output, g_hout.p, obytes);
    return OXH_OK;
}

static int mv_one(uint32_t qtype, const uint8_t *data, size_t rows,
                         size_t cols, size_t row_bytes, const float *input,
                         float *output, float *temp)
{
    const int kind = eligible(qtype, cols, row_bytes);
    if (!kind && f32_path_enabled() && row_bytes != 0 && oxh_f32_path_row_bytes(qtype, cols) == row_bytes)
        return mv_one_f32_path(qtype, data, rows, cols, row_bytes, input, output);
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
    Resident *entry = NULL;
    if ((rc = resident_ptr(data, wbytes, &d_w, &entry))) return rc;
    uint32_t run_type = qtype;
    decode_form(&run_type, entry, data, rows, cols, &d_w);
    /* device and pinned-host images: [output rows][quantised activation] */
    const size_t act_off = align16(obytes);
    if ((rc = reserve(&g_dx, cols * sizeof(float)))) return rc;
    if ((rc = reserve(&g_dout, act_off + abytes))) return rc;
    if ((rc = reserve_host(&g_hin, cols * sizeof(float)))) return rc;
    if ((rc = reserve_host(&g_hout, act_off + abytes))) return rc;

    memcpy(g_hin.p, input, cols * sizeof(float));
    if ((rc = push_input(cols * sizeof(float)))) return rc;
    /* one launch: quantise the activation inside the GEMV kernel */
    const bool direct = act_off + abytes <= HOST_DIRECT_MAX;
    uint8_t *dst = direct ? (uint8_t *)g_hout.p : (uint8_t *)g_dout.p;
    OxhSegment seg = { d_w, (float *)dst, rows, 0, 0, NULL };
    if ((rc = oxh_gemv_segments_f32(run_type, &seg, 1, cols, (const float *)g_dx.p, cols,
                                    dst + act_off, 1, rows, NULL)))
        return rc;
    if (!direct && (rc = oxh_memcpy_d2h(g_hout.p, g_dout.p, act_off + abytes, NULL))) return rc;
    if ((rc = oxh_stream_sync(NULL))) return rc;
    memcpy(output, g_hout.p, obytes);
    memcpy(temp, (const uint8_t *)g_hout.p + act_off, abytes);
    /* Q4_0 and AL5: the reference leaves the int32 sum of every 32-value activation block behind the
     * blocks, from the next multiple of four bytes on (matvec.c:198-227, :866-877); temp has the room
     * (34 + 4 bytes per 32 floats) */
    if (qtype == OXH_Q4_0 || qtype == OXH_AL5) {
        uint8_t *act = (uint8_t *)temp;
        const size_t blocks = cols / 32u, at = (abytes + 3u) & ~(size_t)3u;
        for (size_t b = 0; b < blocks; b++) {
            const int8_t *q = (const int8_t *)(act + b * 34u + 2u);
            int32_t sum = 0;
            for (int i = 0; i < 32; i++) sum += q[i];
            memcpy(act + at + 4u * b, &sum, sizeof sum);
        }
    }
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
    if ((rc = push_input(xbytes))) return rc;
    const bool direct = total_rows * sizeof(float) <= HOST_DIRECT_MAX;
    float *dst = direct ? (float *)g_hout.p : (float *)g_dout.p;
    enum { CHUNK = 32 };
    OxhSegment segs[CHUNK];
    size_t done_rows = 0;
    for (size_t k0 = 0; k0 < n_outs; k0 += CHUNK) {
        const size_t n = n_outs - k0 < CHUNK ? n_outs - k0 : CHUNK;
        const uint8_t *d_plain[CHUNK], *d_alt[CHUNK];
        bool all_alt = qtype == OXH_Q6_K;
        for (size_t i = 0; i < n; i++) {
            const size_t k = k0 + i;
            size_t wbytes;
            if (!mul_ok(rows[k], row_bytes[k], &wbytes)) return bad_arg("grouped: size overflow");
            const uint8_t *d_w = NULL;
            Resident *entry = NULL;
            if (rows[k]) {
                if (!datas[k] || !outs[k]) return bad_arg("grouped: NULL matrix pointer");
                if ((rc = resident_ptr(datas[k], wbytes, &d_w, &entry))) return rc;
            }
            /* one launch has one weight type: the regrouped Q6_K copies are used when every matrix of
             * the launch has one */
            d_plain[i] = d_alt[i] = d_w;
            if (all_alt && rows[k]) {
                uint32_t t = qtype;
                decode_form(&t, entry, datas[k], rows[k], cols, &d_alt[i]);
                if (t != OXH_Q6_K_G8) all_alt = false;
            }
            segs[i].d_w = d_w;
            segs[i].d_out = dst + done_rows;
            segs[i].rows = rows[k];
            segs[i].act_first = n_inputs == 1 ? 0 : k;
            segs[i].n_vec = 0;
            segs[i].d_w_pair = NULL;
            done_rows += rows[k];
        }
        for (size_t i = 0; i < n; i++) segs[i].d_w = all_alt ? d_alt[i] : d_plain[i];
        if ((rc = oxh_gemv_segments_f32(all_alt ? OXH_Q6_K_G8 : qtype, segs, n, cols, (const float *)g_dx.p, cols,
                                        NULL, 1, 0, NULL)))
            return rc;
    }
    if (!direct && (rc = oxh_memcpy_d2h(g_hout.p, g_dout.p, total_rows * sizeof(float), NULL))) return rc;
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

    int rc = oxh_init(0);
    if (rc) return rc;
    const uint8_t *d_w;
    Resident *entry;
    if ((rc = resident_ptr(data, wbytes, &d_w, &entry))) return rc;
    /* Inputs arrive packed [n_vec][cols] on the device and outputs come back packed [n_vec][rows]: one
     * copy each way, two-dimensional when the host strides are padded, so that nothing between `rows`
     * and `out_stride` is written (tests/test_matvec_batch.c:226-230). */
    size_t packed_in, packed_out;
    if (!mul_ok(n_vec, cols * sizeof(float), &packed_in) || !mul_ok(n_vec, rows * sizeof(float), &packed_out))
        return bad_arg("batch: size overflow");
    if ((rc = reserve(&g_dx, packed_in))) return rc;
    if ((rc = reserve(&g_dact, act_total))) return rc;
    if ((rc = reserve(&g_dout, packed_out))) return rc;
    /* a few vectors travel like a single one: through the page-locked images, in place */
    const bool in_direct = packed_in <= HOST_DIRECT_MAX, out_direct = packed_out <= HOST_DIRECT_MAX;
    if (in_direct) {
        if ((rc = reserve_host(&g_hin, packed_in))) return rc;
        for (size_t v = 0; v < n_vec; v++)
            memcpy((float *)g_hin.p + v * cols, inputs + v * in_stride, cols * sizeof(float));
        rc = push_input(packed_in);
    } else if (in_stride == cols)
        rc = oxh_memcpy_h2d(g_dx.p, inputs, packed_in, NULL);
    else
        rc = oxh_memcpy2d_h2d(g_dx.p, cols * sizeof(float), inputs, in_stride * sizeof(float),
                              cols * sizeof(float), n_vec, NULL);
    if (rc) return rc;
    if (out_direct && (rc = reserve_host(&g_hout, packed_out))) return rc;
    float *const d_out = out_direct ? (float *)g_hout.p : (float *)g_dout.p;
    const float *d_x = (const float *)g_dx.p;
    /* More vectors than the GEMV kernel keeps in flight: Q4_K, Q5_K and Q6_K go to the
     * int8-MFMA kernel behind a stand-alone quantiser launch; everything else
     * walks the batch in GEMV-sized slices (every output is the same dot either way). */
    const bool kq456 = qtype == OXH_Q4_K_S || qtype == OXH_Q4_K_M || qtype == OXH_Q5_K_S || qtype == OXH_Q5_K_M ||
                       qtype == OXH_Q6_K;
    /* few rows, many columns, seven activations or more: the tiles' columns shared between workgroups
     * (up to six the dot kernels are as fast: 4096 x 14336 Q6_K 24.7 us at six, 43 at eight, 28 split) */
    const size_t split_ws = (kq456 && n_vec >= mmq_split_min_nv()) ? oxh_mmq_split_workspace(qtype, rows, cols, n_vec, rows) : 0;
    if (split_ws) {
        if ((rc = reserve(&g_dsplit, split_ws))) return rc;
        if ((rc = quantize(kind, d_x, cols, n_vec, cols, g_dact.p))) return rc;
        if ((rc = oxh_mmq_split(qtype, d_w, rows, cols, g_dact.p, n_vec, d_out, rows, g_dsplit.p, g_dsplit.bytes, NULL)))
            return rc;
    } else if (n_vec > 8 && kq456) {
        if ((rc = quantize(kind, d_x, cols, n_vec, cols, g_dact.p))) return rc;
        if ((rc = oxh_mmq_ex(qtype, d_w, rows, cols, g_dact.p, n_vec, d_out, rows,
                             mmq_relaxed_enabled() ? OXH_MMQ_RELAXED : 0u, NULL)))
            return rc;
    } else if (n_vec > 8 && (qtype == OXH_Q2_K || qtype == OXH_Q3_K_S || qtype == OXH_Q3_K_M ||
                             qtype == OXH_Q3_K_L)) {
        /* No MFMA kernel reads these blocks as they are.  Q3_K is exactly a Q6_K matrix in other bytes
         * and Q2_K widens to 210-byte blocks with scale * code in the 6-bit fields: the rewritten matrix
         * is made on the first batch over these weights and stays with their registry entry, as the
         * reference prepares its batch rows (oxk.c:734-745) */
        const uint8_t *d_prep;
        if ((rc = prepared_ptr(entry, data, rows, cols,
                               qtype == OXH_Q2_K ? OXH_PREP_Q2K_WIDE : OXH_PREP_Q3K_AS_Q6K, &d_prep)))
            return rc;
        if ((rc = quantize(kind, d_x, cols, n_vec, cols, g_dact.p))) return rc;
        const uint32_t as = qtype == OXH_Q2_K ? OXH_Q2_K_WIDE : OXH_Q6_K;
        const size_t ws = n_vec >= mmq_split_min_nv() ? oxh_mmq_split_workspace(as, rows, cols, n_vec, rows) : 0;
        if (ws && (rc = reserve(&g_dsplit, ws))) return rc;
        /* without a workspace this is oxh_mmq */
        if ((rc = oxh_mmq_split(as, d_prep, rows, cols, g_dact.p, n_vec, d_out, rows, ws ? g_dsplit.p : NULL,
                                ws ? g_dsplit.bytes : 0, NULL)))
            return rc;
    } else {
        const size_t step = oxh_gemv_max_nvec_buffered(qtype, cols);
        if (step == 0) {
            oxh_set_error("batch: cols too wide for one workgroup%s%s", NULL, NULL);
            return OXH_ERR_TOO_WIDE;
        }
        if (n_vec <= step) {
            /* one launch with the quantisation fused in; with room for the quantised activations a
             * launch of several vectors may run on the matrix cores (same results; the library decides) */
            uint32_t run_type = qtype;
            const uint8_t *run_w = d_w;
            batch_form(&run_type, entry, data, rows, cols, n_vec, &run_w);
            OxhSegment seg = { run_w, d_out, rows, 0, 0, NULL };
            if ((rc = oxh_gemv_segments_f32(run_type, &seg, 1, cols, d_x, cols, g_dact.p, n_vec, rows, NULL)))
                return rc;
        } else {
            /* every activation is quantised once; the 32-value formats then have a token-tiled kernel on
             * the matrix cores (the matrix is streamed once per 64 activations), the rest walk the batch in
             * slices over the stored bytes */
            if ((rc = quantize(kind, d_x, cols, n_vec, cols, g_dact.p))) return rc;
            rc = kind == 1 ? oxh_mmq(qtype, d_w, rows, cols, g_dact.p, n_vec, d_out, rows, NULL)
                           : OXH_DECLINED;
            if (rc != OXH_OK && rc != OXH_DECLINED) return rc;
            if (rc == OXH_DECLINED) {
                /* up to 32 slices per launch, each slice a segment over the same matrix with its own run of
                 * activations and its own place in the output: slices overlap instead of queueing behind
                 * launch gaps */
                enum { SLICES = 32 };
                OxhSegment segs[SLICES];
                size_t v0 = 0;
                while (v0 < n_vec) {
                    size_t n = 0;
                    for (; n < SLICES && v0 < n_vec; n++, v0 += step) {
                        const size_t m = n_vec - v0 < step ? n_vec - v0 : step;
                        const OxhSegment seg = { d_w, d_out + v0 * rows, rows, v0, m, NULL };
                        segs[n] = seg;
                    }
                    if ((rc = oxh_gemv_segments(qtype, segs, n, cols, g_dact.p, step, rows, NULL))) return rc;
                }
            }
        }
    }
    if (out_direct) {
        if ((rc = oxh_stream_sync(NULL))) return rc;
        for (size_t v = 0; v < n_vec; v++)
            memcpy(outputs + v * out_stride, (const float *)g_hout.p + v * rows, rows * sizeof(float));
        return OXH_OK;
    }
    if (out_stride == rows)
        rc = oxh_memcpy_d2h(outputs, g_dout.p, packed_out, NULL);
    else
        rc = oxh_memcpy2d_d2h(outputs, out_stride * sizeof(float), g_dout.p, rows * sizeof(float),
                              rows * sizeof(float), n_vec, NULL);
    if (rc) return rc;
    return oxh_stream_sync(NULL);
}

/* ─── public entry points: one call at a time ─────────────────────────── */

int oxh_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                         const float *input, float *output, float *temp)
{
    pthread_mutex_lock(&g_call);
    g_call_tick = g_tick;
    const int rc = mv_one(qtype, data, rows, cols, row_bytes, input, output, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_fused(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                               size_t cols, const size_t *row_bytes, size_t n_outs, const float *input,
                               float *const *outs, float *temp)
{
    pthread_mutex_lock(&g_call);
    g_call_tick = g_tick;
    const int rc = mv_fused(qtypes, datas, rows, cols, row_bytes, n_outs, input, outs, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_multi_input(const uint32_t *qtypes, const uint8_t *const *datas, const size_t *rows,
                                     size_t cols, const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs, float *const *outs, float *temp)
{
    pthread_mutex_lock(&g_call);
    g_call_tick = g_tick;
    const int rc = mv_multi_input(qtypes, datas, rows, cols, row_bytes, n_outs, inputs, outs, temp);
    pthread_mutex_unlock(&g_call);
    return rc;
}

int oxh_matvec_quantized_batch(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols, size_t row_bytes,
                               const float *inputs, size_t in_stride, float *outputs, size_t out_stride,
                               size_t n_vec, float *temp, uint8_t *act_scratch, size_t act_bytes)
{
    pthread_mutex_lock(&g_call);
    g_call_tick = g_tick;
    const int rc = mv_batch(qtype, data, rows, cols, row_bytes, inputs, in_stride, outputs, out_stride, n_vec,
                            temp, act_scratch, act_bytes);
    pthread_mutex_unlock(&g_call);
    return rc;
}

/* ─── the reference's own symbols ─────────────────────────────────────── */

/* They return void, so a call this library declines (or that fails) has to be finished by somebody else.
 * In this order:
 *   1. the CPU functions installed with oxh_set_cpu_fallback() get the call with its original arguments;
 *   2. else the weak symbols oc_ref_matvec_quantized* do, when the program links them (the reference's
 *      own functions renamed, e.g. objcopy --redefine-sym oc_matvec_quantized=oc_ref_matvec_quantized);
 *   3. else the handler installed with oxh_set_decline_handler() is told;
 *   4. else the process prints the error and aborts — it never silently computes something else. */
extern void oc_ref_matvec_quantized(uint32_t, const uint8_t *, size_t, size_t, size_t, const float *, float *,
                                    float *) __attribute__((weak));
extern void oc_ref_matvec_quantized_fused(const uint32_t *, const uint8_t *const *, const size_t *, size_t,
                                          const size_t *, size_t, const float *, float *const *, float *)
    __attribute__((weak));
extern void oc_ref_matvec_quantized_multi_input(const uint32_t *, const uint8_t *const *, const size_t *, size_t,
                                                const size_t *, size_t, const float *const *, float *const *,
                                                float *) __attribute__((weak));
extern void oc_ref_matvec_quantized_batch(uint32_t, const uint8_t *, size_t, size_t, size_t, const float *, size_t,
                                          float *, size_t, size_t, float *, uint8_t *, size_t)
    __attribute__((weak));

static OxhCpuFallback g_fallback;
static OxhDeclineHandler g_handler = NULL;
static void *g_handler_user = NULL;
static _Atomic size_t g_forwarded = 0;

void oxh_set_cpu_fallback(const OxhCpuFallback *fb)
{
    if (fb) g_fallback = *fb;
    else memset(&g_fallback, 0, sizeof g_fallback);
}

size_t oxh_cpu_fallback_calls(void) { return atomic_load(&g_forwarded); }

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
    fprintf(stderr, "liboxhip: oc_matvec entry %d failed with status %d: %s\n"
            "liboxhip: no CPU fallback is installed (oxh_set_cpu_fallback, or link oc_ref_matvec_quantized*)\n",
            which, status, oxh_last_error());
    abort();
}

void oc_matvec_quantized(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols,
                         size_t row_bytes, const float *input, float *output, float *temp)
{
    const int rc = oxh_matvec_quantized(qtype, data, rows, cols, row_bytes, input, output, temp);
    if (!rc) return;
    void (*fb)(uint32_t, const uint8_t *, size_t, size_t, size_t, const float *, float *, float *) =
        g_fallback.matvec_quantized ? g_fallback.matvec_quantized : oc_ref_matvec_quantized;
    if (!fb) { not_ok(0, rc); return; }
    atomic_fetch_add(&g_forwarded, 1);
    fb(qtype, data, rows, cols, row_bytes, input, output, temp);
}

void oc_matvec_quantized_fused(const uint32_t *qtypes, const uint8_t *const *datas,
                               const size_t *rows, size_t cols, const size_t *row_bytes,
                               size_t n_outs, const float *input, float *const *outs,
                               float *temp)
{
    const int rc = oxh_matvec_quantized_fused(qtypes, datas, rows, cols, row_bytes, n_outs,
                                              input, outs, temp);
    if (!rc) return;
    void (*fb)(const uint32_t *, const uint8_t *const *, const size_t *, size_t, const size_t *, size_t,
               const float *, float *const *, float *) =
        g_fallback.matvec_quantized_fused ? g_fallback.matvec_quantized_fused : oc_ref_matvec_quantized_fused;
    if (!fb) { not_ok(1, rc); return; }
    atomic_fetch_add(&g_forwarded, 1);
    fb(qtypes, datas, rows, cols, row_bytes, n_outs, input, outs, temp);
}

void oc_matvec_quantized_multi_input(const uint32_t *qtypes, const uint8_t *const *datas,
                                     const size_t *rows, size_t cols,
                                     const size_t *row_bytes, size_t n_outs,
                                     const float *const *inputs, float *const *outs,
                                     float *temp)
{
    const int rc = oxh_matvec_quantized_multi_input(qtypes, datas, rows, cols, row_bytes,
                                                    n_outs, inputs, outs, temp);
    if (!rc) return;
    void (*fb)(const uint32_t *, const uint8_t *const *, const size_t *, size_t, const size_t *, size_t,
               const float *const *, float *const *, float *) =
        g_fallback.matvec_quantized_multi_input ? g_fallback.matvec_quantized_multi_input
                                                : oc_ref_matvec_quantized_multi_input;
    if (!fb) { not_ok(2, rc); return; }
    atomic_fetch_add(&g_forwarded, 1);
    fb(qtypes, datas, rows, cols, row_bytes, n_outs, inputs, outs, temp);
}

void oc_matvec_quantized_batch(uint32_t qtype, const uint8_t *data, size_t rows, size_t cols,
                               size_t row_bytes, const float *inputs, size_t in_stride,
                               float *outputs, size_t out_stride, size_t n_vec, float *temp,
                               uint8_t *act_scratch, size_t act_bytes)
{
    const int rc = oxh_matvec_quantized_batch(qtype, data, rows, cols, row_bytes, inputs,
                                              in_stride, outputs, out_stride, n_vec, temp,
                                              act_scratch, act_bytes);
    if (!rc) return;
    void (*fb)(uint32_t, const uint8_t *, size_t, size_t, size_t, const float *, size_t, float *, size_t, size_t,
               float *, uint8_t *, size_t) =
        g_fallback.matvec_quantized_batch ? g_fallback.matvec_quantized_batch : oc_ref_matvec_quantized_batch;
    if (!fb) { not_ok(3, rc); return; }
    atomic_fetch_add(&g_forwarded, 1);
    fb(qtype, data, rows, cols, row_bytes, inputs, in_stride, outputs, out_stride, n_vec, temp, act_scratch,
       act_bytes);
}
