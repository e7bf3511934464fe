/*
 * oxh_gguf.c — GGUF model files in front of the matvec path: map the file,
 * read its header, metadata and tensor table, hand out weight views in the
 * shape the matvec entry points take, and make the quantized tensors resident
 * in HBM.
 *
 * What it replaces in the reference (paths relative to the reference
 * checkout): the parser oxidize-c/src/format/gguf.c:322-505 (same acceptance
 * rules: magic, versions 2 and 3, bounded counts and strings, at most 8
 * dimensions, general.alignment of any integer type but a power of two, data
 * section at the aligned end of the tables, every tensor's declared extent
 * inside the file), the weight view of oxidize-c/src/model/llama.c:108-127
 * (cols = dims[0], rows = the remaining dimensions), the on-disk type ids of
 * oxidize-c/src/compute/quantization.c:2925-2988 and the upload loop of
 * oxidize-c/src/backends/cuda.cu:633-712.
 *
 * The file is never copied: tensors point into a read-only mapping, which is
 * exactly what the host API's weight registry keys its device copies on.
 */
#define _POSIX_C_SOURCE 200809L
#include <errno.h>
#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "oxhip.h"
#include "oxh_internal.h"

#define GGUF_MAGIC 0x46554747u      /* "GGUF" little-endian */
#define GGUF_DEFAULT_ALIGNMENT 32u

enum {                              /* metadata value types, on-disk ids */
    MT_U8 = 0, MT_I8, MT_U16, MT_I16, MT_U32, MT_I32, MT_F32, MT_BOOL, MT_STRING, MT_ARRAY,
    MT_U64, MT_I64, MT_F64, MT_COUNT
};

typedef struct Meta {
    char *key;
    uint32_t type;
    union {
        uint64_t u;
        int64_t i;
        double f;
        struct { const char *p; size_t len; } s;    /* points into the mapping */
        struct { uint32_t elem_type; uint64_t len; } arr;
    } v;
} Meta;

struct OxhGguf {
    uint8_t *map;
    size_t len;
    uint32_t version;
    uint64_t alignment, data_start;
    size_t n_tensors, n_meta;
    OxhTensor *tensors;
    Meta *meta;
    int registered;
};

/* ─── on-disk type ids ────────────────────────────────────────────────── */

typedef struct TypeRow {
    uint32_t ggml_id, qtype, elems, bytes;
} TypeRow;

/* ggml id -> type id of the matvec API and block layout (elements, bytes);
 * layout 0/0 = known id without a fixed-size layout here.  Ids 12 and 13 map
 * to the _M variants as the reference does (quantization.c:2980-2983). */
static const TypeRow k_types[] = {
    { 0, 0, 1, 4 },        /* F32  */
    { 1, 1, 1, 2 },        /* F16  */
    { 30, 2, 1, 2 },       /* BF16 */
    { 2, 3, 32, 18 },      /* Q4_0 */
    { 3, 4, 32, 20 },      /* Q4_1 */
    { 6, 5, 32, 22 },      /* Q5_0 */
    { 7, 6, 32, 24 },      /* Q5_1 */
    { 8, OXH_Q8_0, 32, OXH_Q8_0_BYTES },
    { 10, 8, 256, 84 },    /* Q2_K */
    { 11, 9, 256, 110 },   /* Q3_K */
    { 12, OXH_Q4_K_M, 256, OXH_Q4_K_BYTES },
    { 13, OXH_Q5_K_M, 256, OXH_Q5_K_BYTES },
    { 14, OXH_Q6_K, 256, OXH_Q6_K_BYTES },
    { 21, OXH_IQ3_S, 256, OXH_IQ3_S_BYTES },
    { 66, OXH_IQ1_XXXS, 256, OXH_IQ1_XXXS_BYTES },
    { 20, OXH_IQ4_NL, 32, OXH_IQ4_NL_BYTES },    /* quantization.c:2954-2955 */
    { 23, OXH_IQ4_XS, 256, OXH_IQ4_XS_BYTES },
    { 24, 31, 1, 1 },      /* I8  */
    { 25, 32, 1, 2 },      /* I16 */
    { 26, 33, 1, 4 },      /* I32 */
    { 27, 34, 1, 8 },      /* I64 */
    { 28, 35, 1, 8 },      /* F64 */
    { 240, OXH_AL5, 32, 18 },
    { 241, OXH_AL8, 32, 34 },
    { 242, OXH_AL6, 32, 22 },
    { 243, OXH_AL5_XS, 32, OXH_AL5_XS_BYTES },
};

static const TypeRow *type_row(uint32_t ggml_id)
{
    for (size_t i = 0; i < sizeof k_types / sizeof k_types[0]; i++)
        if (k_types[i].ggml_id == ggml_id) return &k_types[i];
    return NULL;
}

uint32_t oxh_qtype_from_ggml_id(uint32_t ggml_id)
{
    const TypeRow *r = type_row(ggml_id);
    return r ? r->qtype : OXH_QTYPE_UNKNOWN;
}

/* ─── bounded little-endian reader ────────────────────────────────────── */

typedef struct Reader {
    const uint8_t *p;
    size_t len, pos;
} Reader;

static int rd(Reader *r, void *dst, size_t n)
{
    if (n > r->len - r->pos) return 0;
    memcpy(dst, r->p + r->pos, n);      /* the build targets are little-endian */
    r->pos += n;
    return 1;
}

/* length-prefixed string: pointer into the buffer, not NUL-terminated */
static int rd_str(Reader *r, const char **p, size_t *len)
{
    uint64_t n;
    if (!rd(r, &n, 8)) return 0;
    if (n > r->len - r->pos) return 0;
    *p = (const char *)r->p + r->pos;
    *len = (size_t)n;
    r->pos += (size_t)n;
    return 1;
}

static char *dup_str(const char *p, size_t len)
{
    char *s = (char *)malloc(len + 1);
    if (!s) return NULL;
    memcpy(s, p, len);
    s[len] = 0;
    return s;
}

static size_t scalar_size(uint32_t type)
{
    switch (type) {
    case MT_U8: case MT_I8: case MT_BOOL: return 1;
    case MT_U16: case MT_I16: return 2;
    case MT_U32: case MT_I32: case MT_F32: return 4;
    case MT_U64: case MT_I64: case MT_F64: return 8;
    default: return 0;
    }
}

/* Reads (or, for arrays, walks and bounds-checks) one value.  depth guards
 * arrays of arrays. */
static int rd_value(Reader *r, uint32_t type, Meta *m, int depth)
{
    if (type >= MT_COUNT) return 0;
    if (m) m->type = type;
    const size_t sz = scalar_size(type);
    if (sz) {
        uint8_t raw[8] = { 0 };
        if (!rd(r, raw, sz)) return 0;
        if (!m) return 1;
        switch (type) {
        case MT_U8: m->v.u = raw[0]; break;
        case MT_BOOL: m->v.u = raw[0] != 0; break;
        case MT_I8: m->v.i = (int8_t)raw[0]; break;
        case MT_U16: { uint16_t x; memcpy(&x, raw, 2); m->v.u = x; break; }
        case MT_I16: { int16_t x; memcpy(&x, raw, 2); m->v.i = x; break; }
        case MT_U32: { uint32_t x; memcpy(&x, raw, 4); m->v.u = x; break; }
        case MT_I32: { int32_t x; memcpy(&x, raw, 4); m->v.i = x; break; }
        case MT_F32: { float x; memcpy(&x, raw, 4); m->v.f = x; break; }
        case MT_U64: memcpy(&m->v.u, raw, 8); break;
        case MT_I64: memcpy(&m->v.i, raw, 8); break;
        default: memcpy(&m->v.f, raw, 8); break;
        }
        return 1;
    }
    if (type == MT_STRING) {
        const char *p;
        size_t len;
        if (!rd_str(r, &p, &len)) return 0;
        if (m) { m->v.s.p = p; m->v.s.len = len; }
        return 1;
    }
    /* array: element type, count, elements */
    uint32_t et;
    uint64_t n;
    if (depth > 4 || !rd(r, &et, 4) || et >= MT_COUNT || !rd(r, &n, 8)) return 0;
    if (n > r->len) return 0;
    if (m) { m->v.arr.elem_type = et; m->v.arr.len = n; }
    const size_t esz = scalar_size(et);
    if (esz) {
        if (n > (r->len - r->pos) / esz) return 0;
        r->pos += (size_t)n * esz;
        return 1;
    }
    for (uint64_t i = 0; i < n; i++)
        if (!rd_value(r, et, NULL, depth + 1)) return 0;
    return 1;
}

/* ─── errors ──────────────────────────────────────────────────────────── */

static int fmt_fail(const char *what, const char *detail)
{
    oxh_set_error("gguf: %s%s", what, detail ? detail : "");
    return OXH_ERR_FORMAT;
}

static int io_fail(const char *what, const char *path)
{
    char buf[160];
    snprintf(buf, sizeof buf, "%s (%s): ", what, strerror(errno));
    oxh_set_error("gguf: %s%s", buf, path);
    return OXH_ERR_IO;
}

/* ─── parse ───────────────────────────────────────────────────────────── */

static void free_tables(OxhGguf *g)
{
    if (g->tensors) {
        for (size_t i = 0; i < g->n_tensors; i++) free((void *)g->tensors[i].name);
        free(g->tensors);
    }
    if (g->meta) {
        for (size_t i = 0; i < g->n_meta; i++) free(g->meta[i].key);
        free(g->meta);
    }
    g->tensors = NULL;
    g->meta = NULL;
}

static int parse(OxhGguf *g)
{
    Reader r = { g->map, g->len, 0 };
    uint32_t magic, version;
    uint64_t n_tensors, n_meta;
    if (!rd(&r, &magic, 4)) return fmt_fail("truncated header", NULL);
    if (magic != GGUF_MAGIC) return fmt_fail("bad magic", NULL);
    if (!rd(&r, &version, 4)) return fmt_fail("truncated header", NULL);
    if (version != 2u && version != 3u) return fmt_fail("unsupported version", NULL);
    if (!rd(&r, &n_tensors, 8) || !rd(&r, &n_meta, 8)) return fmt_fail("truncated header", NULL);
    /* every entry takes at least a few bytes */
    if (n_tensors > g->len || n_meta > g->len) return fmt_fail("header counts exceed the file size", NULL);
    g->version = version;

    g->meta = (Meta *)calloc(n_meta ? (size_t)n_meta : 1, sizeof(Meta));
    g->tensors = (OxhTensor *)calloc(n_tensors ? (size_t)n_tensors : 1, sizeof(OxhTensor));
    if (!g->meta || !g->tensors) {
        oxh_set_error("gguf: out of host memory for the tables%s%s", NULL, NULL);
        return OXH_ERR_NOMEM;
    }
    for (uint64_t i = 0; i < n_meta; i++) {
        const char *k;
        size_t klen;
        uint32_t type;
        if (!rd_str(&r, &k, &klen) || !rd(&r, &type, 4)) return fmt_fail("truncated metadata", NULL);
        if (type >= MT_COUNT) return fmt_fail("unknown metadata value type", NULL);
        Meta *m = &g->meta[g->n_meta];
        if (!(m->key = dup_str(k, klen))) return OXH_ERR_NOMEM;
        g->n_meta++;
        if (!rd_value(&r, type, m, 0)) return fmt_fail("truncated or malformed metadata value of ", m->key);
    }
    for (uint64_t i = 0; i < n_tensors; i++) {
        const char *nm;
        size_t nlen;
        OxhTensor *t = &g->tensors[g->n_tensors];
        if (!rd_str(&r, &nm, &nlen)) return fmt_fail("truncated tensor table", NULL);
        if (!(t->name = dup_str(nm, nlen))) return OXH_ERR_NOMEM;
        g->n_tensors++;
        if (!rd(&r, &t->n_dims, 4)) return fmt_fail("truncated tensor table at ", t->name);
        if (t->n_dims > OXH_GGUF_MAX_DIMS) return fmt_fail("too many dimensions in ", t->name);
        for (uint32_t d = 0; d < t->n_dims; d++)
            if (!rd(&r, &t->dims[d], 8)) return fmt_fail("truncated tensor table at ", t->name);
        if (!rd(&r, &t->ggml_type, 4) || !rd(&r, &t->offset, 8))
            return fmt_fail("truncated tensor table at ", t->name);
    }

    /* general.alignment: any unsigned type, or a positive signed one */
    uint64_t alignment = GGUF_DEFAULT_ALIGNMENT;
    for (size_t i = 0; i < g->n_meta; i++) {
        const Meta *m = &g->meta[i];
        if (strcmp(m->key, "general.alignment")) continue;
        switch (m->type) {
        case MT_U8: case MT_U16: case MT_U32: case MT_U64: alignment = m->v.u; break;
        case MT_I8: case MT_I16: case MT_I32: case MT_I64:
            if (m->v.i <= 0) return fmt_fail("general.alignment is not positive", NULL);
            alignment = (uint64_t)m->v.i;
            break;
        default: return fmt_fail("general.alignment is not an integer", NULL);
        }
        break;
    }
    if (alignment == 0 || (alignment & (alignment - 1))) return fmt_fail("alignment is not a power of two", NULL);
    if ((uint64_t)r.pos > UINT64_MAX - (alignment - 1)) return fmt_fail("data section offset overflows", NULL);
    const uint64_t data_start = ((uint64_t)r.pos + alignment - 1) & ~(alignment - 1);
    if (data_start > g->len) return fmt_fail("data section starts beyond the end of the file", NULL);
    g->alignment = alignment;
    g->data_start = data_start;

    for (size_t i = 0; i < g->n_tensors; i++) {
        OxhTensor *t = &g->tensors[i];
        if (t->offset > UINT64_MAX - data_start) return fmt_fail("offset overflow in ", t->name);
        const uint64_t abs = data_start + t->offset;
        if (abs > g->len) return fmt_fail("tensor starts beyond the end of the file: ", t->name);
        uint64_t numel = 1;
        for (uint32_t d = 0; d < t->n_dims; d++) {
            if (t->dims[d] && numel > UINT64_MAX / t->dims[d]) return fmt_fail("dimension product overflows in ", t->name);
            numel *= t->dims[d];
        }
        const TypeRow *row = type_row(t->ggml_type);
        t->qtype = row ? row->qtype : OXH_QTYPE_UNKNOWN;
        t->data = g->map + abs;
        t->cols = t->n_dims ? (size_t)t->dims[0] : 0;
        t->rows = t->n_dims >= 2 ? (size_t)(t->cols ? numel / t->cols : 0) : (t->n_dims ? 1 : 0);
        /* a type with a block layout and a whole number of blocks has a known
         * extent, which must end inside the file; the others are left to whoever
         * asks for them */
        if (row && row->elems && numel % row->elems == 0) {
            if (numel / row->elems > UINT64_MAX / row->bytes) return fmt_fail("size overflows in ", t->name);
            const uint64_t nbytes = numel / row->elems * row->bytes;
            if (nbytes > g->len - abs) return fmt_fail("tensor data runs past the end of the file: ", t->name);
            t->nbytes = (size_t)nbytes;
            if (t->cols && t->cols % row->elems == 0) t->row_bytes = t->cols / row->elems * row->bytes;
        }
    }
    return OXH_OK;
}

/* ─── public API ──────────────────────────────────────────────────────── */

int oxh_gguf_open(const char *path, OxhGguf **out)
{
    if (!path || !out) {
        oxh_set_error("invalid argument: %s%s", "oxh_gguf_open: NULL", NULL);
        return OXH_ERR_ARG;
    }
    *out = NULL;
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return io_fail("cannot open", path);
    struct stat st;
    if (fstat(fd, &st) != 0) {
        const int rc = io_fail("cannot stat", path);
        close(fd);
        return rc;
    }
    if (st.st_size <= 0) {
        close(fd);
        return fmt_fail("empty file: ", path);
    }
    void *map = mmap(NULL, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    const int map_errno = errno;
    close(fd);
    if (map == MAP_FAILED) {
        errno = map_errno;
        return io_fail("cannot map", path);
    }
    OxhGguf *g = (OxhGguf *)calloc(1, sizeof *g);
    if (!g) {
        munmap(map, (size_t)st.st_size);
        oxh_set_error("gguf: out of host memory%s%s", NULL, NULL);
        return OXH_ERR_NOMEM;
    }
    g->map = (uint8_t *)map;
    g->len = (size_t)st.st_size;
    const int rc = parse(g);
    if (rc != OXH_OK) {
        free_tables(g);
        munmap(g->map, g->len);
        free(g);
        return rc;
    }
    *out = g;
    return OXH_OK;
}

void oxh_gguf_close(OxhGguf *g)
{
    if (!g) return;
    if (g->registered)
        for (size_t i = 0; i < g->n_tensors; i++)
            if (g->tensors[i].resident) (void)oxh_weight_unregister(g->tensors[i].data);
    free_tables(g);
    munmap(g->map, g->len);
    free(g);
}

int oxh_gguf_info(const OxhGguf *g, uint32_t *version, uint64_t *alignment, uint64_t *data_start,
                  size_t *n_tensors, size_t *n_metadata)
{
    if (!g) return OXH_ERR_ARG;
    if (version) *version = g->version;
    if (alignment) *alignment = g->alignment;
    if (data_start) *data_start = g->data_start;
    if (n_tensors) *n_tensors = g->n_tensors;
    if (n_metadata) *n_metadata = g->n_meta;
    return OXH_OK;
}

int oxh_gguf_tensor_at(const OxhGguf *g, size_t index, OxhTensor *out)
{
    if (!g || !out || index >= g->n_tensors) {
        oxh_set_error("invalid argument: %s%s", "oxh_gguf_tensor_at: index out of range", NULL);
        return OXH_ERR_ARG;
    }
    *out = g->tensors[index];
    return OXH_OK;
}

int oxh_gguf_tensor_find(const OxhGguf *g, const char *name, OxhTensor *out)
{
    if (!g || !name || !out) return OXH_ERR_ARG;
    for (size_t i = 0; i < g->n_tensors; i++)
        if (!strcmp(g->tensors[i].name, name)) {
            *out = g->tensors[i];
            return OXH_OK;
        }
    oxh_set_error("gguf: no tensor named %s%s", name, NULL);
    return OXH_DECLINED;
}

static const Meta *meta_find(const OxhGguf *g, const char *key)
{
    if (!g || !key) return NULL;
    for (size_t i = 0; i < g->n_meta; i++)
        if (!strcmp(g->meta[i].key, key)) return &g->meta[i];
    return NULL;
}

int oxh_gguf_meta_u64(const OxhGguf *g, const char *key, uint64_t *out)
{
    const Meta *m = meta_find(g, key);
    if (!m || !out) return OXH_DECLINED;
    switch (m->type) {
    case MT_U8: case MT_U16: case MT_U32: case MT_U64: case MT_BOOL: *out = m->v.u; return OXH_OK;
    case MT_I8: case MT_I16: case MT_I32: case MT_I64:
        if (m->v.i < 0) return OXH_DECLINED;
        *out = (uint64_t)m->v.i;
        return OXH_OK;
    default: return OXH_DECLINED;
    }
}

int oxh_gguf_meta_f64(const OxhGguf *g, const char *key, double *out)
{
    const Meta *m = meta_find(g, key);
    if (!m || !out) return OXH_DECLINED;
    if (m->type == MT_F32 || m->type == MT_F64) { *out = m->v.f; return OXH_OK; }
    return OXH_DECLINED;
}

int oxh_gguf_meta_str(const OxhGguf *g, const char *key, const char **data, size_t *len)
{
    const Meta *m = meta_find(g, key);
    if (!m || m->type != MT_STRING || !data || !len) return OXH_DECLINED;
    *data = m->v.s.p;
    *len = m->v.s.len;
    return OXH_OK;
}

int oxh_gguf_register_all(OxhGguf *g, size_t *n_registered, size_t *bytes)
{
    if (!g) return OXH_ERR_ARG;
    size_t n = 0, total = 0;
    for (size_t i = 0; i < g->n_tensors; i++) {
        OxhTensor *t = &g->tensors[i];
        if (t->resident) { n++; total += t->nbytes; continue; }
        /* types with an integer path, and those that run on f32 inputs on the device */
        if (t->n_dims < 2 || t->nbytes == 0 ||
            (!oxh_act_kind(t->qtype, t->cols) && !oxh_f32_path_row_bytes(t->qtype, t->cols))) continue;
        const int rc = oxh_weight_register(t->data, t->nbytes);
        if (rc != OXH_OK) return rc;
        t->resident = 1;
        g->registered = 1;
        n++;
        total += t->nbytes;
    }
    if (n_registered) *n_registered = n;
    if (bytes) *bytes = total;
    return OXH_OK;
}
