/*
 * GGUF tensor directory reader and resident-arena loader: the way real encoded tensors reach the
 * kernels of this backend. The structural rules are the reference reader's
 * (src/gguf/core.c:850-1250: version 3, general.alignment as a non-zero uint32 with 32 as the
 * default, rank 1..4, non-zero dimensions, storage bytes from the qtype geometry, relative
 * offsets that are multiples of the alignment, unique non-empty names of at most 64 bytes, a
 * data section that starts at the aligned end of the directory) with the reference's mapping of
 * refusals to status codes (core.c:52-79). Metadata values are walked and kept when scalar or
 * string; arrays are skipped over. The loader copies the whole tensor-data section into a
 * resident arena and publishes it, after which weight views are plain offsets into the arena
 * (expert-major 3-D tensors read as rows = dims[1] * dims[2], the layout the sweeps take).
 */
#include <limits.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "private.h"

#define GGUF_MAGIC 0x46554747u
#define GGUF_VERSION 3u
#define GGUF_DEFAULT_ALIGNMENT 32u
#define GGUF_MAX_KEY 65535ull
#define GGUF_MAX_NAME 64ull
#define GGUF_MAX_STRING 67108864ull
#define GGUF_MAX_ARRAY 16777216ull
#define GGUF_MAX_DEPTH 16u
#define GGUF_MAX_ENTRIES 1048576ull

enum { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64, T_INVALID };

typedef struct {
    char *key;
    unsigned int type;
    unsigned long long u;    /* integers and bool; string length */
    double f;
    char *text;              /* strings (NUL-terminated copy) */
} gguf_entry;

struct yvex_rocm_gguf {
    FILE *file;
    unsigned long long file_size, cursor;
    unsigned int version, alignment;
    unsigned long long tensor_count, metadata_count, tensor_data_offset;
    gguf_entry *metadata;
    yvex_gguf_tensor_info *tensors;
    unsigned long long *by_name;      /* tensor indices sorted by name */
};

static int fail(yvex_error *err, int code, const char *where, const char *message)
{
    return yvex_rocm_refuse(err, (yvex_status)code, where, message);
}

static int take(yvex_rocm_gguf *g, void *out, unsigned long long bytes, const char *where, yvex_error *err)
{
    if (bytes > g->file_size - g->cursor) return fail(err, YVEX_ERR_BOUNDS, where, "GGUF input is truncated");
    if (bytes && fread(out, 1u, (size_t)bytes, g->file) != (size_t)bytes)
        return fail(err, YVEX_ERR_IO, where, "GGUF input cannot be read");
    g->cursor += bytes;
    return YVEX_OK;
}

static int skip(yvex_rocm_gguf *g, unsigned long long bytes, const char *where, yvex_error *err)
{
    if (bytes > g->file_size - g->cursor) return fail(err, YVEX_ERR_BOUNDS, where, "GGUF input is truncated");
    if (bytes && fseeko(g->file, (off_t)(g->cursor + bytes), SEEK_SET) != 0)
        return fail(err, YVEX_ERR_IO, where, "GGUF input cannot be read");
    g->cursor += bytes;
    return YVEX_OK;
}

static unsigned long long le(const unsigned char *b, unsigned int n)
{
    unsigned long long v = 0ull;
    while (n--) v = (v << 8) | b[n];
    return v;
}

static int take_u32(yvex_rocm_gguf *g, unsigned int *out, const char *where, yvex_error *err)
{
    unsigned char b[4];
    int rc = take(g, b, 4u, where, err);
    if (rc == YVEX_OK) *out = (unsigned int)le(b, 4u);
    return rc;
}

static int take_u64(yvex_rocm_gguf *g, unsigned long long *out, const char *where, yvex_error *err)
{
    unsigned char b[8];
    int rc = take(g, b, 8u, where, err);
    if (rc == YVEX_OK) *out = le(b, 8u);
    return rc;
}

/* Length-prefixed string; keep = 0 skips the bytes. Embedded NUL bytes are refused in kept text. */
static int take_string(yvex_rocm_gguf *g, char **out, unsigned long long *len, unsigned long long limit,
                       int keep, const char *where, yvex_error *err)
{
    unsigned long long n;
    char *text;
    int rc = take_u64(g, &n, where, err);
    if (rc != YVEX_OK) return rc;
    if (n > limit) return fail(err, YVEX_ERR_BOUNDS, where, "GGUF string exceeds the reader's limit");
    if (len) *len = n;
    if (!keep) return skip(g, n, where, err);
    text = (char *)malloc((size_t)n + 1u);
    if (!text) return fail(err, YVEX_ERR_NOMEM, where, "out of host memory");
    rc = take(g, text, n, where, err);
    if (rc == YVEX_OK && memchr(text, 0, (size_t)n)) rc = fail(err, YVEX_ERR_FORMAT, where, "GGUF string holds a NUL byte");
    if (rc != YVEX_OK) {
        free(text);
        return rc;
    }
    text[n] = 0;
    *out = text;
    return YVEX_OK;
}

static unsigned int scalar_bytes(unsigned int type)
{
    switch (type) {
    case T_U8: case T_I8: case T_BOOL: return 1u;
    case T_U16: case T_I16: return 2u;
    case T_U32: case T_I32: case T_F32: return 4u;
    case T_U64: case T_I64: case T_F64: return 8u;
    default: return 0u;
    }
}

static int walk_array(yvex_rocm_gguf *g, unsigned int depth, yvex_error *err)
{
    unsigned int element;
    unsigned long long count, i;
    int rc;
    if (depth >= GGUF_MAX_DEPTH) return fail(err, YVEX_ERR_BOUNDS, "gguf.metadata.array", "GGUF array nesting is too deep");
    rc = take_u32(g, &element, "gguf.metadata.array", err);
    if (rc == YVEX_OK) rc = take_u64(g, &count, "gguf.metadata.array", err);
    if (rc != YVEX_OK) return rc;
    if (element >= T_INVALID) return fail(err, YVEX_ERR_UNSUPPORTED, "gguf.metadata.array", "unknown GGUF metadata type");
    if (count > GGUF_MAX_ARRAY) return fail(err, YVEX_ERR_BOUNDS, "gguf.metadata.array", "GGUF array exceeds the reader's limit");
    if (scalar_bytes(element)) return skip(g, count * scalar_bytes(element), "gguf.metadata.array", err);
    for (i = 0ull; i < count; ++i) {
        rc = element == T_STRING ? take_string(g, NULL, NULL, GGUF_MAX_STRING, 0, "gguf.metadata.array", err)
                                 : walk_array(g, depth + 1u, err);
        if (rc != YVEX_OK) return rc;
    }
    return YVEX_OK;
}

/* src/gguf/core.c:491-527: segments joined by '.', each starting with a lower-case letter and
 * holding lower-case letters, digits and single underscores that are not at its end */
static int key_valid(const char *key, unsigned long long len)
{
    unsigned long long i;
    int segment_start = 1, previous_underscore = 0;
    if (!len) return 0;
    for (i = 0ull; i < len; ++i) {
        unsigned char ch = (unsigned char)key[i];
        if (ch == '.') {
            if (segment_start || previous_underscore || i + 1ull == len) return 0;
            segment_start = 1;
            previous_underscore = 0;
        } else if (segment_start) {
            if (ch < 'a' || ch > 'z') return 0;
            segment_start = 0;
        } else if (ch == '_') {
            if (previous_underscore) return 0;
            previous_underscore = 1;
        } else {
            if (!((ch >= 'a' && ch <= 'z') || (ch >= '0' && ch <= '9'))) return 0;
            previous_underscore = 0;
        }
    }
    return !segment_start && !previous_underscore;
}

static int parse_metadata(yvex_rocm_gguf *g, yvex_error *err)
{
    unsigned long long i, j;
    if (g->metadata_count > GGUF_MAX_ENTRIES)
        return fail(err, YVEX_ERR_BOUNDS, "gguf.metadata", "GGUF metadata count exceeds the reader's limit");
    g->metadata = (gguf_entry *)calloc((size_t)(g->metadata_count ? g->metadata_count : 1ull), sizeof(*g->metadata));
    if (!g->metadata) return fail(err, YVEX_ERR_NOMEM, "gguf.metadata", "out of host memory");
    for (i = 0ull; i < g->metadata_count; ++i) {
        gguf_entry *e = &g->metadata[i];
        unsigned long long len = 0ull;
        unsigned char b[8];
        int rc = take_string(g, &e->key, &len, GGUF_MAX_KEY, 1, "gguf.metadata.key", err);
        if (rc != YVEX_OK) return rc;
        if (!key_valid(e->key, len)) return fail(err, YVEX_ERR_FORMAT, "gguf.metadata.key", "GGUF metadata key violates the key grammar");
        for (j = 0ull; j < i; ++j)
            if (!strcmp(g->metadata[j].key, e->key))
                return fail(err, YVEX_ERR_FORMAT, "gguf.metadata.key", "duplicate GGUF metadata key");
        rc = take_u32(g, &e->type, "gguf.metadata.type", err);
        if (rc != YVEX_OK) return rc;
        if (e->type >= T_INVALID) return fail(err, YVEX_ERR_UNSUPPORTED, "gguf.metadata.type", "unknown GGUF metadata type");
        if (e->type == T_STRING) rc = take_string(g, &e->text, &e->u, GGUF_MAX_STRING, 1, "gguf.metadata.value", err);
        else if (e->type == T_ARRAY) rc = walk_array(g, 0u, err);
        else {
            unsigned int n = scalar_bytes(e->type);
            rc = take(g, b, n, "gguf.metadata.value", err);
            if (rc == YVEX_OK) {
                e->u = le(b, n);
                if (e->type == T_F32) {
                    float v;
                    unsigned int bits = (unsigned int)e->u;
                    memcpy(&v, &bits, sizeof(v));
                    e->f = v;
                } else if (e->type == T_F64) {
                    memcpy(&e->f, &e->u, sizeof(e->f));
                } else if (e->type == T_BOOL && e->u > 1ull) {
                    rc = fail(err, YVEX_ERR_FORMAT, "gguf.metadata.value", "GGUF bool is neither 0 nor 1");
                }
            }
        }
        if (rc != YVEX_OK) return rc;
    }
    return YVEX_OK;
}

static const gguf_entry *find_entry(const yvex_rocm_gguf *g, const char *key)
{
    unsigned long long i;
    for (i = 0ull; g && key && i < g->metadata_count; ++i)
        if (g->metadata[i].key && !strcmp(g->metadata[i].key, key)) return &g->metadata[i];
    return NULL;
}

/* storage bytes of a tensor: rows of dims[0] values, blocked along the row (qtype.c geometry) */
static int tensor_storage(unsigned int qtype, const unsigned long long *dims, unsigned int rank,
                          unsigned long long *bytes)
{
    const yvex_rocm_qtype_geometry *geometry = yvex_rocm_gguf_qtype_geometry_find(qtype);
    unsigned long long rows = 1ull, row_bytes;
    unsigned int d;
    if (!geometry || !geometry->block_size || !geometry->bytes_per_block) return YVEX_ERR_UNSUPPORTED;
    if (dims[0] % geometry->block_size) return YVEX_ERR_FORMAT;
    for (d = 1u; d < rank; ++d) {
        if (rows > ULLONG_MAX / dims[d]) return YVEX_ERR_BOUNDS;
        rows *= dims[d];
    }
    if (dims[0] / geometry->block_size > ULLONG_MAX / geometry->bytes_per_block) return YVEX_ERR_BOUNDS;
    row_bytes = dims[0] / geometry->block_size * geometry->bytes_per_block;
    if (rows > ULLONG_MAX / row_bytes) return YVEX_ERR_BOUNDS;
    *bytes = rows * row_bytes;
    return YVEX_OK;
}

typedef struct {
    const char *name;
    unsigned long long index;
} named_index;

static int by_name_compare(const void *a, const void *b)
{
    return strcmp(((const named_index *)a)->name, ((const named_index *)b)->name);
}

static int parse_tensors(yvex_rocm_gguf *g, yvex_error *err)
{
    unsigned long long i, remainder;
    unsigned int d;
    int rc;
    if (g->tensor_count > GGUF_MAX_ENTRIES)
        return fail(err, YVEX_ERR_BOUNDS, "gguf.tensor", "GGUF tensor count exceeds the reader's limit");
    g->tensors = (yvex_gguf_tensor_info *)calloc((size_t)(g->tensor_count ? g->tensor_count : 1ull), sizeof(*g->tensors));
    g->by_name = (unsigned long long *)calloc((size_t)(g->tensor_count ? g->tensor_count : 1ull), sizeof(*g->by_name));
    if (!g->tensors || !g->by_name) return fail(err, YVEX_ERR_NOMEM, "gguf.tensor", "out of host memory");
    for (i = 0ull; i < g->tensor_count; ++i) {
        yvex_gguf_tensor_info *t = &g->tensors[i];
        char *name = NULL;
        rc = take_string(g, &name, &t->name_len, GGUF_MAX_NAME, 1, "gguf.tensor.name", err);
        if (rc != YVEX_OK) return rc;
        t->name = name;
        g->by_name[i] = i;
        if (!t->name_len) return fail(err, YVEX_ERR_FORMAT, "gguf.tensor.name", "GGUF tensor name is empty");
        rc = take_u32(g, &t->rank, "gguf.tensor.rank", err);
        if (rc != YVEX_OK) return rc;
        if (!t->rank || t->rank > YVEX_GGUF_MAX_DIMS)
            return fail(err, YVEX_ERR_FORMAT, "gguf.tensor.rank", "GGUF tensor rank is outside the admitted range");
        for (d = 0u; d < t->rank; ++d) {
            rc = take_u64(g, &t->dims[d], "gguf.tensor.dimension", err);
            if (rc != YVEX_OK) return rc;
            if (!t->dims[d]) return fail(err, YVEX_ERR_FORMAT, "gguf.tensor.dimension", "GGUF tensor dimension is zero");
        }
        rc = take_u32(g, &t->ggml_type, "gguf.tensor.qtype", err);
        if (rc != YVEX_OK) return rc;
        rc = tensor_storage(t->ggml_type, t->dims, t->rank, &t->storage_bytes);
        if (rc != YVEX_OK)
            return fail(err, rc, "gguf.tensor.qtype",
                        rc == YVEX_ERR_UNSUPPORTED ? "GGUF tensor qtype has no storage geometry here"
                        : rc == YVEX_ERR_FORMAT ? "GGUF tensor row is not a whole number of blocks"
                                                : "GGUF tensor storage extent overflows");
        t->ggml_type_name = yvex_rocm_gguf_qtype_geometry_find(t->ggml_type)->name;
        rc = take_u64(g, &t->relative_offset, "gguf.tensor.offset", err);
        if (rc != YVEX_OK) return rc;
        if (t->relative_offset % g->alignment)
            return fail(err, YVEX_ERR_FORMAT, "gguf.tensor.offset", "GGUF tensor relative offset is misaligned");
    }
    {
        named_index *order = (named_index *)calloc((size_t)(g->tensor_count ? g->tensor_count : 1ull), sizeof(*order));
        if (!order) return fail(err, YVEX_ERR_NOMEM, "gguf.tensor", "out of host memory");
        for (i = 0ull; i < g->tensor_count; ++i) {
            order[i].name = g->tensors[i].name;
            order[i].index = i;
        }
        qsort(order, (size_t)g->tensor_count, sizeof(*order), by_name_compare);
        for (i = 0ull; i < g->tensor_count; ++i) g->by_name[i] = order[i].index;
        free(order);
    }
    for (i = 1ull; i < g->tensor_count; ++i)
        if (!strcmp(g->tensors[g->by_name[i - 1u]].name, g->tensors[g->by_name[i]].name))
            return fail(err, YVEX_ERR_FORMAT, "gguf.tensor.name", "duplicate GGUF tensor name");
    remainder = g->cursor % g->alignment;
    g->tensor_data_offset = g->cursor + (remainder ? g->alignment - remainder : 0ull);
    if (g->tensor_data_offset > g->file_size)
        return fail(err, YVEX_ERR_BOUNDS, "gguf.range", "GGUF tensor-data boundary exceeds file size");
    for (i = 0ull; i < g->tensor_count; ++i) {
        yvex_gguf_tensor_info *t = &g->tensors[i];
        if (t->relative_offset > ULLONG_MAX - g->tensor_data_offset ||
            t->storage_bytes > ULLONG_MAX - g->tensor_data_offset - t->relative_offset)
            return fail(err, YVEX_ERR_BOUNDS, "gguf.range", "GGUF tensor absolute range overflows");
        t->absolute_offset = g->tensor_data_offset + t->relative_offset;
        t->absolute_end_offset = t->absolute_offset + t->storage_bytes;
        t->range_addressable = t->absolute_end_offset <= g->file_size;
    }
    return YVEX_OK;
}

int yvex_rocm_gguf_open_path(yvex_rocm_gguf **out, const char *path, yvex_error *err)
{
    yvex_rocm_gguf *g;
    unsigned char header[24];
    const gguf_entry *alignment;
    int rc;
    if (out) *out = NULL;
    if (!out || !path) return fail(err, YVEX_ERR_INVALID_ARG, "yvex_rocm_gguf_open_path", "output and path are required");
    g = (yvex_rocm_gguf *)calloc(1u, sizeof(*g));
    if (!g) return fail(err, YVEX_ERR_NOMEM, "yvex_rocm_gguf_open_path", "out of host memory");
    g->file = fopen(path, "rb");
    if (!g->file || fseeko(g->file, 0, SEEK_END) != 0 || ftello(g->file) < 0 || fseeko(g->file, 0, SEEK_SET) != 0) {
        rc = fail(err, YVEX_ERR_IO, "yvex_rocm_gguf_open_path", "GGUF file cannot be opened");
        goto failed;
    }
    fseeko(g->file, 0, SEEK_END);
    g->file_size = (unsigned long long)ftello(g->file);
    fseeko(g->file, 0, SEEK_SET);
    g->alignment = GGUF_DEFAULT_ALIGNMENT;
    rc = take(g, header, sizeof(header), "gguf.header", err);
    if (rc != YVEX_OK) goto failed;
    if ((unsigned int)le(header, 4u) != GGUF_MAGIC) {
        rc = fail(err, YVEX_ERR_FORMAT, "yvex_rocm_gguf_open_path", "invalid GGUF magic");
        goto failed;
    }
    g->version = (unsigned int)le(header + 4, 4u);
    if (g->version != GGUF_VERSION) {
        rc = fail(err, YVEX_ERR_UNSUPPORTED, "yvex_rocm_gguf_open_path", "unsupported GGUF container version");
        goto failed;
    }
    g->tensor_count = le(header + 8, 8u);
    g->metadata_count = le(header + 16, 8u);
    rc = parse_metadata(g, err);
    if (rc != YVEX_OK) goto failed;
    alignment = find_entry(g, "general.alignment");
    if (alignment) {
        if (alignment->type != T_U32 || !alignment->u) {
            rc = fail(err, YVEX_ERR_FORMAT, "gguf.metadata.alignment", "general.alignment must be uint32 and nonzero");
            goto failed;
        }
        g->alignment = (unsigned int)alignment->u;
    }
    rc = parse_tensors(g, err);
    if (rc != YVEX_OK) goto failed;
    *out = g;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
failed:
    yvex_rocm_gguf_close(g);
    return rc;
}

void yvex_rocm_gguf_close(yvex_rocm_gguf *g)
{
    unsigned long long i;
    if (!g) return;
    for (i = 0ull; g->metadata && i < g->metadata_count; ++i) {
        free(g->metadata[i].key);
        free(g->metadata[i].text);
    }
    for (i = 0ull; g->tensors && i < g->tensor_count; ++i) free((char *)g->tensors[i].name);
    free(g->metadata);
    free(g->tensors);
    free(g->by_name);
    if (g->file) fclose(g->file);
    free(g);
}

unsigned long long yvex_rocm_gguf_tensor_count(const yvex_rocm_gguf *g) { return g ? g->tensor_count : 0ull; }
unsigned long long yvex_rocm_gguf_metadata_count(const yvex_rocm_gguf *g) { return g ? g->metadata_count : 0ull; }
unsigned long long yvex_rocm_gguf_tensor_data_offset(const yvex_rocm_gguf *g) { return g ? g->tensor_data_offset : 0ull; }
unsigned int yvex_rocm_gguf_alignment(const yvex_rocm_gguf *g) { return g ? g->alignment : 0u; }
unsigned long long yvex_rocm_gguf_file_size(const yvex_rocm_gguf *g) { return g ? g->file_size : 0ull; }

const yvex_gguf_tensor_info *yvex_rocm_gguf_tensor_at(const yvex_rocm_gguf *g, unsigned long long index)
{
    return g && index < g->tensor_count ? &g->tensors[index] : NULL;
}

const yvex_gguf_tensor_info *yvex_rocm_gguf_tensor_find(const yvex_rocm_gguf *g, const char *name)
{
    unsigned long long low = 0ull, high;
    if (!g || !name) return NULL;
    high = g->tensor_count;
    while (low < high) {
        unsigned long long mid = low + (high - low) / 2ull;
        int order = strcmp(g->tensors[g->by_name[mid]].name, name);
        if (!order) return &g->tensors[g->by_name[mid]];
        if (order < 0) low = mid + 1ull;
        else high = mid;
    }
    return NULL;
}

int yvex_rocm_gguf_metadata_u64(const yvex_rocm_gguf *g, const char *key, unsigned long long *out)
{
    const gguf_entry *e = find_entry(g, key);
    if (!e || !out || e->type == T_STRING || e->type == T_ARRAY || e->type == T_F32 || e->type == T_F64)
        return YVEX_ERR_FORMAT;
    if ((e->type == T_I8 && (e->u & 0x80ull)) || (e->type == T_I16 && (e->u & 0x8000ull)) ||
        (e->type == T_I32 && (e->u & 0x80000000ull)) || (e->type == T_I64 && (e->u >> 63)))
        return YVEX_ERR_BOUNDS;      /* negative */
    *out = e->u;
    return YVEX_OK;
}

int yvex_rocm_gguf_metadata_f64(const yvex_rocm_gguf *g, const char *key, double *out)
{
    const gguf_entry *e = find_entry(g, key);
    if (!e || !out || (e->type != T_F32 && e->type != T_F64)) return YVEX_ERR_FORMAT;
    *out = e->f;
    return YVEX_OK;
}

int yvex_rocm_gguf_metadata_string(const yvex_rocm_gguf *g, const char *key, const char **text, unsigned long long *len)
{
    const gguf_entry *e = find_entry(g, key);
    if (!e || !text || e->type != T_STRING) return YVEX_ERR_FORMAT;
    *text = e->text;
    if (len) *len = e->u;
    return YVEX_OK;
}

/* ---- tensor data -> resident arena ---------------------------------------------------------- */

int yvex_rocm_gguf_resident_load(yvex_rocm_backend *backend, const yvex_rocm_gguf *g,
                                         unsigned long long generation, yvex_device_tensor **arena,
                                         unsigned char **host_base, yvex_error *err)
{
    yvex_backend_tensor_desc desc;
    unsigned long long bytes, i, done = 0ull;
    unsigned char *host = NULL;
    int rc;
    if (arena) *arena = NULL;
    if (host_base) *host_base = NULL;
    if (!backend || !g || !arena || !host_base)
        return fail(err, YVEX_ERR_INVALID_ARG, "rocm.gguf.load", "backend, reader and outputs are required");
    if (!g->tensor_count || g->tensor_data_offset >= g->file_size)
        return fail(err, YVEX_ERR_FORMAT, "rocm.gguf.load", "GGUF file holds no tensor data");
    for (i = 0ull; i < g->tensor_count; ++i)
        if (!g->tensors[i].range_addressable)
            return fail(err, YVEX_ERR_BOUNDS, "rocm.gguf.load", "a GGUF tensor range ends beyond the file");
    bytes = g->file_size - g->tensor_data_offset;
    memset(&desc, 0, sizeof(desc));
    desc.name = "gguf-tensor-data";
    desc.dtype = YVEX_DTYPE_I8;
    desc.rank = 1u;
    desc.dims[0] = bytes;
    desc.bytes = bytes;
    rc = yvex_rocm_backend_resident_alloc(backend, &desc, arena, &host, err);
    if (rc != YVEX_OK) return rc;
    if (fseeko(g->file, (off_t)g->tensor_data_offset, SEEK_SET) != 0) rc = YVEX_ERR_IO;
    while (rc == YVEX_OK && done < bytes) {
        size_t want = bytes - done > (1ull << 26) ? (size_t)(1ull << 26) : (size_t)(bytes - done);
        size_t got = fread(host + done, 1u, want, g->file);
        if (!got) rc = YVEX_ERR_IO;
        done += got;
    }
    if (rc != YVEX_OK) {
        (void)yvex_rocm_backend_tensor_release(backend, arena, NULL);
        return fail(err, YVEX_ERR_IO, "rocm.gguf.load", "GGUF tensor data cannot be read");
    }
    rc = yvex_rocm_backend_resident_attach(backend, host, bytes, *arena, generation, err);
    if (rc != YVEX_OK) {
        (void)yvex_rocm_backend_tensor_release(backend, arena, NULL);
        return rc;
    }
    *host_base = host;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_gguf_weight_view(const yvex_rocm_gguf *g, const unsigned char *host_base, const char *name,
                                       yvex_moe_weight_view *view, yvex_error *err)
{
    const yvex_gguf_tensor_info *t = yvex_rocm_gguf_tensor_find(g, name);
    const yvex_rocm_qtype_geometry *geometry;
    const yvex_rocm_numeric_capability *capability;
    unsigned long long rows = 1ull;
    unsigned int d;
    if (view) memset(view, 0, sizeof(*view));
    if (!g || !host_base || !name || !view)
        return fail(err, YVEX_ERR_INVALID_ARG, "rocm.gguf.view", "reader, arena base, name and view are required");
    if (!t) return fail(err, YVEX_ERR_FORMAT, "rocm.gguf.view", "GGUF tensor is not in the directory");
    geometry = yvex_rocm_gguf_qtype_geometry_find(t->ggml_type);
    capability = yvex_rocm_quant_numeric_capability_at(t->ggml_type);
    if (!geometry || !capability || !capability->device_compute_available)
        return fail(err, YVEX_ERR_UNSUPPORTED, "rocm.gguf.view", "qtype has no device compute on this backend");
    if (!t->range_addressable)
        return fail(err, YVEX_ERR_BOUNDS, "rocm.gguf.view", "GGUF tensor range ends beyond the file");
    for (d = 1u; d < t->rank; ++d) rows *= t->dims[d];
    view->qtype = t->ggml_type;
    view->layout = t->rank >= 3u ? YVEX_EXECUTION_LAYOUT_EXPERT_MAJOR : YVEX_EXECUTION_LAYOUT_CANONICAL_ROW;
    view->activation = YVEX_EXECUTION_ACTIVATION_DEVICE_F32;
    view->encoded = host_base + t->relative_offset;
    view->encoded_bytes = (size_t)t->storage_bytes;
    view->storage_bytes = (size_t)t->storage_bytes;
    view->row_width = t->dims[0];
    view->row_count = rows;
    view->row_bytes = t->dims[0] / geometry->block_size * geometry->bytes_per_block;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
