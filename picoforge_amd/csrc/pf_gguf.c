/* GGUF v3 checkpoints as the source of the MoE block's weights (include/pf_gguf.h).
 *
 * Host-only C11.  The header is decoded through a cursor that remembers its first
 * failure, so decoding code reads straight through and the status is looked at once
 * per descriptor; where the reference's reader ends the process (src/gguf_reader.c,
 * src/gguf.c) this one returns.  Nothing here touches the device except
 * pf_gguf_moe_create, which goes through qwen4_moe_create. */
#define _DEFAULT_SOURCE
#include "../../include/pf_gguf.h"
#include <errno.h>
#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

_Static_assert(sizeof(size_t) == 8, "GGUF offsets need a 64-bit host");

#define HEADER_LIMIT ((size_t)128 << 20)   /* src/gguf.c:39 */
#define MAX_DESCRIPTORS 100000u            /* src/gguf.c:47 */
#define MAX_STRING ((uint64_t)16 << 20)    /* src/gguf_reader.c:35 */
#define MAX_ARRAY 2000000u                 /* src/gguf_reader.c:64 */

typedef struct { char name[128]; uint32_t type; size_t offset, bytes; } Meta;

struct PfGguf {
    int fd;
    const unsigned char *map;      /* the whole file, read-only */
    size_t file_size, header_size, data_offset, tensor_count, meta_count;
    GgufTensor *tensors;           /* sorted by file offset */
    Meta *meta;
};

/* ---- error records ---- */

static Qwen4Status fail(Qwen4Error *err, Qwen4Status code, const char *subject, const char *detail) {
    if (err) {
        memset(err, 0, sizeof *err);
        err->code = code;
        snprintf(err->subject, sizeof err->subject, "%s", subject ? subject : "");
        snprintf(err->detail, sizeof err->detail, "%s", detail ? detail : "");
    }
    return code;
}

/* ---- cursor with a sticky first failure ---- */

typedef struct {
    const unsigned char *data;
    size_t size, pos;
    Qwen4Status status;
    const char *why;
} Cursor;

static void cur_fail(Cursor *c, Qwen4Status s, const char *why) {
    if (c->status == QW4_OK) { c->status = s; c->why = why; }
}

static const unsigned char *cur_take(Cursor *c, size_t n) {
    if (c->status != QW4_OK) return NULL;
    if (c->pos > c->size || n > c->size - c->pos) {
        cur_fail(c, QW4_FORMAT, "gguf: truncated or oversized header");
        return NULL;
    }
    const unsigned char *p = c->data + c->pos;
    c->pos += n;
    return p;
}

static uint64_t cur_uint(Cursor *c, size_t width) {
    const unsigned char *p = cur_take(c, width);
    uint64_t v = 0;
    if (p) for (size_t i = width; i-- > 0;) v = v << 8 | p[i];
    return v;
}

static const unsigned char *cur_string(Cursor *c, size_t *length) {
    uint64_t n = cur_uint(c, 8);
    *length = 0;
    if (c->status != QW4_OK) return NULL;
    if (n > MAX_STRING) { cur_fail(c, QW4_FORMAT, "gguf: oversized string"); return NULL; }
    *length = (size_t)n;
    return cur_take(c, *length);
}

static bool identifier_byte(unsigned char b) {
    return (b >= 'a' && b <= 'z') || (b >= 'A' && b <= 'Z') || (b >= '0' && b <= '9') || b == '_' || b == '.' || b == '-';
}

/* A descriptor name: 1..capacity-1 identifier bytes (src/gguf_reader.c:40-52). */
static void cur_name(Cursor *c, char *out, size_t capacity) {
    size_t n;
    const unsigned char *p = cur_string(c, &n);
    out[0] = 0;
    if (!p) return;
    if (n == 0 || n >= capacity) { cur_fail(c, QW4_FORMAT, "gguf: invalid name length"); return; }
    for (size_t i = 0; i < n; i++)
        if (!identifier_byte(p[i])) { cur_fail(c, QW4_FORMAT, "gguf: unsupported identifier byte"); return; }
    memcpy(out, p, n);
    out[n] = 0;
}

/* Width in bytes of the fixed-size metadata value types 0..12; strings (8) and arrays (9) are 0. */
static const unsigned char value_width[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};

static void cur_skip_value(Cursor *c, uint32_t type) {
    if (c->status != QW4_OK) return;
    if (type > 12) { cur_fail(c, QW4_FORMAT, "gguf: unsupported metadata type"); return; }
    if (type == 8) {
        size_t n;
        (void)cur_string(c, &n);
    } else if (type == 9) {
        uint32_t element = (uint32_t)cur_uint(c, 4);
        uint64_t count = cur_uint(c, 8);
        if (c->status != QW4_OK) return;
        if (element > 12 || element == 9 || count > MAX_ARRAY) { cur_fail(c, QW4_FORMAT, "gguf: invalid metadata array"); return; }
        for (uint64_t i = 0; i < count && c->status == QW4_OK; i++) cur_skip_value(c, element);
    } else if (type == 7) {
        if (cur_uint(c, 1) > 1) cur_fail(c, QW4_FORMAT, "gguf: invalid boolean");
    } else {
        (void)cur_take(c, value_width[type]);
    }
}

/* ---- open ---- */

static int cmp_tensor_name(const void *a, const void *b) {
    return strcmp(((const GgufTensor *)a)->name, ((const GgufTensor *)b)->name);
}
static int cmp_meta_name(const void *a, const void *b) { return strcmp(((const Meta *)a)->name, ((const Meta *)b)->name); }
static int cmp_tensor_offset(const void *a, const void *b) {
    size_t x = ((const GgufTensor *)a)->file_offset, y = ((const GgufTensor *)b)->file_offset;
    return (x > y) - (x < y);
}

static bool mul_ok(size_t a, size_t b, size_t *out) {
    if (a && b > SIZE_MAX / a) return false;
    *out = a * b;
    return true;
}

static Qwen4Status decode_header(PfGguf *g, Qwen4Error *err) {
    Cursor c = {g->map, g->header_size, 0, QW4_OK, NULL};
    const unsigned char *magic = cur_take(&c, 4);
    uint64_t version = cur_uint(&c, 4);
    if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);
    if (memcmp(magic, "GGUF", 4) != 0 || version != 3) return fail(err, QW4_FORMAT, "gguf", "gguf: expected little-endian GGUF v3");
    uint64_t n_tensors = cur_uint(&c, 8), n_meta = cur_uint(&c, 8);
    if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);
    if (n_tensors == 0 || n_tensors > MAX_DESCRIPTORS || n_meta > MAX_DESCRIPTORS)
        return fail(err, QW4_FORMAT, "gguf", "gguf: invalid descriptor counts");
    g->tensor_count = (size_t)n_tensors;
    g->meta_count = (size_t)n_meta;
    g->tensors = calloc(g->tensor_count, sizeof *g->tensors);
    g->meta = calloc(g->meta_count + 1, sizeof *g->meta);
    if (!g->tensors || !g->meta) return fail(err, QW4_OOM, "gguf", "gguf: descriptor allocation failed");

    size_t alignment = 32;
    bool qwen4exp = false;
    for (size_t i = 0; i < g->meta_count; i++) {
        Meta *m = &g->meta[i];
        cur_name(&c, m->name, sizeof m->name);
        m->type = (uint32_t)cur_uint(&c, 4);
        m->offset = c.pos;
        cur_skip_value(&c, m->type);
        if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);
        m->bytes = c.pos - m->offset;
        if (!strcmp(m->name, "general.architecture")) {
            if (m->type != 8) return fail(err, QW4_FORMAT, "gguf", "gguf: architecture must be a string");
            qwen4exp = m->bytes == 16 && !memcmp(g->map + m->offset + 8, "qwen4exp", 8);
        } else if (!strcmp(m->name, "general.alignment")) {
            if (m->type != 4) return fail(err, QW4_FORMAT, "gguf", "gguf: alignment must be uint32");
            Cursor v = {g->map, c.pos, m->offset, QW4_OK, NULL};
            alignment = (size_t)cur_uint(&v, 4);
        }
    }
    qsort(g->meta, g->meta_count, sizeof *g->meta, cmp_meta_name);
    for (size_t i = 1; i < g->meta_count; i++)
        if (!strcmp(g->meta[i - 1].name, g->meta[i].name)) return fail(err, QW4_FORMAT, "gguf", "gguf: duplicate metadata key");
    if (!qwen4exp) return fail(err, QW4_UNSUPPORTED, "gguf", "gguf: expected qwen4exp architecture");
    if (alignment == 0 || (alignment & (alignment - 1)) || alignment > HEADER_LIMIT)
        return fail(err, QW4_FORMAT, "gguf", "gguf: invalid alignment");

    for (size_t i = 0; i < g->tensor_count; i++) {
        GgufTensor *t = &g->tensors[i];
        cur_name(&c, t->name, sizeof t->name);
        t->rank = (uint32_t)cur_uint(&c, 4);
        if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);
        if (t->rank == 0 || t->rank > 4) return fail(err, QW4_FORMAT, "gguf", "gguf: invalid tensor rank");
        for (uint32_t d = 0; d < t->rank; d++) {
            t->shape[d] = (size_t)cur_uint(&c, 8);
            if (c.status == QW4_OK && t->shape[d] == 0) return fail(err, QW4_FORMAT, "gguf", "gguf: zero tensor dimension");
        }
        t->type = (uint32_t)cur_uint(&c, 4);
        t->file_offset = (size_t)cur_uint(&c, 8);      /* relative to the data section until all are read */
        if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);
        const GgufFormat *f = gguf_format(t->type);
        char text[200];
        if (!f) {
            snprintf(text, sizeof text, "gguf: unsupported tensor format %u", t->type);
            return fail(err, QW4_FORMAT, t->name, text);
        }
        if (t->shape[0] % f->block || t->file_offset % alignment) {
            snprintf(text, sizeof text, "gguf: unaligned tensor row or offset: %s", t->name);
            return fail(err, QW4_FORMAT, t->name, text);
        }
        bool fits = mul_ok(t->shape[0] / f->block, f->bytes, &t->bytes);
        for (uint32_t d = 1; d < t->rank && fits; d++) fits = mul_ok(t->bytes, t->shape[d], &t->bytes);
        if (!fits) return fail(err, QW4_OVERFLOW, t->name, "gguf: size overflow");
    }
    if (alignment - 1 > SIZE_MAX - c.pos) return fail(err, QW4_OVERFLOW, "gguf", "gguf: offset overflow");
    g->data_offset = (c.pos + alignment - 1) & ~(alignment - 1);
    (void)cur_take(&c, g->data_offset - c.pos);        /* the padding up to the data section must be there */
    if (c.status != QW4_OK) return fail(err, c.status, "gguf", c.why);

    qsort(g->tensors, g->tensor_count, sizeof *g->tensors, cmp_tensor_name);
    for (size_t i = 1; i < g->tensor_count; i++)
        if (!strcmp(g->tensors[i - 1].name, g->tensors[i].name)) return fail(err, QW4_FORMAT, g->tensors[i].name, "gguf: duplicate tensor name");
    qsort(g->tensors, g->tensor_count, sizeof *g->tensors, cmp_tensor_offset);
    size_t end = g->data_offset;
    for (size_t i = 0; i < g->tensor_count; i++) {
        GgufTensor *t = &g->tensors[i];
        if (t->file_offset > SIZE_MAX - g->data_offset) return fail(err, QW4_OVERFLOW, t->name, "gguf: offset overflow");
        t->file_offset += g->data_offset;
        if (t->file_offset < end || t->file_offset > g->file_size || t->bytes > g->file_size - t->file_offset) {
            char text[200];
            snprintf(text, sizeof text, "gguf: overlapping or out-of-file tensor: %s", t->name);
            return fail(err, QW4_FORMAT, t->name, text);
        }
        end = t->file_offset + t->bytes;
    }
    return QW4_OK;
}

Qwen4Status pf_gguf_open(const char *path, PfGguf **out, Qwen4Error *err) {
    if (out) *out = NULL;
    if (!path || !out) return fail(err, QW4_INVALID_ARGUMENT, "gguf", "null argument");
    PfGguf *g = calloc(1, sizeof *g);
    if (!g) return fail(err, QW4_OOM, "gguf", "gguf: descriptor allocation failed");
    g->fd = open(path, O_RDONLY | O_CLOEXEC);
    struct stat st;
    if (g->fd < 0 || fstat(g->fd, &st) != 0 || !S_ISREG(st.st_mode) || st.st_size < 24) {
        int code = errno;
        Qwen4Status s = fail(err, QW4_IO, "gguf", "gguf: cannot open a complete regular file");
        if (err) err->os_errno = g->fd < 0 ? code : 0;
        pf_gguf_close(g);
        return s;
    }
    g->file_size = (size_t)st.st_size;
    g->header_size = g->file_size < HEADER_LIMIT ? g->file_size : HEADER_LIMIT;
    void *map = mmap(NULL, g->file_size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (map == MAP_FAILED) {
        int code = errno;
        Qwen4Status s = fail(err, QW4_IO, "gguf", "gguf: header mapping failed");
        if (err) err->os_errno = code;
        pf_gguf_close(g);
        return s;
    }
    g->map = map;
    Qwen4Status s = decode_header(g, err);
    if (s != QW4_OK) { pf_gguf_close(g); return s; }
    *out = g;
    return fail(err, QW4_OK, NULL, NULL);
}

void pf_gguf_close(PfGguf *g) {
    if (!g) return;
    if (g->map) munmap((void *)g->map, g->file_size);
    if (g->fd >= 0) close(g->fd);
    free(g->tensors);
    free(g->meta);
    free(g);
}

size_t pf_gguf_tensor_count(const PfGguf *g) { return g ? g->tensor_count : 0; }
const GgufTensor *pf_gguf_tensor(const PfGguf *g, size_t index) {
    return g && index < g->tensor_count ? &g->tensors[index] : NULL;
}
const GgufTensor *pf_gguf_find(const PfGguf *g, const char *name) {
    if (!g || !name) return NULL;
    for (size_t i = 0; i < g->tensor_count; i++)
        if (!strcmp(g->tensors[i].name, name)) return &g->tensors[i];
    return NULL;
}
size_t pf_gguf_data_offset(const PfGguf *g) { return g ? g->data_offset : 0; }
size_t pf_gguf_file_size(const PfGguf *g) { return g ? g->file_size : 0; }
const unsigned char *pf_gguf_tensor_bytes(const PfGguf *g, const GgufTensor *t) {
    if (!g || !t || t < g->tensors || t >= g->tensors + g->tensor_count) return NULL;
    return g->map + t->file_offset;
}

/* ---- metadata the MoE path reads ---- */

/* The value bytes of a key of a given type (the job of qw4a_meta, src/qwen4_config.c:6-27). */
static Qwen4Status meta_value(const PfGguf *g, const char *key, uint32_t type, const unsigned char **data, size_t *bytes,
                              Qwen4Error *err) {
    const Meta *found = NULL;
    for (size_t i = 0; i < g->meta_count; i++)
        if (!strcmp(g->meta[i].name, key)) found = &g->meta[i];   /* duplicates were refused at open */
    if (!found) return fail(err, QW4_MISSING, key, "required metadata");
    if (found->type != type) return fail(err, QW4_TYPE, key, "metadata type");
    *data = g->map + found->offset;
    *bytes = found->bytes;
    return QW4_OK;
}

static uint32_t le32(const unsigned char *p) { return (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 | (uint32_t)p[3] << 24; }

static Qwen4Status meta_u32(const PfGguf *g, const char *key, uint32_t *out, Qwen4Error *err) {
    const unsigned char *p;
    size_t n;
    Qwen4Status s = meta_value(g, key, 4, &p, &n, err);
    if (s != QW4_OK) return s;
    if (n != 4) return fail(err, QW4_FORMAT, key, "uint32 width");
    *out = le32(p);
    return QW4_OK;
}

/* A dimension: uint32 and not zero; the subject of the zero error is the key without its prefix
 * (src/qwen4_config.c:158-160). */
static Qwen4Status meta_dim(const PfGguf *g, const char *short_key, uint32_t *out, Qwen4Error *err) {
    char key[160];
    snprintf(key, sizeof key, "qwen4exp.%s", short_key);
    Qwen4Status s = meta_u32(g, key, out, err);
    if (s != QW4_OK) return s;
    if (*out == 0) return fail(err, QW4_RANGE, short_key, "positive dimension");
    return QW4_OK;
}

static Qwen4Status meta_positive_float(const PfGguf *g, const char *key, float *out, Qwen4Error *err) {
    const unsigned char *p;
    size_t n;
    Qwen4Status s = meta_value(g, key, 6, &p, &n, err);
    if (s != QW4_OK) return s;
    if (n != 4) return fail(err, QW4_FORMAT, key, "float32 width");
    uint32_t bits = le32(p);
    memcpy(out, &bits, 4);
    if (!isfinite(*out)) return fail(err, QW4_NONFINITE, key, "finite value required");
    if (*out <= 0) return fail(err, QW4_RANGE, key, "positive value required");
    return QW4_OK;
}

/* Every qwen4exp.* key must be one the reference knows (src/qwen4_config.c:61-84): an unknown
 * one could change what the numbers mean. */
static Qwen4Status admit_keys(const PfGguf *g, Qwen4Error *err) {
    static const char *const known[] = {
        "attention.compress_ratios", "attention.head_count", "attention.head_count_kv", "attention.indexer.head_count",
        "attention.indexer.key_length", "attention.indexer.top_k", "attention.key_length",
        "attention.layer_norm_rms_epsilon", "attention.value_length", "block_count", "context_length",
        "embedding_length", "embedding_length_per_layer_input", "expert_count", "expert_feed_forward_length",
        "expert_shared_feed_forward_length", "expert_used_count", "full_attention_interval", "hyper_connection.count",
        "hyper_connection.low_rank", "nextn_predict_layers", "ple.conv_kernel", "ple.eos_token_id", "ple.head_offsets",
        "ple.head_vocab_sizes", "ple.heads_per_ngram", "ple.layer_multipliers", "ple.layers", "ple.ngram_size",
        "ple.row_count", "ple.row_dimension", "ple.seed", "ple.vocab_base", "ple.vocab_divisor", "rope.dimension_count",
        "rope.freq_base", "ssm.conv_kernel", "ssm.group_count", "ssm.inner_size", "ssm.output_gate_type",
        "ssm.state_size", "ssm.time_step_rank", "vocab_size"};
    for (size_t i = 0; i < g->meta_count; i++) {
        const char *key = g->meta[i].name;
        if (strncmp(key, "qwen4exp.", 9) != 0) continue;
        bool ok = false;
        for (size_t j = 0; j < sizeof known / sizeof *known && !ok; j++) ok = !strcmp(key + 9, known[j]);
        if (!ok) return fail(err, QW4_UNSUPPORTED, "config", "unknown computational metadata");
    }
    return QW4_OK;
}

Qwen4Status pf_gguf_moe_model(const PfGguf *g, PfGgufMoeModel *out, Qwen4Error *err) {
    if (!g || !out) return fail(err, QW4_INVALID_ARGUMENT, "config", "null argument");
    PfGgufMoeModel m;
    memset(&m, 0, sizeof m);
    Qwen4Status s = admit_keys(g, err);
    if (s != QW4_OK) return s;
    uint32_t hidden, streams, low_rank;
    /* in the order the reference reads them, so that a file with several faults reports the same one */
    if ((s = meta_dim(g, "block_count", &m.blocks, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "embedding_length", &hidden, err)) != QW4_OK) return s;
    if ((s = meta_u32(g, "qwen4exp.nextn_predict_layers", &m.mtp_blocks, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "expert_count", &m.moe.experts, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "expert_used_count", &m.moe.top_k, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "expert_feed_forward_length", &m.moe.intermediate, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "expert_shared_feed_forward_length", &m.moe.shared_intermediate, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "hyper_connection.count", &streams, err)) != QW4_OK) return s;
    if ((s = meta_dim(g, "hyper_connection.low_rank", &low_rank, err)) != QW4_OK) return s;
    float eps;
    if ((s = meta_positive_float(g, "qwen4exp.attention.layer_norm_rms_epsilon", &eps, err)) != QW4_OK) return s;

    /* The two profiles of trunk experts, told apart by layer 0's routed tensors (src/qwen4_config.c:197-216). */
    const GgufTensor *gate = pf_gguf_find(g, "blk.0.ffn_gate_exps.weight"), *down = pf_gguf_find(g, "blk.0.ffn_down_exps.weight");
    if (!gate || !down) return fail(err, QW4_FORMAT, "experts", "layer 0 routed expert tensors");
    if (gate->type == 16 && down->type == 10) {
        uint32_t logical;
        if ((s = meta_u32(g, "ds4.qwen4.down.logical_input", &logical, err)) != QW4_OK) return s;
        if (logical != m.moe.intermediate) return fail(err, QW4_SHAPE, "down", "logical K mismatch");
        if ((s = meta_u32(g, "ds4.qwen4.down.physical_input", &m.moe.down_physical, err)) != QW4_OK) return s;
        m.moe.trunk_type[0] = m.moe.trunk_type[1] = 16;
        m.moe.trunk_type[2] = 10;
        m.semantic_profile = "qwen38-q2-text-f32-v1";
    } else if (gate->type == 12 && down->type == 39) {
        m.moe.down_physical = m.moe.intermediate;
        m.moe.trunk_type[0] = m.moe.trunk_type[1] = 12;
        m.moe.trunk_type[2] = 39;
        m.semantic_profile = "qwen38-q4-text-f32-v1";
    } else {
        return fail(err, QW4_UNSUPPORTED, "experts", "routed expert formats are neither the Q2 nor the Q4 profile");
    }
    m.moe.norm_topk_prob = true;           /* not exported to GGUF; the checkpoint's fixed profile (src/qwen4_config.c:217-220) */
    m.moe.hidden_size = hidden;
    m.hc = (Qwen4HcShape){.streams = streams, .hidden_size = hidden, .low_rank = low_rank, .rms_eps = eps};

    /* the checks of validate_fields that concern these fields (src/qwen4_config.c:33-54) */
    if (m.blocks > 4096 || m.mtp_blocks >= m.blocks) return fail(err, QW4_RANGE, "config", "layer/order admission");
    m.trunk_blocks = m.blocks - m.mtp_blocks;
    if (m.moe.top_k > m.moe.experts) return fail(err, QW4_SHAPE, "config", "head/rotary/expert dimensions");
    uint64_t padded = m.moe.trunk_type[2] == 10 ? ((uint64_t)m.moe.intermediate + 255) / 256 * 256 : m.moe.intermediate;
    if (padded > UINT32_MAX || padded != m.moe.down_physical)
        return fail(err, QW4_SHAPE, "down", "physical K must round logical K to 256");
    if ((uint64_t)hidden * streams > UINT32_MAX) return fail(err, QW4_OVERFLOW, "config", "derived dimension exceeds uint32");
    *out = m;
    return fail(err, QW4_OK, NULL, NULL);
}

Qwen4Status pf_gguf_moe_layer_config(const PfGgufMoeModel *model, uint32_t layer, Qwen4MoeConfig *out, Qwen4Error *err) {
    if (!model || !out) return fail(err, QW4_INVALID_ARGUMENT, "weights", "null argument");
    if (layer >= model->blocks) return fail(err, QW4_RANGE, "weights", "layer/role index");
    *out = model->moe;
    if (layer >= model->trunk_blocks) {
        out->trunk_type[0] = out->trunk_type[1] = 12;
        out->trunk_type[2] = 39;
        out->down_physical = out->intermediate;
    }
    return fail(err, QW4_OK, NULL, NULL);
}

/* ---- the eight tensors of one layer ---- */

typedef struct {
    const char *suffix;
    uint32_t type, rank;
    size_t k, n, experts, k_logical;
} Row;

/* One catalog row: presence, format, rank, physical shape, byte count (src/qwen4_weights.c:19-48),
 * then the view the packed contract takes (src/qwen4_forward.c:72-79). */
static Qwen4Status bind_row(const PfGguf *g, uint32_t layer, const Row *r, QW4PackedCpuView *view, Qwen4Error *err) {
    char name[128];
    snprintf(name, sizeof name, "blk.%u.%s", layer, r->suffix);
    const GgufTensor *t = pf_gguf_find(g, name);
    if (!t) return fail(err, QW4_MISSING, name, "required tensor");
    if (t->type != r->type) return fail(err, QW4_FORMAT, name, "Q2 recipe format mismatch");
    const size_t shape[4] = {r->k, r->n, r->experts, 1};
    if (t->rank != r->rank) return fail(err, QW4_SHAPE, name, "rank mismatch");
    for (uint32_t i = 0; i < r->rank; i++)
        if (t->shape[i] != shape[i]) return fail(err, QW4_SHAPE, name, "physical shape mismatch");
    const GgufFormat *f = gguf_format(r->type);
    if (!f || r->k == 0 || r->k % f->block || r->k_logical == 0 || r->k_logical > r->k)
        return fail(err, QW4_SHAPE, name, "packed row alignment");
    size_t row, plane, bytes;
    if (!mul_ok(r->k / f->block, f->bytes, &row) || !mul_ok(row, r->n, &plane) || !mul_ok(plane, r->experts, &bytes))
        return fail(err, QW4_OVERFLOW, name, "tensor extent");
    if (bytes != t->bytes) return fail(err, QW4_FORMAT, name, "physical byte count");
    Qwen4Status s = qw4_packed_layout_init(t, r->k_logical, &view->layout, err);
    if (s != QW4_OK) return s;
    view->span = (Qwen4CpuSpan){g->map + t->file_offset, t->bytes};
    return QW4_OK;
}

Qwen4Status pf_gguf_moe_weights(const PfGguf *g, const PfGgufMoeModel *model, uint32_t layer, Qwen4MoeWeights *out,
                                Qwen4Error *err) {
    if (!g || !model || !out) return fail(err, QW4_INVALID_ARGUMENT, "weights", "null argument");
    Qwen4MoeConfig c;
    Qwen4Status s = pf_gguf_moe_layer_config(model, layer, &c, err);
    if (s != QW4_OK) return s;
    const size_t d = c.hidden_size, f = c.intermediate, fs = c.shared_intermediate, ne = c.experts;
    /* in the catalog's order (src/qwen4_weights.c:91-99) */
    const Row rows[8] = {
        {"ffn_gate_inp.weight", 0, 2, d, ne, 1, d},
        {"ffn_gate_inp_shexp.weight", 0, 1, d, 1, 1, d},
        {"ffn_gate_shexp.weight", 8, 2, d, fs, 1, d},
        {"ffn_up_shexp.weight", 8, 2, d, fs, 1, d},
        {"ffn_down_shexp.weight", 8, 2, fs, d, 1, fs},
        {"ffn_gate_exps.weight", c.trunk_type[0], 3, d, f, ne, d},
        {"ffn_up_exps.weight", c.trunk_type[1], 3, d, f, ne, d},
        {"ffn_down_exps.weight", c.trunk_type[2], 3, c.down_physical, d, ne, f},
    };
    Qwen4MoeWeights w;
    memset(&w, 0, sizeof w);
    QW4PackedCpuView *const views[8] = {&w.router, &w.shared_router, &w.shared_gate, &w.shared_up, &w.shared_down,
                                        &w.gate, &w.up, &w.down};
    for (int i = 0; i < 8; i++)
        if ((s = bind_row(g, layer, &rows[i], views[i], err)) != QW4_OK) return s;
    *out = w;
    return fail(err, QW4_OK, NULL, NULL);
}

Qwen4Status pf_gguf_moe_create(const PfGguf *g, const PfGgufMoeModel *model, uint32_t layer, Qwen4Moe **out,
                               Qwen4Error *err) {
    if (out) *out = NULL;
    if (!g || !model || !out) return fail(err, QW4_INVALID_ARGUMENT, "weights", "null argument");
    Qwen4MoeWeights w;
    Qwen4MoeConfig c;
    Qwen4Status s = pf_gguf_moe_weights(g, model, layer, &w, err);
    if (s != QW4_OK) return s;
    if ((s = pf_gguf_moe_layer_config(model, layer, &c, err)) != QW4_OK) return s;
    s = qwen4_moe_create(&c, &w, out, err);
    /* the layer may outlive the mapping: its views are not compared with the file's addresses later */
    if (s == QW4_OK) pf_moe_forget_host_weights(*out);
    return s;
}
