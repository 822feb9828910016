/* Oracle, packed linear part: TEST INFRASTRUCTURE, never linked into the product.
 * Follows src/qwen4_packed.c and the helpers of src/qwen4_packed_internal.h:27-81
 * for GGUF types 0 (F32), 12 (Q4_K) and 16 (IQ2_XXS). */
#include "orc.h"
#include "../include/pf_iq2_codes.h"
#include <math.h>
#include <stdio.h>
#include <string.h>

static Qwen4Status packed_fail(Qwen4Error *err, Qwen4Status code, const char *detail) {
    /* src/qwen4_packed_internal.h:27-38: the record is rewritten on success too */
    if (err) {
        memset(err, 0, sizeof *err);
        err->code = code;
        if (code != QW4_OK) {
            snprintf(err->subject, sizeof err->subject, "packed weights");
            snprintf(err->detail, sizeof err->detail, "%s", detail);
        }
    }
    return code;
}

static bool mul_size(size_t a, size_t b, size_t *out) {
    if (a != 0 && b > SIZE_MAX / a) return false;
    *out = a * b;
    return true;
}

static bool addressable(const void *p, size_t bytes) {
    return p != NULL && bytes <= UINTPTR_MAX - (uintptr_t)p;
}

static bool ranges_overlap(const void *a, size_t na, const void *b, size_t nb) {
    uintptr_t pa = (uintptr_t)a, pb = (uintptr_t)b;
    return na != 0 && nb != 0 && pa < pb + nb && pb < pa + na;
}

/* src/gguf.c:12-16 */
const GgufFormat *orc_format(uint32_t id) {
    static const GgufFormat table[] = {
        {0, "F32", 1, 4}, {1, "F16", 1, 2}, {8, "Q8_0", 32, 34}, {10, "Q2_K", 256, 84},
        {12, "Q4_K", 256, 144}, {16, "IQ2_XXS", 256, 66}, {30, "BF16", 1, 2}, {39, "MXFP4", 32, 17},
    };
    for (size_t i = 0; i < sizeof table / sizeof table[0]; i++)
        if (table[i].id == id) return &table[i];
    return NULL;
}

/* src/qwen4_packed.c:8-33 */
Qwen4Status orc_packed_layout_init(const GgufTensor *t, size_t logical, QW4PackedLayout *out,
                                   Qwen4Error *err) {
    if (out) memset(out, 0, sizeof *out);
    if (!t || !out) return packed_fail(err, QW4_INVALID_ARGUMENT, "null descriptor/output");
    if (t->rank < 1 || t->rank > 3) return packed_fail(err, QW4_SHAPE, "expected rank 1, 2 or 3");
    const GgufFormat *f = orc_format(t->type);
    if (!f) return packed_fail(err, QW4_FORMAT, "format not executable");
    QW4PackedLayout l;
    memset(&l, 0, sizeof l);
    l.gguf_type = t->type;
    l.k_storage = t->shape[0];
    l.k_logical = logical;
    l.n_out = t->rank > 1 ? t->shape[1] : 1;
    l.n_experts = t->rank > 2 ? t->shape[2] : 1;
    if (logical == 0 || logical > l.k_storage || l.n_out == 0 || l.n_experts == 0)
        return packed_fail(err, QW4_SHAPE, "empty or incompatible dimensions");
    if (l.k_storage % f->block != 0) return packed_fail(err, QW4_FORMAT, "incomplete physical block");
    if (!mul_size(l.k_storage / f->block, f->bytes, &l.row_bytes) ||
        !mul_size(l.row_bytes, l.n_out, &l.expert_bytes) ||
        !mul_size(l.expert_bytes, l.n_experts, &l.tensor_bytes) ||
        t->file_offset > SIZE_MAX - l.tensor_bytes)
        return packed_fail(err, QW4_OVERFLOW, "tensor extent overflow");
    if (t->bytes != l.tensor_bytes)
        return packed_fail(err, QW4_FORMAT, "descriptor bytes differ from physical shape");
    *out = l;
    return packed_fail(err, QW4_OK, "");
}

/* src/qwen4_packed.c:35-50: a view is admitted only if its layout is exactly
 * what layout_init derives from its own dimensions */
static Qwen4Status check_view(const QW4PackedCpuView *w, size_t expert) {
    if (!w) return QW4_INVALID_ARGUMENT;
    const QW4PackedLayout *l = &w->layout;
    GgufTensor t;
    memset(&t, 0, sizeof t);
    t.type = l->gguf_type;
    t.rank = 3;
    t.shape[0] = l->k_storage; t.shape[1] = l->n_out; t.shape[2] = l->n_experts; t.shape[3] = 1;
    t.bytes = l->tensor_bytes;
    QW4PackedLayout want;
    Qwen4Status st = orc_packed_layout_init(&t, l->k_logical, &want, NULL);
    if (st) return st;
    if (l->gguf_type != want.gguf_type || l->k_storage != want.k_storage ||
        l->k_logical != want.k_logical || l->n_out != want.n_out || l->n_experts != want.n_experts ||
        l->row_bytes != want.row_bytes || l->expert_bytes != want.expert_bytes ||
        l->tensor_bytes != want.tensor_bytes)
        return QW4_FORMAT;
    if (expert >= l->n_experts) return QW4_RANGE;
    if (w->span.bytes < l->tensor_bytes) return QW4_CAPACITY;
    if (!addressable(w->span.data, l->tensor_bytes)) return QW4_INVALID_ARGUMENT;
    return QW4_OK;
}

/* src/qwen4_packed.c:54-66: exact binary16 -> binary32, by bit construction */
float orc_half_value(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u, m = h & 1023u, bits;
    if (e == 0 && m != 0) {
        e = 113;
        while ((m & 1024u) == 0) { m <<= 1; e--; }
        bits = sign | (e << 23) | ((m & 1023u) << 13);
    } else if (e == 0) {
        bits = sign;
    } else {
        bits = sign | ((e == 31 ? 255u : e + 112u) << 23) | (m << 13);
    }
    float v;
    memcpy(&v, &bits, 4);
    return v;
}

static uint16_t le16(const unsigned char *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* src/qwen4_packed.c:67-122 */
float orc_packed_value(const unsigned char *row, size_t column, uint32_t type) {
    if (type == 0 || type == 30) {   /* F32; BF16 = the upper half of an F32 */
        uint32_t bits;
        if (type == 30) bits = (uint32_t)le16(row + 2 * column) << 16;
        else bits = (uint32_t)le16(row + 4 * column) | ((uint32_t)le16(row + 4 * column + 2) << 16);
        float v;
        memcpy(&v, &bits, 4);
        return v;
    }
    if (type == 1) return orc_half_value(le16(row + 2 * column));
    if (type == 8) {                 /* Q8_0: half scale, 32 signed bytes */
        const unsigned char *blk = row + column / 32 * 34;
        int code = blk[2 + column % 32];
        if (code >= 128) code -= 256;
        return orc_half_value(le16(blk)) * (float)code;
    }
    if (type == 39) {                /* MXFP4: one E8M0 scale byte, 32 E2M1 codes, low nibbles first */
        static const float e2m1[16] = {0, .5f, 1, 1.5f, 2, 3, 4, 6, -0.0f, -.5f, -1, -1.5f, -2, -3, -4, -6};
        const unsigned char *blk = row + column / 32 * 17;
        unsigned lane = (unsigned)(column % 32), code = (blk[1 + lane % 16] >> ((lane / 16) * 4)) & 15u;
        uint32_t bits = blk[0] ? (uint32_t)blk[0] << 23 : 0x00400000u;   /* 2^(e - 127); e = 0 is 2^-127 */
        float scale;
        memcpy(&scale, &bits, 4);
        return e2m1[code] * scale;
    }
    if (type == 10) {                /* Q2_K: 16 scale/min nibble pairs, 64 bytes of 2-bit codes, d, dmin */
        const unsigned char *blk = row + column / 256 * 84;
        size_t lane = column % 256;
        unsigned sm = blk[lane / 16];
        unsigned code = (blk[16 + lane / 128 * 32 + lane % 32] >> (2 * (lane % 128 / 32))) & 3u;
        return (orc_half_value(le16(blk + 80)) * (float)(sm & 15u)) * (float)code -
               orc_half_value(le16(blk + 82)) * (float)(sm >> 4);
    }
    if (type == 12) {
        const unsigned char *blk = row + column / 256 * 144, *sc = blk + 4;
        size_t lane = column % 256, g = lane / 32;
        unsigned scale, minimum;
        if (g < 4) {
            scale = sc[g] & 63u;
            minimum = sc[g + 4] & 63u;
        } else {
            scale = (sc[g + 4] & 15u) | ((sc[g - 4] & 192u) >> 2);
            minimum = (sc[g + 4] >> 4) | ((sc[g] & 192u) >> 2);
        }
        unsigned code = (blk[16 + (g / 2) * 32 + lane % 32] >> ((g % 2) * 4)) & 15u;
        float d = orc_half_value(le16(blk)), dmin = orc_half_value(le16(blk + 2));
        /* ((d*scale)*code) - (dmin*minimum): three roundings, then the subtraction */
        return (d * (float)scale) * (float)code - dmin * (float)minimum;
    }
    /* type 16 */
    const unsigned char *blk = row + column / 256 * 66;
    size_t lane = column % 256, slot = lane % 32 / 8;
    const unsigned char *grp = blk + 2 + lane / 32 * 8;
    uint32_t word = (uint32_t)le16(grp + 4) | ((uint32_t)le16(grp + 6) << 16);
    unsigned signs = (word >> (7 * slot)) & 127u;
    unsigned parity = signs;
    parity ^= parity >> 4; parity ^= parity >> 2; parity ^= parity >> 1;
    signs |= (parity & 1u) << 7;
    unsigned magnitude = pf_iq2_grid_byte(grp[slot], (unsigned)(lane % 8));
    float scale = orc_half_value(le16(blk)) * (float)(2 * (word >> 28) + 1) * 0.125f;
    float v = scale * (float)magnitude;
    return (signs & (1u << (lane % 8))) ? -v : v;
}

/* src/qwen4_packed.c:124-143 */
Qwen4Status orc_packed_decode_row(const QW4PackedCpuView *w, size_t expert, size_t row, float *out,
                                  size_t count, Qwen4Error *err) {
    Qwen4Status st = check_view(w, expert);
    if (st) return packed_fail(err, st, "invalid weight view");
    size_t bytes;
    if (row >= w->layout.n_out) return packed_fail(err, QW4_RANGE, "row outside tensor");
    if (!mul_size(w->layout.k_storage, sizeof(float), &bytes))
        return packed_fail(err, QW4_OVERFLOW, "decoded row extent overflow");
    if (count < w->layout.k_storage) return packed_fail(err, QW4_CAPACITY, "short output row");
    if (!addressable(out, bytes) || (uintptr_t)out % _Alignof(float) ||
        ranges_overlap(w->span.data, w->layout.tensor_bytes, out, bytes))
        return packed_fail(err, QW4_INVALID_ARGUMENT, "invalid or aliased output");
    const unsigned char *src = w->span.data + expert * w->layout.expert_bytes + row * w->layout.row_bytes;
    for (size_t k = 0; k < w->layout.k_storage; k++) {
        float v = orc_packed_value(src, k, w->layout.gguf_type);
        if (!isfinite(v)) return packed_fail(err, QW4_NONFINITE, "nonfinite packed value");
        out[k] = v;
    }
    return packed_fail(err, QW4_OK, "");
}

/* src/qwen4_packed_internal.h:66-81 */
static Qwen4Status check_matrix(size_t rank, const size_t dim[4], const size_t stride[4], size_t capacity,
                                size_t *extent) {
    *extent = 0;
    if (rank != 2 || dim[1] == 0) return QW4_SHAPE;
    size_t width;
    if (!mul_size(dim[1], sizeof(float), &width)) return QW4_OVERFLOW;
    if (stride[1] != sizeof(float) || stride[0] % sizeof(float) || stride[0] < width) return QW4_STRIDE;
    if (dim[0]) {
        size_t prefix;
        if (!mul_size(dim[0] - 1, stride[0], &prefix) || prefix > SIZE_MAX - width) return QW4_OVERFLOW;
        *extent = prefix + width;
    }
    return *extent > capacity ? QW4_CAPACITY : QW4_OK;
}

/* src/qwen4_packed.c:145-181: rows outer, outputs, k ascending;
 * product = value * input; sum += product; finite check after every step */
Qwen4Status orc_packed_matmul(const QW4PackedCpuView *w, size_t expert, Qwen4F32 x, Qwen4F32Mut y,
                              Qwen4Error *err) {
    Qwen4Status st = check_view(w, expert);
    if (st) return packed_fail(err, st, "invalid weight view");
    size_t xbytes, ybytes;
    st = check_matrix(x.rank, x.dim, x.stride_bytes, x.capacity_bytes, &xbytes);
    if (st) return packed_fail(err, st, "invalid input matrix");
    st = check_matrix(y.rank, y.dim, y.stride_bytes, y.capacity_bytes, &ybytes);
    if (st) return packed_fail(err, st, "invalid output matrix");
    const QW4PackedLayout *l = &w->layout;
    if (x.dim[0] != y.dim[0] || x.dim[1] != l->k_logical || y.dim[1] != l->n_out)
        return packed_fail(err, QW4_SHAPE, "incompatible matrix dimensions");
    if (x.dim[0] == 0) return packed_fail(err, QW4_OK, "");
    if (!addressable(x.data, xbytes) || !addressable(y.data, ybytes) ||
        (uintptr_t)x.data % _Alignof(float) || (uintptr_t)y.data % _Alignof(float))
        return packed_fail(err, QW4_INVALID_ARGUMENT, "invalid activation address");
    if (ranges_overlap(x.data, xbytes, y.data, ybytes) ||
        ranges_overlap(w->span.data, l->tensor_bytes, x.data, xbytes) ||
        ranges_overlap(w->span.data, l->tensor_bytes, y.data, ybytes))
        return packed_fail(err, QW4_INVALID_ARGUMENT, "aliased matrices");
    const unsigned char *base = w->span.data + expert * l->expert_bytes;
    for (size_t m = 0; m < x.dim[0]; m++) {
        const float *in = x.data + m * (x.stride_bytes[0] / sizeof(float));
        float *o = y.data + m * (y.stride_bytes[0] / sizeof(float));
        for (size_t n = 0; n < l->n_out; n++) {
            const unsigned char *row = base + n * l->row_bytes;
            float sum = 0;
            for (size_t k = 0; k < l->k_logical; k++) {
                float v = orc_packed_value(row, k, l->gguf_type);
                float p = v * in[k];
                sum += p;
                if (!isfinite(v) || !isfinite(in[k]) || !isfinite(p) || !isfinite(sum))
                    return packed_fail(err, QW4_NONFINITE, "nonfinite input or arithmetic");
            }
            o[n] = sum;
        }
    }
    return packed_fail(err, QW4_OK, "");
}

/* src/qwen4_cpu_internal.h:103-107 */
float orc_sigmoid(float x) {
    if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
    float z = expf(x);
    return z / (1.0f + z);
}
float orc_silu(float x) { return x * orc_sigmoid(x); }

/* src/qwen4_base.c:76-99 for dense or pitched rank-2 views, disjoint in/out:
 * v = x / 1.0f; r = f(v); r *= 1.0f; a nonfinite result stops the call. */
Qwen4Status orc_activate(int kind, Qwen4F32 x, Qwen4F32Mut out, Qwen4Error *err) {
    if (kind != 0 && kind != 1) return packed_fail(err, QW4_UNSUPPORTED, "unknown activation");
    if (x.rank != 2 || out.rank != 2 || x.dim[0] != out.dim[0] || x.dim[1] != out.dim[1])
        return packed_fail(err, QW4_SHAPE, "activation shape");
    size_t xs = x.stride_bytes[0] / 4, os = out.stride_bytes[0] / 4;
    for (size_t r = 0; r < x.dim[0]; r++)
        for (size_t c = 0; c < x.dim[1]; c++)
            if (!isfinite(x.data[r * xs + c])) return packed_fail(err, QW4_NONFINITE, "nonfinite input");
    for (size_t r = 0; r < x.dim[0]; r++)
        for (size_t c = 0; c < x.dim[1]; c++) {
            float v = x.data[r * xs + c] / 1.0f;
            float res = kind == 0 ? orc_sigmoid(v) : orc_silu(v);
            res *= 1.0f;
            if (!isfinite(res)) return packed_fail(err, QW4_NONFINITE, "activation overflow");
            out.data[r * os + c] = res;
        }
    return packed_fail(err, QW4_OK, "");
}
