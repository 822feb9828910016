/* C11 host side of the packed linear contract (include/qwen4_packed.h).
 *
 * Admission (layout, spans, strides, aliasing) is done here in the order of the
 * reference's src/qwen4_packed.c so that status codes agree; the arithmetic runs
 * on the device through the C-ABI shim (include/pf_moe_hip.h). */
#include "../../include/qwen4_packed.h"
#include "../../include/pf_moe_hip.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static Qwen4Status packed_status(Qwen4Error *err, Qwen4Status code, const char *detail) {
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

static bool checked_mul(size_t a, size_t b, size_t *out) {
    if (a != 0 && b > SIZE_MAX / a) return false;
    *out = a * b;
    return true;
}
static bool has_extent(const void *p, size_t bytes) { return p && bytes <= UINTPTR_MAX - (uintptr_t)p; }
static bool intersects(const void *a, size_t na, const void *b, size_t nb) {
    uintptr_t pa = (uintptr_t)a, pb = (uintptr_t)b;
    return na && nb && pa < pb + nb && pb < pa + na;
}
const GgufFormat *gguf_format(uint32_t id);
static bool executable(uint32_t type) { return gguf_format(type) != NULL; }

/* Block geometry of every format the reference registers (src/gguf.c:12-16); all have kernels here. */
const GgufFormat *gguf_format(uint32_t id) {
    static const GgufFormat formats[] = {
        {0, "F32", 1, 4},      {1, "F16", 1, 2},          {8, "Q8_0", 32, 34},   {10, "Q2_K", 256, 84},
        {12, "Q4_K", 256, 144}, {16, "IQ2_XXS", 256, 66}, {30, "BF16", 1, 2},    {39, "MXFP4", 32, 17},
    };
    for (size_t i = 0; i < sizeof formats / sizeof formats[0]; i++)
        if (formats[i].id == id) return &formats[i];
    return NULL;
}

Qwen4Status qw4_packed_layout_init(const GgufTensor *t, size_t logical, QW4PackedLayout *out, Qwen4Error *err) {
    if (out) memset(out, 0, sizeof *out);
    if (!t || !out) return packed_status(err, QW4_INVALID_ARGUMENT, "null descriptor/output");
    if (t->rank < 1 || t->rank > 3) return packed_status(err, QW4_SHAPE, "expected rank 1, 2 or 3");
    const GgufFormat *f = gguf_format(t->type);
    if (!f) return packed_status(err, QW4_FORMAT, "format not executable");
    QW4PackedLayout l;
    memset(&l, 0, sizeof l);
    l.gguf_type = t->type;
    l.k_storage = t->shape[0];
    l.k_logical = logical;
    l.n_out = t->rank > 1 ? t->shape[1] : 1;
    l.n_experts = t->rank > 2 ? t->shape[2] : 1;
    if (!logical || logical > l.k_storage || !l.n_out || !l.n_experts)
        return packed_status(err, QW4_SHAPE, "empty or incompatible dimensions");
    if (l.k_storage % f->block) return packed_status(err, QW4_FORMAT, "incomplete physical block");
    if (!checked_mul(l.k_storage / f->block, f->bytes, &l.row_bytes) ||
        !checked_mul(l.row_bytes, l.n_out, &l.expert_bytes) ||
        !checked_mul(l.expert_bytes, l.n_experts, &l.tensor_bytes) || t->file_offset > SIZE_MAX - l.tensor_bytes)
        return packed_status(err, QW4_OVERFLOW, "tensor extent overflow");
    if (t->bytes != l.tensor_bytes) return packed_status(err, QW4_FORMAT, "descriptor bytes differ from physical shape");
    *out = l;
    return packed_status(err, QW4_OK, "");
}

/* Same admission as the reference's packed_view (src/qwen4_packed.c:35-50). */
/* The layout alone: a view of a tensor whose bytes are not in host memory (a streamed layer's routed tensors). */
Qwen4Status pf_layout_admit(const QW4PackedLayout *l) {
    if (!l) return QW4_INVALID_ARGUMENT;
    GgufTensor t;
    memset(&t, 0, sizeof t);
    t.type = l->gguf_type;
    t.rank = 3;
    t.shape[0] = l->k_storage; t.shape[1] = l->n_out; t.shape[2] = l->n_experts; t.shape[3] = 1;
    t.bytes = l->tensor_bytes;
    QW4PackedLayout want;
    Qwen4Status st = qw4_packed_layout_init(&t, l->k_logical, &want, NULL);
    if (st) return st;
    if (memcmp(&want.k_storage, &l->k_storage, sizeof want - offsetof(QW4PackedLayout, k_storage)) ||
        want.gguf_type != l->gguf_type)
        return QW4_FORMAT;
    return QW4_OK;
}

Qwen4Status pf_packed_admit(const QW4PackedCpuView *w, size_t expert) {
    if (!w) return QW4_INVALID_ARGUMENT;
    const QW4PackedLayout *l = &w->layout;
    Qwen4Status st = pf_layout_admit(l);
    if (st) return st;
    if (expert >= l->n_experts) return QW4_RANGE;
    if (w->span.bytes < l->tensor_bytes) return QW4_CAPACITY;
    if (!has_extent(w->span.data, l->tensor_bytes)) return QW4_INVALID_ARGUMENT;
    return QW4_OK;
}

Qwen4Status pf_device_status(int rc, Qwen4Error *err, const char *subject) {
    if (rc == PF_HIP_OK) return QW4_OK;
    Qwen4Status code = rc == PF_HIP_E_MEMORY ? QW4_OOM : rc == PF_HIP_E_UNSUPPORTED ? QW4_UNSUPPORTED
                     : rc == PF_HIP_E_ARGUMENT ? QW4_INVALID_ARGUMENT : QW4_GPU_ERROR;
    if (err) {
        memset(err, 0, sizeof *err);
        err->code = code;
        snprintf(err->subject, sizeof err->subject, "%s", subject);
        snprintf(err->detail, sizeof err->detail, "device: %s", pf_hip_last_error());
    }
    return code;
}

Qwen4Status qw4_packed_decode_row(const QW4PackedCpuView *w, size_t expert, size_t row, float *out, size_t count,
                                  Qwen4Error *err) {
    Qwen4Status st = pf_packed_admit(w, expert);
    if (st) return packed_status(err, st, "invalid weight view");
    const QW4PackedLayout *l = &w->layout;
    size_t bytes;
    if (row >= l->n_out) return packed_status(err, QW4_RANGE, "row outside tensor");
    if (!checked_mul(l->k_storage, sizeof(float), &bytes))
        return packed_status(err, QW4_OVERFLOW, "decoded row extent overflow");
    if (count < l->k_storage) return packed_status(err, QW4_CAPACITY, "short output row");
    if (!has_extent(out, bytes) || (uintptr_t)out % _Alignof(float) ||
        intersects(w->span.data, l->tensor_bytes, out, bytes))
        return packed_status(err, QW4_INVALID_ARGUMENT, "invalid or aliased output");
    if (!executable(l->gguf_type)) return packed_status(err, QW4_UNSUPPORTED, "format has no device kernel");
    uint32_t word = 0;
    int rc = pf_hip_packed_decode_row_host(l->gguf_type, w->span.data + expert * l->expert_bytes + row * l->row_bytes,
                                           l->row_bytes, l->k_storage, out, &word);
    if (rc) return pf_device_status(rc, err, "packed weights");
    if (word & PF_HIP_ERR_NONFINITE) return packed_status(err, QW4_NONFINITE, "nonfinite packed value");
    if (word) return packed_status(err, QW4_GPU_ERROR, "device error word");
    return packed_status(err, QW4_OK, "");
}

/* src/qwen4_packed_internal.h:66-81 */
static Qwen4Status admit_matrix(size_t rank, const size_t dim[4], const size_t stride[4], size_t capacity,
                                size_t *extent) {
    *extent = 0;
    if (rank != 2 || !dim[1]) return QW4_SHAPE;
    size_t width;
    if (!checked_mul(dim[1], sizeof(float), &width)) return QW4_OVERFLOW;
    if (stride[1] != sizeof(float) || stride[0] % sizeof(float) || stride[0] < width) return QW4_STRIDE;
    if (dim[0]) {
        size_t prefix;
        if (!checked_mul(dim[0] - 1, stride[0], &prefix) || prefix > SIZE_MAX - width) return QW4_OVERFLOW;
        *extent = prefix + width;
    }
    return *extent > capacity ? QW4_CAPACITY : QW4_OK;
}

Qwen4Status qw4_packed_matmul(const QW4PackedCpuView *w, size_t expert, Qwen4F32 x, Qwen4F32Mut y, Qwen4Error *err) {
    Qwen4Status st = pf_packed_admit(w, expert);
    if (st) return packed_status(err, st, "invalid weight view");
    size_t xbytes, ybytes;
    st = admit_matrix(x.rank, x.dim, x.stride_bytes, x.capacity_bytes, &xbytes);
    if (st) return packed_status(err, st, "invalid input matrix");
    st = admit_matrix(y.rank, y.dim, y.stride_bytes, y.capacity_bytes, &ybytes);
    if (st) return packed_status(err, st, "invalid output matrix");
    const QW4PackedLayout *l = &w->layout;
    if (x.dim[0] != y.dim[0] || x.dim[1] != l->k_logical || y.dim[1] != l->n_out)
        return packed_status(err, QW4_SHAPE, "incompatible matrix dimensions");
    if (!x.dim[0]) return packed_status(err, QW4_OK, "");
    if (!has_extent(x.data, xbytes) || !has_extent(y.data, ybytes) || (uintptr_t)x.data % _Alignof(float) ||
        (uintptr_t)y.data % _Alignof(float))
        return packed_status(err, QW4_INVALID_ARGUMENT, "invalid activation address");
    if (intersects(x.data, xbytes, y.data, ybytes) || intersects(w->span.data, l->tensor_bytes, x.data, xbytes) ||
        intersects(w->span.data, l->tensor_bytes, y.data, ybytes))
        return packed_status(err, QW4_INVALID_ARGUMENT, "aliased matrices");
    if (!executable(l->gguf_type)) return packed_status(err, QW4_UNSUPPORTED, "format has no device kernel");
    const size_t rows = x.dim[0], K = l->k_logical, N = l->n_out;
    /* dense staging copies: the shim takes unpitched matrices */
    float *xd = malloc(rows * K * sizeof(float)), *yd = malloc(rows * N * sizeof(float));
    if (!xd || !yd) { free(xd); free(yd); return packed_status(err, QW4_OOM, "staging"); }
    for (size_t m = 0; m < rows; m++) memcpy(xd + m * K, x.data + m * (x.stride_bytes[0] / 4), K * 4);
    uint32_t word = 0;
    int rc = pf_hip_packed_matmul_host(l->gguf_type, w->span.data + expert * l->expert_bytes, l->row_bytes, N, K, xd,
                                       rows, yd, &word);
    if (rc == PF_HIP_OK && word == 0)
        for (size_t m = 0; m < rows; m++) memcpy(y.data + m * (y.stride_bytes[0] / 4), yd + m * N, N * 4);
    free(xd);
    free(yd);
    if (rc) return pf_device_status(rc, err, "packed weights");
    if (word & PF_HIP_ERR_NONFINITE) return packed_status(err, QW4_NONFINITE, "nonfinite input or arithmetic");
    if (word) return packed_status(err, QW4_GPU_ERROR, "device error word");
    return packed_status(err, QW4_OK, "");
}
