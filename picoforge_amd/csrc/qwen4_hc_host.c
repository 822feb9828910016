/* C11 host side of the two hyper-connection steps either side of the MoE block
 * (include/qwen4_hc.h): the reference's preflight validation in the reference's
 * order (src/qwen4_base.c:127-175, src/qwen4_cpu_internal.h:38-122), then the
 * HIP kernels behind include/pf_moe_hip.h.  No CPU fallback: without a device
 * both operators fail.  Nonfinite inputs are found by the kernels while they
 * stream the data, so a call that reports QW4_NONFINITE leaves its output
 * untouched (the reference's CPU loop has written the elements before an
 * overflowing one by then). */
#include "../../include/qwen4_hc.h"
#include "../../include/pf_moe_hip.h"
#include "pf_hc_host.h"
#include <math.h>
#include <stdio.h>
#include <string.h>

Qwen4Status pf_device_status(int rc, Qwen4Error *err, const char *subject);   /* qwen4_packed_host.c */

static Qwen4Status hc_status(Qwen4Error *err, Qwen4Status code, const char *detail) {
    if (err) {
        memset(err, 0, sizeof *err);
        err->code = code;
        if (code != QW4_OK) {
            snprintf(err->subject, sizeof err->subject, "qwen4/C");
            snprintf(err->detail, sizeof err->detail, "%s", detail);
        }
    }
    return code;
}
#define TRY(expr) do { Qwen4Status st_ = (expr); if (st_ != QW4_OK) return st_; } while (0)

/* src/qwen4_cpu_internal.h:38-62 and :109-114: layout from the innermost axis out, then the
 * pointer, then rank and dimensions.  *span receives the bytes from the first element to the end
 * of the last one (0 for an empty view). */
Qwen4Status pf_hc_admit_view(const float *data, size_t capacity, size_t rank, const size_t dim[4],
                             const size_t stride[4], size_t want_rank, const size_t *want_dim, size_t *span,
                             Qwen4Error *err) {
    *span = 0;
    if (rank < 1 || rank > QWEN4_MAX_RANK) return hc_status(err, QW4_SHAPE, "rank must be 1..4");
    size_t bytes = sizeof(float);
    for (size_t axis = rank; axis-- > 0;) {
        if (!dim[axis] && axis) return hc_status(err, QW4_SHAPE, "only the first axis may be empty");
        if (dim[axis] > UINT32_MAX) return hc_status(err, QW4_RANGE, "dimension exceeds uint32");
        const size_t pitch = stride[axis];
        if (pitch % sizeof(float) || pitch < bytes || (axis == rank - 1 && pitch != sizeof(float)))
            return hc_status(err, QW4_STRIDE, "noncontiguous feature or overlapping axes");
        if (dim[axis]) {
            const size_t steps = dim[axis] - 1;
            if ((pitch && steps > SIZE_MAX / pitch) || steps * pitch > SIZE_MAX - bytes)
                return hc_status(err, QW4_OVERFLOW, "view span overflows");
            bytes += steps * pitch;
        }
    }
    if (dim[0]) {
        if (!data) return hc_status(err, QW4_INVALID_ARGUMENT, "null nonempty view");
        if ((uintptr_t)data % _Alignof(float)) return hc_status(err, QW4_STRIDE, "unaligned float pointer");
        if (bytes > UINTPTR_MAX - (uintptr_t)data) return hc_status(err, QW4_OVERFLOW, "pointer span overflows");
        if (bytes > capacity) return hc_status(err, QW4_CAPACITY, "view exceeds capacity");
        *span = bytes;
    }
    if (rank != want_rank) return hc_status(err, QW4_SHAPE, "unexpected rank");
    for (size_t axis = 0; axis < rank; axis++)
        if (dim[axis] != want_dim[axis]) return hc_status(err, QW4_SHAPE, "unexpected shape");
    return QW4_OK;
}
#define ADMIT(v, rank_, dims_, span_) \
    pf_hc_admit_view((v).data, (v).capacity_bytes, (v).rank, (v).dim, (v).stride_bytes, rank_, dims_, span_, err)

Qwen4Status pf_hc_disjoint(const void *a, size_t na, const void *b, size_t nb, Qwen4Error *err) {
    if (na && nb && (uintptr_t)a < (uintptr_t)b + nb && (uintptr_t)b < (uintptr_t)a + na)
        return hc_status(err, QW4_INVALID_ARGUMENT, "forbidden view alias");
    return QW4_OK;
}

/* src/qwen4_base.c:71-75, :127-133 */
Qwen4Status pf_hc_admit_shape(const Qwen4HcShape *s, Qwen4Error *err) {
    if (!s) return hc_status(err, QW4_INVALID_ARGUMENT, "null HC shape");
    if (!s->streams || !s->hidden_size || !s->low_rank) return hc_status(err, QW4_SHAPE, "zero HC dimension");
    if (s->streams > UINT32_MAX || s->hidden_size > UINT32_MAX || s->low_rank > UINT32_MAX)
        return hc_status(err, QW4_RANGE, "HC dimension exceeds uint32");
    if (!isfinite(s->rms_eps)) return hc_status(err, QW4_NONFINITE, "nonfinite normalization epsilon");
    if (s->rms_eps <= 0) return hc_status(err, QW4_RANGE, "normalization epsilon must be positive");
    return QW4_OK;
}

/* the read's preflight up to the alias checks against its output (src/qwen4_base.c:144-146) */
Qwen4Status pf_hc_admit_read_inputs(const Qwen4HcShape *s, Qwen4F32 normed, Qwen4F32 logits, size_t span[2],
                                    Qwen4Error *err) {
    const size_t cube[3] = {normed.dim[0], s->streams, s->hidden_size};
    TRY(ADMIT(normed, 3, cube, &span[0]));
    TRY(ADMIT(logits, 3, normed.dim, &span[1]));
    return QW4_OK;
}

/* the add's preflight (src/qwen4_base.c:162-166) */
Qwen4Status pf_hc_admit_add(const Qwen4HcShape *s, Qwen4F32Mut residual, const float *block_data,
                            size_t block_span, Qwen4F32 inject, size_t *residual_span, Qwen4Error *err) {
    const size_t tokens = residual.dim[0];
    const size_t cube[3] = {tokens, s->streams, s->hidden_size}, gates[2] = {tokens, s->streams};
    size_t ispan;
    TRY(ADMIT(residual, 3, cube, residual_span));
    TRY(ADMIT(inject, 2, gates, &ispan));
    TRY(pf_hc_disjoint(residual.data, *residual_span, block_data, block_span, err));
    TRY(pf_hc_disjoint(residual.data, *residual_span, inject.data, ispan, err));
    return QW4_OK;
}

static Qwen4Status finish(int rc, uint32_t word, const char *overflow, Qwen4Error *err) {
    if (rc) return pf_device_status(rc, err, "qwen4/C");
    if (word & PF_HIP_ERR_NONFINITE) return hc_status(err, QW4_NONFINITE, overflow);
    if (word) return hc_status(err, QW4_GPU_ERROR, "device error word");
    return hc_status(err, QW4_OK, NULL);
}

Qwen4Status qwen4_hc_read(const Qwen4HcShape *s, Qwen4F32 normed, Qwen4F32 logits, Qwen4F32Mut mixed,
                          Qwen4Error *err) {
    TRY(pf_hc_admit_shape(s, err));
    const size_t tokens = normed.dim[0], rows[2] = {tokens, s->hidden_size};
    size_t span[2], out_span;
    TRY(pf_hc_admit_read_inputs(s, normed, logits, span, err));
    TRY(ADMIT(mixed, 2, rows, &out_span));
    TRY(pf_hc_disjoint(mixed.data, out_span, normed.data, span[0], err));
    TRY(pf_hc_disjoint(mixed.data, out_span, logits.data, span[1], err));
    if (!tokens) return hc_status(err, QW4_OK, NULL);
    uint32_t word = 0;
    const int rc = pf_hip_hc_read_host(normed.data, normed.stride_bytes[0], normed.stride_bytes[1], logits.data,
                                       logits.stride_bytes[0], logits.stride_bytes[1], mixed.data,
                                       mixed.stride_bytes[0], tokens, s->streams, s->hidden_size, &word);
    return finish(rc, word, "nonfinite input or HC read overflow", err);
}

Qwen4Status qwen4_hc_add(const Qwen4HcShape *s, Qwen4F32Mut residual, Qwen4F32 block, Qwen4F32 inject,
                         Qwen4Error *err) {
    TRY(pf_hc_admit_shape(s, err));
    const size_t tokens = residual.dim[0], rows[2] = {tokens, s->hidden_size};
    const size_t cube[3] = {tokens, s->streams, s->hidden_size};
    size_t rspan, bspan;
    /* the reference admits residual, block, inject in this order before any alias check */
    TRY(ADMIT(residual, 3, cube, &rspan));
    TRY(ADMIT(block, 2, rows, &bspan));
    TRY(pf_hc_admit_add(s, residual, block.data, bspan, inject, &rspan, err));
    if (!tokens) return hc_status(err, QW4_OK, NULL);
    uint32_t word = 0;
    const int rc = pf_hip_hc_add_host(residual.data, residual.stride_bytes[0], residual.stride_bytes[1], block.data,
                                      block.stride_bytes[0], inject.data, inject.stride_bytes[0], tokens, s->streams,
                                      s->hidden_size, &word);
    return finish(rc, word, "nonfinite input or HC residual overflow", err);
}
