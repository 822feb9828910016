/* CPU oracle of the two hyper-connection steps either side of the MoE block:
 * TEST INFRASTRUCTURE ONLY (see orc.h).  Restates src/qwen4_base.c:127-175 and
 * the view helpers of src/qwen4_cpu_internal.h:38-122 in the reference's
 * evaluation order; compiled without contraction the results are bit-identical
 * to a build of the reference, which tests/test_oracle_hc.py checks. */
#include "orc.h"
#include <math.h>
#include <stdio.h>
#include <string.h>

static Qwen4Status hc_fail(Qwen4Error *err, Qwen4Status code, const char *detail) {
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
#define TRY(expr) do { Qwen4Status s_ = (expr); if (s_ != QW4_OK) return s_; } while (0)

static Qwen4F32 read_only(Qwen4F32Mut v) {
    Qwen4F32 r = {.data = v.data, .capacity_bytes = v.capacity_bytes, .rank = v.rank};
    memcpy(r.dim, v.dim, sizeof r.dim);
    memcpy(r.stride_bytes, v.stride_bytes, sizeof r.stride_bytes);
    return r;
}

/* src/qwen4_cpu_internal.h:38-62: innermost axis first; each stride a multiple of
 * four bytes and at least the span of the axes inside it */
static Qwen4Status check_view(Qwen4F32 v, Qwen4Error *err) {
    if (v.rank < 1 || v.rank > QWEN4_MAX_RANK) return hc_fail(err, QW4_SHAPE, "rank must be 1..4");
    size_t span = sizeof(float);
    for (size_t i = v.rank; i-- > 0;) {
        if (!v.dim[i] && i != 0) return hc_fail(err, QW4_SHAPE, "only the first axis may be empty");
        if (v.dim[i] > UINT32_MAX) return hc_fail(err, QW4_RANGE, "dimension exceeds uint32");
        size_t stride = v.stride_bytes[i];
        if (stride % sizeof(float) || stride < span || (i == v.rank - 1 && stride != sizeof(float)))
            return hc_fail(err, QW4_STRIDE, "noncontiguous feature or overlapping axes");
        if (v.dim[i]) {
            size_t steps = v.dim[i] - 1;
            if ((stride && steps > SIZE_MAX / stride) || span > SIZE_MAX - steps * stride)
                return hc_fail(err, QW4_OVERFLOW, "view span overflows");
            span += steps * stride;
        }
    }
    if (!v.dim[0]) return QW4_OK;
    if (!v.data) return hc_fail(err, QW4_INVALID_ARGUMENT, "null nonempty view");
    if ((uintptr_t)v.data % _Alignof(float)) return hc_fail(err, QW4_STRIDE, "unaligned float pointer");
    if (span > UINTPTR_MAX - (uintptr_t)v.data) return hc_fail(err, QW4_OVERFLOW, "pointer span overflows");
    if (span > v.capacity_bytes) return hc_fail(err, QW4_CAPACITY, "view exceeds capacity");
    return QW4_OK;
}

/* src/qwen4_cpu_internal.h:109-114 */
static Qwen4Status check_dims(Qwen4F32 v, size_t rank, const size_t *dims, Qwen4Error *err) {
    TRY(check_view(v, err));
    if (v.rank != rank) return hc_fail(err, QW4_SHAPE, "unexpected rank");
    for (size_t i = 0; i < rank; i++)
        if (v.dim[i] != dims[i]) return hc_fail(err, QW4_SHAPE, "unexpected shape");
    return QW4_OK;
}

static size_t element_count(Qwen4F32 v) {
    size_t n = 1;
    for (size_t i = 0; i < v.rank; i++) n *= v.dim[i];
    return n;
}
/* src/qwen4_cpu_internal.h:67-74: row-major element index -> float offset */
static float element(Qwen4F32 v, size_t index) {
    size_t offset = 0;
    for (size_t i = v.rank; i-- > 0;) {
        offset += (index % v.dim[i]) * (v.stride_bytes[i] / sizeof(float));
        index /= v.dim[i];
    }
    return v.data[offset];
}
static size_t byte_span(Qwen4F32 v) {
    if (!v.dim[0]) return 0;
    size_t n = sizeof(float);
    for (size_t i = 0; i < v.rank; i++) n += (v.dim[i] - 1) * v.stride_bytes[i];
    return n;
}
/* src/qwen4_cpu_internal.h:81-97 with exact == false: any overlap is refused */
static Qwen4Status check_disjoint(Qwen4F32 out, Qwen4F32 in, Qwen4Error *err) {
    size_t na = byte_span(out), nb = byte_span(in);
    uintptr_t a = (uintptr_t)out.data, b = (uintptr_t)in.data;
    if (na && nb && a < b + nb && b < a + na) return hc_fail(err, QW4_INVALID_ARGUMENT, "forbidden view alias");
    return QW4_OK;
}
static Qwen4Status check_finite(Qwen4F32 v, Qwen4Error *err) {
    size_t n = element_count(v);
    for (size_t i = 0; i < n; i++)
        if (!isfinite(element(v, i))) return hc_fail(err, QW4_NONFINITE, "nonfinite input");
    return QW4_OK;
}

/* src/qwen4_base.c:71-75, :127-133 */
static Qwen4Status check_shape(const Qwen4HcShape *s, Qwen4Error *err) {
    if (!s) return hc_fail(err, QW4_INVALID_ARGUMENT, "null HC shape");
    if (!s->streams || !s->hidden_size || !s->low_rank) return hc_fail(err, QW4_SHAPE, "zero HC dimension");
    if (s->streams > UINT32_MAX || s->hidden_size > UINT32_MAX || s->low_rank > UINT32_MAX)
        return hc_fail(err, QW4_RANGE, "HC dimension exceeds uint32");
    if (!isfinite(s->rms_eps)) return hc_fail(err, QW4_NONFINITE, "nonfinite normalization epsilon");
    if (s->rms_eps <= 0) return hc_fail(err, QW4_RANGE, "normalization epsilon must be positive");
    return QW4_OK;
}

/* src/qwen4_base.c:142-160: per (token, column) the streams in ascending order,
 * product rounded, then added; the mean is one division by (float)streams.  An
 * overflowing sum stops the call with the columns before it already written. */
Qwen4Status orc_hc_read(const Qwen4HcShape *s, Qwen4F32 normed, Qwen4F32 logits, Qwen4F32Mut out,
                        Qwen4Error *err) {
    TRY(check_shape(s, err));
    size_t tokens = normed.dim[0];
    Qwen4F32 y = read_only(out);
    TRY(check_dims(normed, 3, (size_t[]){tokens, s->streams, s->hidden_size}, err));
    TRY(check_dims(logits, 3, normed.dim, err));
    TRY(check_dims(y, 2, (size_t[]){tokens, s->hidden_size}, err));
    TRY(check_disjoint(y, normed, err));
    TRY(check_disjoint(y, logits, err));
    TRY(check_finite(normed, err));
    TRY(check_finite(logits, err));
    for (size_t t = 0; t < tokens; t++)
        for (size_t j = 0; j < s->hidden_size; j++) {
            float sum = 0;
            for (size_t h = 0; h < s->streams; h++) {
                size_t i = (t * s->streams + h) * s->hidden_size + j;
                sum += element(normed, i) * orc_sigmoid(element(logits, i));
            }
            if (!isfinite(sum)) return hc_fail(err, QW4_NONFINITE, "HC read overflow");
            out.data[t * (y.stride_bytes[0] / 4) + j] = sum / (float)s->streams;
        }
    return hc_fail(err, QW4_OK, NULL);
}

/* src/qwen4_base.c:161-175: in place, token-major then stream then column; a
 * nonfinite result stops the call with the elements before it already updated. */
Qwen4Status orc_hc_add(const Qwen4HcShape *s, Qwen4F32Mut residual, Qwen4F32 block, Qwen4F32 inject,
                       Qwen4Error *err) {
    TRY(check_shape(s, err));
    Qwen4F32 r = read_only(residual);
    size_t tokens = r.dim[0];
    TRY(check_dims(r, 3, (size_t[]){tokens, s->streams, s->hidden_size}, err));
    TRY(check_dims(block, 2, (size_t[]){tokens, s->hidden_size}, err));
    TRY(check_dims(inject, 2, (size_t[]){tokens, s->streams}, err));
    TRY(check_disjoint(r, block, err));
    TRY(check_disjoint(r, inject, err));
    TRY(check_finite(r, err));
    TRY(check_finite(block, err));
    TRY(check_finite(inject, err));
    for (size_t t = 0; t < tokens; t++)
        for (size_t h = 0; h < s->streams; h++)
            for (size_t j = 0; j < s->hidden_size; j++) {
                size_t ri = t * (r.stride_bytes[0] / 4) + h * (r.stride_bytes[1] / 4) + j;
                float result = residual.data[ri] +
                               element(inject, t * s->streams + h) * element(block, t * s->hidden_size + j);
                if (!isfinite(result)) return hc_fail(err, QW4_NONFINITE, "HC residual overflow");
                residual.data[ri] = result;
            }
    return hc_fail(err, QW4_OK, NULL);
}
