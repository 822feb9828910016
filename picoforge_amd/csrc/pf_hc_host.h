/* Preflight checks of the hyper-connection operators, shared by qwen4_hc_host.c and the chained
 * forward in qwen4_moe_host.c.  Each follows src/qwen4_cpu_internal.h:38-122 in order and codes. */
#ifndef PF_HC_HOST_H
#define PF_HC_HOST_H
#include "../../include/qwen4_hc.h"

Qwen4Status pf_hc_admit_shape(const Qwen4HcShape *s, Qwen4Error *err);
Qwen4Status pf_hc_admit_view(const float *data, size_t capacity, size_t rank, const size_t dim[4],
                             const size_t stride[4], size_t want_rank, const size_t *want_dim, size_t *span,
                             Qwen4Error *err);
Qwen4Status pf_hc_disjoint(const void *a, size_t na, const void *b, size_t nb, Qwen4Error *err);
Qwen4Status pf_hc_admit_read_inputs(const Qwen4HcShape *s, Qwen4F32 normed, Qwen4F32 logits, size_t span[2],
                                    Qwen4Error *err);
Qwen4Status pf_hc_admit_add(const Qwen4HcShape *s, Qwen4F32Mut residual, const float *block_data,
                            size_t block_span, Qwen4F32 inject, size_t *residual_span, Qwen4Error *err);
#endif
