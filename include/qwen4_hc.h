/* The two hyper-connection steps either side of the MoE block in the forward
 * loop (src/qwen4_forward.c:362-367): the gated read that produces the block's
 * input from the residual streams, and the injection that adds the block's
 * output back into every stream.
 *
 *   mixed[t, j]       = (sum_h normed[t, h, j] * sigmoid(gate_logits[t, h, j])) / streams
 *   residual[t, h, j] += inject[t, h] * block_out[t, j]
 *
 * Same names, argument meaning, validation order and status codes as the
 * reference's CPU operators; views are HOST memory, the arithmetic runs on the
 * GPU.  pf_moe_forward_hc chains read -> MoE -> add on the device so that the
 * [tokens, hidden] input and output of the block never leave HBM. */
#ifndef PF_QWEN4_HC_H
#define PF_QWEN4_HC_H
#include "qwen4_moe.h"

#ifdef __cplusplus
extern "C" {
#endif

/* src/qwen4_ops.h:43-44, src/qwen4_base.c:142-160.  normed and gate_logits are
 * [tokens, streams, hidden]; mixed is [tokens, hidden] and must not overlap them.
 * Streams are summed in ascending order, each product rounded before it is added.
 * QW4_NONFINITE for a nonfinite input or sum. */
Qwen4Status qwen4_hc_read(const Qwen4HcShape *, Qwen4F32 normed, Qwen4F32 gate_logits, Qwen4F32Mut mixed,
                          Qwen4Error *);

/* src/qwen4_ops.h:47-48, src/qwen4_base.c:161-175.  residual is [tokens, streams,
 * hidden] (token and stream axes may be pitched), block_out [tokens, hidden],
 * inject [tokens, streams]; neither input may overlap residual.  Bit-identical to
 * the reference: one product and one sum, each rounded. */
Qwen4Status qwen4_hc_add(const Qwen4HcShape *, Qwen4F32Mut residual, Qwen4F32 block_out, Qwen4F32 inject,
                         Qwen4Error *);

/* No counterpart as one call in the reference's CPU path; its GPU path fuses the
 * injection into the down projection the same way (src/qwen4_moe_internal.h:55-58).
 * Equivalent to qwen4_hc_read into a [tokens, hidden] buffer, qwen4_moe_forward on
 * it, qwen4_hc_add of the result: same validation (the read's, then the forward's,
 * then the add's), same routes, residual within the forward's tolerance.  The
 * workspace must have been created for at least `tokens` tokens. */
Qwen4Status pf_moe_forward_hc(const Qwen4Moe *, const Qwen4HcShape *, Qwen4F32 normed, Qwen4F32 gate_logits,
                              Qwen4F32Mut residual, Qwen4F32 inject, Qwen4MoeRoutes *optional_routes,
                              Qwen4MoeWork *, Qwen4Error *);

#ifdef __cplusplus
}
#endif
#endif
