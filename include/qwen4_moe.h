/* MoE feed-forward block: the drop-in boundary.
 *
 * Same names, argument meaning, ownership and status codes as the reference's
 * src/qwen4_moe.h:13-27.  The reference has no plugin registry for this block
 * ("Direct B calls; no callback plugin ABI", src/qwen4_moe.h:12): a replacement
 * is linked in place of src/qwen4_moe.c and src/qwen4_packed.c.  The functions
 * below compute the routed + shared contribution and never add the residual.
 *
 * What differs from the CPU reference, by construction of a device path:
 *  - qwen4_moe_create uploads the eight weight tensors to device memory once.
 *    The host bytes are read during create only; later changes to them are not
 *    seen (the reference borrows them until destroy, src/qwen4_moe.h:12).
 *  - Workspaces hold device buffers for the whole token capacity, not for
 *    32-token microbatches, so qwen4_moe_work_size grows with token_cap.
 *  - Arithmetic runs in FP32 with a different summation order: expert ids equal
 *    the reference's whenever adjacent top-(k+1) router logits differ by more
 *    than the rounding noise of the logit sum; rows closer than that are
 *    re-evaluated in the reference's serial order before selection.  Outputs
 *    agree within 1e-3 absolute + 1e-4 relative.
 *  - Nonfinite values are detected from an error word written by the kernels
 *    (inputs, every intermediate vector and the outputs are checked), not after
 *    every scalar operation. */
#ifndef PF_QWEN4_MOE_H
#define PF_QWEN4_MOE_H
#include "qwen4_packed.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct Qwen4Moe Qwen4Moe;
typedef struct Qwen4MoeWork Qwen4MoeWork;

/* Order of src/qwen4_moe.h:7-10. */
typedef struct {
    QW4PackedCpuView router, gate, up, down;
    QW4PackedCpuView shared_gate, shared_up, shared_down, shared_router;
} Qwen4MoeWeights;

typedef struct {
    Qwen4U32Mut ids;      /* [T, top_k] expert ids, slot order = selection order */
    Qwen4F32Mut weights;  /* [T, top_k] (renormalised) probabilities */
} Qwen4MoeRoutes;

/* Replaces qwen4_moe_create / qwen4_moe_destroy (src/qwen4_moe.c:47-76).
 * Validates shapes ({h,h,h,i,h,h,s,h} in, {E,i,i,h,s,s,h,1} out), expert counts
 * and that both routers are F32, copies the config, uploads the weights. */
Qwen4Status qwen4_moe_create(const Qwen4MoeConfig *config, const Qwen4MoeWeights *weights,
                             Qwen4Moe **out, Qwen4Error *err);
void qwen4_moe_destroy(Qwen4Moe *moe);

/* Replace qwen4_moe_work_size/create/reset/destroy (src/qwen4_moe.c:80-129).
 * *bytes counts host metadata plus device scratch for token_cap tokens. */
Qwen4Status qwen4_moe_work_size(const Qwen4Moe *moe, size_t token_cap, size_t *bytes,
                                Qwen4Error *err);
Qwen4Status qwen4_moe_work_create(const Qwen4Moe *moe, size_t token_cap, size_t byte_budget,
                                  Qwen4MoeWork **out, Qwen4Error *err);
Qwen4Status qwen4_moe_work_reset(Qwen4MoeWork *work, Qwen4Error *err);
void qwen4_moe_work_destroy(Qwen4MoeWork *work);

/* Replaces qwen4_moe_route (src/qwen4_moe.c:188-249): softmax over caller-owned
 * logits, k rounds of arg-max with ties to the lower id, optional
 * renormalisation.  All four views are pitched and pairwise disjoint; a
 * nonfinite logit gives QW4_NONFINITE with err->row set and nothing written.
 * The kernel keeps the reference's evaluation order (serial exponent sum). */
Qwen4Status qwen4_moe_route(const Qwen4MoeConfig *config, Qwen4F32 logits,
                            Qwen4MoeRoutes routes, Qwen4F32Mut probabilities,
                            Qwen4Error *err);

/* Replaces qwen4_moe_forward (src/qwen4_moe.c:384-431): x [T,H] -> y [T,H],
 * optionally the routes.  Preflight errors leave every output untouched; a
 * failure during execution marks the workspace failed until reset. */
Qwen4Status qwen4_moe_forward(const Qwen4Moe *moe, Qwen4F32 x, Qwen4F32Mut y,
                              Qwen4MoeRoutes *optional_routes, Qwen4MoeWork *work,
                              Qwen4Error *err);

/* Private-but-tested helpers of the reference (src/qwen4_moe_internal.h:9-15,78-95). */
typedef struct {
    size_t *offsets;                 /* [experts+1] */
    size_t offsets_capacity_bytes;
    size_t *cursors;                 /* [experts] scratch; ends at offsets[e+1] */
    size_t cursors_capacity_bytes;
    size_t *pair_to_row, *row_to_pair; /* [T*K], inverse permutations */
    size_t pair_to_row_capacity_bytes, row_to_pair_capacity_bytes;
} QW4MoeGrouping;

/* Replaces qw4_moe_group_pairs (src/qwen4_moe.c:251-303): stable counting sort
 * of (token, slot) pairs by expert id, run as histogram + scan + placement
 * kernels.  Error preflight leaves all arrays unchanged. */
Qwen4Status qw4_moe_group_pairs(const Qwen4MoeConfig *config, Qwen4U32Mut ids,
                                QW4MoeGrouping grouping, Qwen4Error *err);

/* Replaces qw4_moe_observe (src/qwen4_moe.c:130-132).  Stage numbers follow
 * src/qwen4_moe_internal.h:9-12: 0..7 projections in weight order, 8 SiLU,
 * 9 product, 10 sigmoid, 11 routed, 12 y; the (stage, expert, token, input, output) sequence is the
 * reference's (src/qwen4_moe.c:305-382), per microbatch of at most 32 tokens.  While an observer is
 * set, forward runs the block as that sequence of operators, one device call each in the reference's
 * evaluation order (slow; outputs bit-identical to the reference's), and reads the weights from the
 * caller's host views: QW4_BAD_STATE after pf_moe_forget_host_weights.  Views passed to the observer
 * are host staging memory, valid during the callback. */
typedef void (*QW4MoeObserver)(void *ctx, size_t stage, size_t expert, size_t token,
                               Qwen4F32 input, Qwen4F32 output);
void qw4_moe_observe(Qwen4MoeWork *work, QW4MoeObserver observer, void *ctx);

/* Extension without a counterpart in the reference: the device-side handles behind a
 * layer and a workspace (include/pf_moe_hip.h), for callers that keep activations
 * resident in HBM and enqueue forwards on their own stream.  Owned by the handles
 * they come from. */
struct PfHipMoe *pf_moe_device_layer(const Qwen4Moe *moe);
/* Extension: qwen4_moe_create copies the weight bytes to device memory, but like the reference
 * (src/qwen4_moe.h:12, src/qwen4_moe.c:403-410) qwen4_moe_forward refuses views that overlap the
 * host bytes the layer was created from, so those must stay allocated until destroy.  A caller
 * that releases them earlier calls this first; forward then skips that comparison for the layer
 * (pf_gguf_moe_create does so itself: its layers may outlive the file mapping). */
void pf_moe_forget_host_weights(Qwen4Moe *moe);

/* Extension for models larger than device memory, the counterpart of the reference's expert streaming
 * (src/qwen4_expert_pool.h; the remap hook of src/qwen4_moe_internal.h:49-54; its caller in
 * src/qwen4_forward_gpu.m).  pf_moe_create_streamed takes the same arguments as qwen4_moe_create with
 * the gate, up and down views carrying their layouts and a NULL span: those tensors stay in the model
 * file (where they are IQ2_XXS, Q8_0 or MXFP4 the pool must know its formats: pf_pool_set_formats, else
 * QW4_SHAPE from the forward).  pf_moe_forward_streamed is
 * qwen4_moe_forward for such a layer: after the routing it acquires the batch's experts from `pool` as
 * layer `layer` (tokens * top_k pins: the pool needs that many slots), runs the expert products on the
 * pool's slots and releases them.  QW4_IO when the pool cannot take the batch or a read fails;
 * qwen4_moe_forward on a streamed layer, or a pool with a resident one: QW4_BAD_STATE. */
struct QW4ExpertPool;
Qwen4Status pf_moe_create_streamed(const Qwen4MoeConfig *config, const Qwen4MoeWeights *weights, Qwen4Moe **out,
                                   Qwen4Error *err);
Qwen4Status pf_moe_forward_streamed(const Qwen4Moe *moe, struct QW4ExpertPool *pool, uint32_t layer, Qwen4F32 x,
                                    Qwen4F32Mut y, Qwen4MoeRoutes *optional_routes, Qwen4MoeWork *work, Qwen4Error *err);
struct PfHipWork *pf_moe_device_work(Qwen4MoeWork *work);

#ifdef __cplusplus
}
#endif
#endif
