/* C-ABI shim between the C11 host side (qwen4_moe.h entry points) and the HIP
 * kernels for gfx950.  Plain pointers and sizes only; no HIP or C++ types.
 *
 * These entry points take the place of the reference's device-side MoE step,
 * qw4f_routed_encode and its scratch description QW4FRoutedWork
 * (src/qwen4_moe_internal.h:36-78, src/qwen4_moe.m:271-402): router product,
 * softmax/top-k, indexed expert products and the weighted reduction all run on
 * the device and expert ids are not read back unless the caller asks for them.
 *
 * Every function returns PF_HIP_OK (0) or one of the codes below.  Pointers
 * named d_* are device pointers, everything else is host memory.  `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  A workspace serves
 * one forward at a time; different workspaces of one layer are independent. */
#ifndef PF_MOE_HIP_H
#define PF_MOE_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    PF_HIP_OK = 0,
    PF_HIP_E_ARGUMENT = 1,     /* null pointer, bad size */
    PF_HIP_E_UNSUPPORTED = 2,  /* format or dimension outside the kernels' range */
    PF_HIP_E_MEMORY = 3,       /* device or host allocation failed */
    PF_HIP_E_RUNTIME = 4,      /* a HIP call or launch failed; see pf_hip_last_error */
    PF_HIP_E_NO_DEVICE = 5
};

/* Bits of the error word the kernels maintain (the reference's convention,
 * src/qwen4_gpu.h:27-31: bit 1 nonfinite, bit 2 bounds). */
#define PF_HIP_ERR_NONFINITE 2u
#define PF_HIP_ERR_BOUNDS 4u
#define PF_HIP_ERR_TIMEOUT 8u   /* a workgroup gave up waiting for another of its launch (build-defined bit) */

typedef struct PfHipMoe PfHipMoe;    /* one layer's eight tensors, resident in HBM */
typedef struct PfHipWork PfHipWork;  /* device scratch for up to token_cap tokens */

/* Dimensions of Qwen4MoeConfig (src/qwen4_types.h:75-80) plus the GGUF type of
 * each tensor in Qwen4MoeWeights order: router, gate, up, down, shared gate,
 * shared up, shared down, shared router (src/qwen4_moe.h:7-10). */
typedef struct {
    uint32_t hidden, experts, top_k, inter, shared_inter, down_physical;
    uint32_t norm_topk;
    uint32_t type[8];
} PfHipMoeDesc;

int pf_hip_device_count(void);
const char *pf_hip_last_error(void);

/* Uploads the eight tensors (GGUF byte layout, bytes[i] each) into HBM.  The
 * host bytes are not referenced after the call returns. */
int pf_hip_moe_create(const PfHipMoeDesc *desc, const void *const host_weights[8],
                      const size_t bytes[8], PfHipMoe **out);
void pf_hip_moe_destroy(PfHipMoe *moe);
/* Total HBM bytes held by the layer. */
size_t pf_hip_moe_bytes(const PfHipMoe *moe);

size_t pf_hip_work_bytes(const PfHipMoeDesc *desc, size_t token_cap);
int pf_hip_work_create(const PfHipMoe *moe, size_t token_cap, PfHipWork **out);
void pf_hip_work_destroy(PfHipWork *work);

/* Enqueues one forward on `stream`: d_x [tokens, hidden] -> d_y [tokens, hidden],
 * row pitches in floats.  Asynchronous; results, routes (in the workspace) and
 * the error word are valid after the stream has been synchronised. */
int pf_hip_moe_forward_device(const PfHipMoe *moe, PfHipWork *work, const float *d_x,
                              size_t x_pitch, float *d_y, size_t y_pitch, size_t tokens,
                              void *stream);
/* No counterpart in the reference.  The same forward for callers that cannot allocate or hold a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Its scratch is a static device array of the library (1 MiB per GPU, held until the process
 * ends), so the call allocates and frees nothing; at most 4 tokens, and PF_HIP_E_UNSUPPORTED
 * (with pf_hip_last_error saying how much was needed) when the layer's scratch for `tokens`
 * tokens exceeds the array.  Outputs are the caller's: d_y [tokens, hidden] (pitch in floats),
 * optionally d_ids and d_route_weights (dense [tokens, top_k], NULL = not wanted), and
 * d_error_word, one device uint32 the kernels OR PF_HIP_ERR_* bits into (the caller clears
 * it).  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU race. */
int pf_hip_moe_forward_static(const PfHipMoe *moe, const float *d_x, size_t x_pitch, float *d_y,
                              size_t y_pitch, uint32_t *d_ids, float *d_route_weights,
                              uint32_t *d_error_word, size_t tokens, void *stream);
/* Which kernels a forward of `tokens` tokens runs on this layer and workspace: 1 the
 * decode kernels (1..4 tokens, 1..16 with the tile-ordered copies; supported shapes and formats),
 * 2 the matrix-core prefill kernels, 0 the general kernels (any shape and format mix).  A streamed
 * layer: 1 for the batches its decode kernels take when the pool keeps Q4_K slots in the tile order. */
int pf_hip_moe_kernel_family(const PfHipMoe *moe, const PfHipWork *work, size_t tokens);
/* Dependent launches of such a forward on the decode kernels: 3 (router logits; routing, gate/up and
 * SwiGLU; down products and combine), or 2 where one launch takes the whole expert stage (one token,
 * Q4_K or IQ2_XXS throughout, a workspace created with PF_MOE_DECODE_FUSED=1 in the environment, a
 * device with a compute unit per workgroup: an option, slower than the three kernels where it was
 * measured), or 4 where the routing runs in a launch of its own between the router logits and a
 * gate/up kernel that is given the experts (three tokens or more on the tile-ordered kernels).
 * 0: the forward runs other kernels. */
int pf_hip_moe_decode_launches(const PfHipMoe *moe, const PfHipWork *work, size_t tokens);
/* Device pointers into the workspace, valid after a forward: expert ids
 * [tokens, top_k] uint32, route weights [tokens, top_k], router logits
 * [tokens, experts], the error word (one uint32). */
const uint32_t *pf_hip_work_ids(const PfHipWork *work);
const float *pf_hip_work_route_weights(const PfHipWork *work);
const float *pf_hip_work_logits(const PfHipWork *work);
const uint32_t *pf_hip_work_error_word(const PfHipWork *work);
/* Number of tokens of the last forward whose routing was re-evaluated in the
 * reference's serial order because two candidate logits were too close. */
int pf_hip_work_exact_rows(PfHipWork *work, uint32_t *count);
/* Of those, the tokens that summing only the doubtful experts again did not settle (two of their
 * probabilities within a few ulps without being equal, more than 64 doubtful experts, probabilities near the
 * subnormals): all their logits were summed serially.  Kernels that re-route every flagged token that way
 * (more than 1024 experts, the segment decode kernels) do not count here. */
int pf_hip_work_full_reroutes(PfHipWork *work, uint32_t *count);

/* The error word and the re-route counter accumulate over forwards (a forward only
 * enqueues kernels, so it can be captured into a graph); this clears both. */
int pf_hip_work_clear_status(PfHipWork *work);
/* Host-buffer forward used by qwen4_moe_forward: copies x in, runs the forward,
 * copies y (and ids/weights when non-NULL) out, returns the error word.  Pitches
 * in bytes.  Outputs are written only when the error word is zero.  Batches of up
 * to 16 tokens go through a pinned host block the workspace owns (one enqueued copy
 * in, output rows written into the block by the kernels, one enqueued copy for the
 * error word, ids and weights, one wait); longer ones use a blocking copy per buffer. */
int pf_hip_moe_forward_host(const PfHipMoe *moe, PfHipWork *work, const float *x,
                            size_t x_pitch_bytes, float *y, size_t y_pitch_bytes,
                            uint32_t *ids, size_t ids_pitch_bytes, float *weights,
                            size_t weights_pitch_bytes, size_t tokens, uint32_t *error_word);

/* The hyper-connection steps either side of the block (src/qwen4_base.c:142-175).
 * Device forms: enqueue only, pitches in FLOATS (token pitch, then stream pitch of
 * the [tokens, streams, hidden] cubes; row pitch of matrices); d_error_word is a
 * device uint32 that receives PF_HIP_ERR_NONFINITE for a nonfinite input or result.
 *   read: d_mixed[t, j] = (sum_h d_normed[t, h, j] * sigmoid(d_logits[t, h, j])) / streams
 *   add:  d_residual[t, h, j] += d_inject[t, h] * d_block[t, j]   (bit-identical to the reference) */
int pf_hip_hc_read_device(const float *d_normed, size_t n_token_pitch, size_t n_stream_pitch,
                          const float *d_logits, size_t g_token_pitch, size_t g_stream_pitch,
                          float *d_mixed, size_t m_pitch, size_t tokens, size_t streams,
                          size_t hidden, uint32_t *d_error_word, void *stream);
int pf_hip_hc_add_device(float *d_residual, size_t r_token_pitch, size_t r_stream_pitch,
                         const float *d_block, size_t b_pitch, const float *d_inject,
                         size_t i_pitch, size_t tokens, size_t streams, size_t hidden,
                         uint32_t *d_error_word, void *stream);
/* read -> forward -> add as one enqueue: the read fills the workspace's input rows and
 * the forward's last kernel adds weight * output into every residual stream instead of
 * writing an output matrix (the reference's device path fuses the add the same way,
 * src/qwen4_moe_internal.h:55-58).  d_inject is dense [tokens, streams].  Allocates
 * nothing, synchronises nothing; errors accumulate in the workspace's error word. */
int pf_hip_moe_forward_hc_device(const PfHipMoe *moe, PfHipWork *work, const float *d_normed,
                                 size_t n_token_pitch, size_t n_stream_pitch,
                                 const float *d_logits, size_t g_token_pitch,
                                 size_t g_stream_pitch, float *d_residual, size_t r_token_pitch,
                                 size_t r_stream_pitch, const float *d_inject, size_t streams,
                                 size_t tokens, void *stream);
/* Host-buffer forms used by qwen4_hc_read, qwen4_hc_add and pf_moe_forward_hc: copy
 * in, run, copy out; pitches in BYTES; outputs written only when the returned error
 * word is zero. */
int pf_hip_hc_read_host(const float *normed, size_t n_token_pitch_bytes,
                        size_t n_stream_pitch_bytes, const float *logits,
                        size_t g_token_pitch_bytes, size_t g_stream_pitch_bytes, float *mixed,
                        size_t m_pitch_bytes, size_t tokens, size_t streams, size_t hidden,
                        uint32_t *error_word);
int pf_hip_hc_add_host(float *residual, size_t r_token_pitch_bytes, size_t r_stream_pitch_bytes,
                       const float *block, size_t b_pitch_bytes, const float *inject,
                       size_t i_pitch_bytes, size_t tokens, size_t streams, size_t hidden,
                       uint32_t *error_word);
int pf_hip_moe_forward_hc_host(const PfHipMoe *moe, PfHipWork *work, const float *normed,
                               size_t n_token_pitch_bytes, size_t n_stream_pitch_bytes,
                               const float *logits, size_t g_token_pitch_bytes,
                               size_t g_stream_pitch_bytes, float *residual,
                               size_t r_token_pitch_bytes, size_t r_stream_pitch_bytes,
                               const float *inject, size_t i_pitch_bytes, size_t streams,
                               size_t tokens, uint32_t *ids, size_t ids_pitch_bytes,
                               float *weights, size_t weights_pitch_bytes, uint32_t *error_word);

/* qwen4_moe_route on the device (src/qwen4_moe.c:188-249), reference evaluation
 * order.  Dense host arrays: logits/probs [tokens, experts], ids/weights
 * [tokens, top_k].  *bad_row receives the first row with a nonfinite logit when
 * the error word has PF_HIP_ERR_NONFINITE set; nothing is written then. */
int pf_hip_route_host(const float *logits, size_t tokens, size_t experts, size_t top_k,
                      int norm_topk, float *probs, uint32_t *ids, float *weights,
                      uint32_t *error_word, uint64_t *bad_row);

/* qw4_moe_group_pairs on the device (src/qwen4_moe.c:251-303): histogram,
 * exclusive scan, stable placement.  ids dense [tokens, top_k]; outputs
 * offsets [experts+1], pair_to_row/row_to_pair [tokens*top_k] as uint64.  Error
 * word: PF_HIP_ERR_BOUNDS for an id >= experts, PF_HIP_ERR_NONFINITE is unused;
 * *duplicate is set when a token repeats an id.  Outputs untouched on error. */
int pf_hip_group_pairs_host(const uint32_t *ids, size_t tokens, size_t experts, size_t top_k,
                            uint64_t *offsets, uint64_t *pair_to_row, uint64_t *row_to_pair,
                            uint32_t *error_word, int *duplicate);

/* qw4_packed_matmul / qw4_packed_decode_row on the device for one expert's
 * bytes (src/qwen4_packed.c:124-181), reference evaluation order, bit-identical.
 * x dense [rows, k_logical], y dense [rows, n_out]. */
int pf_hip_packed_matmul_host(uint32_t gguf_type, const void *expert_bytes, size_t row_bytes,
                              size_t n_out, size_t k_logical, const float *x, size_t rows,
                              float *y, uint32_t *error_word);
int pf_hip_packed_decode_row_host(uint32_t gguf_type, const void *row_bytes_ptr, size_t row_bytes,
                                  size_t k_storage, float *out, uint32_t *error_word);

/* The block's elementwise steps in the reference's evaluation order, bit-identical on hosts whose C
 * library computes expf as glibc 2.27+ does.  op 0: SiLU, op 1: sigmoid (qwen4_activate,
 * src/qwen4_base.c:76-99), op 2: out[j] = a[j] * b[j] (src/qwen4_moe.c:327-330).  A nonfinite input
 * or result sets PF_HIP_ERR_NONFINITE and leaves out untouched. */
int pf_hip_exact_elementwise_host(int op, const float *a, const float *b, size_t n, float *out,
                                  uint32_t *error_word);

/* src/qwen4_moe.c:350-368: routed[t, c] = the slot-order sum of weights[t, s] * down[pair_to_row[t*k+s], c],
 * y = routed + shared_gate[t] * shared[t, c].  Dense host arrays.  Both outputs are written even when
 * the error word is set. */
int pf_hip_exact_combine_host(const float *down, const uint64_t *pair_to_row, const float *weights,
                              const float *shared_gate, const float *shared, size_t tokens, size_t top_k,
                              size_t hidden, float *routed, float *y, uint32_t *error_word);

/* A layer created with its three routed tensors absent (host_weights[1..3] all NULL) keeps none of them
 * in device memory.  Its
 * forward is two calls with an expert pool in between, the shape of the reference's remap hook
 * (src/qwen4_moe_internal.h:49-54): the first runs the router and the routing and returns the pairs'
 * expert ids (dense [tokens, top_k]); the caller makes them resident and passes the pool's three device
 * regions, the payload bytes of one expert and the offset of the scales in each (pf_hip_pool_region_plan's
 * layout for the pool's slot count), the slot count and the pairs' slots to the second, which runs the
 * expert products and the combine.  pf_hip_moe_forward_* refuse such a layer.
 * tiled_mask, the same in both calls: bit j set when region j holds Q4_K or IQ2_XXS slots in the tile order
 * (what pf_hip_pool_store writes where pf_hip_pool_slot_tiled says so).  With every such region set -- all
 * three of a layer that is Q4_K or IQ2_XXS throughout, gate and up of one in a checkpoint profile (Q4_K with
 * an MXFP4 down tensor, IQ2_XXS with a Q2_K one; Q8_0 shared expert) -- batches of up to 16 tokens run the
 * decode kernels on the slots (the first call the router kernel and the routing, the second the expert
 * kernels); otherwise the general kernels, which read either order. */
int pf_hip_moe_route_streamed_host(const PfHipMoe *moe, PfHipWork *work, const float *x, size_t x_pitch_bytes,
                                   size_t tokens, uint32_t tiled_mask, uint32_t *ids, uint32_t *error_word);
int pf_hip_moe_experts_streamed_host(const PfHipMoe *moe, PfHipWork *work, const void *const regions[3],
                                     const size_t expert_bytes[3], const size_t scale_offsets[3],
                                     uint32_t pool_slots, uint32_t tiled_mask, const uint32_t *slots,
                                     float *y, size_t y_pitch_bytes, uint32_t *ids, size_t ids_pitch_bytes,
                                     float *weights, size_t weights_pitch_bytes, size_t tokens,
                                     uint32_t *error_word);

/* Pool regions in the device layout: a region of `slots` experts of one matrix is laid out as a resident
 * tensor of `slots` experts (formats stored as the file stores them slot after slot; IQ2_XXS, Q8_0 and
 * MXFP4 as all payloads, then all scales).  pf_hip_pool_region_plan gives the region's size, the bytes
 * of one expert in the file, the bytes of its payload in a slot and the offset of the scales (0: not split); pf_hip_pool_store copies one
 * expert's file bytes from host memory into a slot, splitting on the device where the format needs it
 * (a Q4_K or IQ2_XXS matrix whose row count is a multiple of 32 goes into the tile order:
 * pf_hip_pool_slot_tiled; an IQ2_XXS slot in that order holds its block scales inside its chunks, so the
 * scale offset is 0 and the payload bytes are those of the chunks), and returns when the slot is readable. */
int pf_hip_pool_region_plan(uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, size_t *region_bytes,
                            size_t *file_expert_bytes, size_t *payload_expert_bytes, size_t *scale_offset);
int pf_hip_pool_store(uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, void *region, size_t slot,
                      const void *file_bytes);
int pf_hip_pool_slot_tiled(uint32_t gguf_type, size_t n_out);
/* A reader's staging, allocated once: `bytes` of page-locked host memory to read the file into (pf_hip_stage_host),
 * as much device memory for the bytes on their way into a split or tile kernel, and a stream of the reader's own.
 * pf_hip_pool_store_staged stores the `file_bytes` the host memory holds like pf_hip_pool_store does (gguf_type
 * UINT32_MAX: as they are, at region + slot * file_bytes), enqueued on that stream and waited for: it allocates
 * nothing, and readers with stages of their own run side by side. */
typedef struct PfHipStage PfHipStage;
int pf_hip_stage_create(size_t bytes, PfHipStage **out);
void pf_hip_stage_destroy(PfHipStage *stage);
void *pf_hip_stage_host(PfHipStage *stage);
int pf_hip_pool_store_staged(PfHipStage *stage, uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots,
                             void *region, size_t slot, size_t file_bytes);

/* Minimal device-memory helpers so that a host program can keep inputs resident. */
int pf_hip_malloc(void **d_ptr, size_t bytes);
void pf_hip_free(void *d_ptr);
int pf_hip_memcpy_h2d(void *d_dst, const void *src, size_t bytes);
int pf_hip_memcpy_d2h(void *dst, const void *d_src, size_t bytes);
int pf_hip_synchronize(void);
#ifdef __cplusplus
}
#endif
#endif
