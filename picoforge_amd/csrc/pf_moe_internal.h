// Internal declarations shared by the HIP translation units of the MoE library.
#pragma once
#include "pf_device.h"
#include "../../include/pf_moe_hip.h"

#define PF_DECODE_MAX_TOKENS 4
#define PF_TILE_DECODE_MAX_TOKENS 16   // Q4_K layers whose tile-ordered copies are kept: one token per grid row

// Everything a kernel needs, passed by value.  Weight index order is
// Qwen4MoeWeights': router, gate, up, down, shared gate/up/down, shared router.
struct PfKernelArgs {
    int hidden, experts, top_k, inter, shared_inter, down_physical, norm_topk;
    uint32_t type[8];
    const uint8_t *w[8];
    size_t row_bytes[8], expert_bytes[8];   // of the payload (IQ2_XXS: 64 bytes per block)
    size_t scale_offset[8];                 // IQ2_XXS: byte offset of the half scales in the tensor buffer
    int k_logical[8], blocks_per_row[8], n_out[8];
    const uint8_t *wt[8];            // Q4_K expert tensors in tile order for the grouped product (null: not kept)
    const uint8_t *wi[8];            // IQ2_XXS expert tensors in tile order for the decode kernels (null: not kept)
    const uint8_t *wq[8];            // Q8_0 tensors (the profiles' shared gate and up) in tile order (null: not kept)
    const float *router_t;           // router as [slab of 64 experts][hidden / 4][64][4] (serial-order re-routing)
    const uint64_t *iq2_grid;        // 256 x 8 magnitudes, device memory
    const uint32_t *iq2_signed;      // 2 x 4096 words: four signed magnitudes per (grid entry, sign nibble)
    const float *x;                  // [tokens, hidden], pitch in floats
    size_t x_pitch;
    float *y;
    size_t y_pitch;
    float *logits, *logit_ssq;       // [tokens, experts]
    uint32_t *ids;                   // [tokens, top_k]
    float *route_weights;            // [tokens, top_k]
    float *act;                      // general path [tokens * top_k, inter]; decode path [unique, tokens, inter]
    float *shared_act;               // [tokens, shared_inter]
    float *shared_scale;             // [tokens] sigmoid of the shared router logit
    uint32_t *ximg, *aimg;           // decode path, tile-ordered Q4_K: digit images (pf_image2_words) of the token rows, written
                                     // by kernel 1, and of the activation rows [unique, tokens] then [tokens] shared, by kernel 2
    uint32_t *uniq;                  // decode path: [0] count, then ids[P], then pair->unique[P], then token masks[P]
    // decode path, one token, the expert stage in one launch (null: three kernels): the workgroups' activation lines
    // (FUSE_REPLICAS copies) and the counter whose value tags a forward's lines, incremented by the router kernel
    uint32_t *fuse_lines, *fuse_gen;
    // expert streaming: w[1..3] (wt[1..3] for Q4_K slots in tile order) are pool regions of pool_slots experts each and the routed
    // tensors are addressed by slots[pair] instead of ids[pair] (null: every expert resident, addressed by id)
    const uint32_t *slots;
    uint32_t pool_slots;
    uint32_t *error_word;
    uint32_t *exact_rows;            // count of tokens re-routed in serial order
    uint32_t *route_flags;           // tokens to route again in serial order: [0] their number, then the tokens; the kernel
                                     // before the routing clears [0]
    // prefill path
    uint32_t token_cap;              // rows the workspace holds; row token_cap (token_cap * top_k for act16) of an fp16 form is all zero
    uint16_t *x16, *act16, *sact16;  // fp16 forms of x, act (pairs in expert order), shared act: per row the high
                                     // parts, the low parts, then 8 + 8 group-sum parts per 256 columns
    float *x_scale, *act_scale, *sact_scale;   // per row: the power of two the fp16 form was divided by
    float *x_max2;                   // [tokens] largest squared magnitude of the row
    const float *w_norm2;            // [experts] squared norm of each router row
    float *down;                     // [pairs + tokens, hidden] down products in expert order, then the shared expert's
    uint32_t *counts, *offsets, *pair_to_row, *row_to_pair, *group_bad, *tiles;
    // injection into hyper-connection streams in place of writing y (null: y is written)
    float *hc_residual;              // [tokens, streams, hidden], pitches in floats
    const float *hc_inject;          // [tokens, streams], dense
    size_t hc_token_pitch, hc_stream_pitch;
    int hc_streams;
};

// One finished element of the block's output.  Normally y[t, n]; when the forward injects into the
// residual streams (at most PF_HC_FOLD_MAX of them), residual[t, h, n] += inject[t, h] * value for
// every stream h, product and sum each rounded (src/qwen4_base.c:168-173).  The residual values are
// requested early (pf_output_prefetch, before the kernel's long loop) and used at the end
// (pf_output_commit), so their latency hides behind the products.  commit returns false if
// anything written is not finite.
#define PF_HC_FOLD_MAX 4
struct PfOutputRegs { float r[PF_HC_FOLD_MAX]; };

__device__ __forceinline__ void pf_output_prefetch(const PfKernelArgs &a, int t, int n, PfOutputRegs &q) {
    if (!a.hc_residual) return;
    const float *r = a.hc_residual + (size_t)t * a.hc_token_pitch + n;
#pragma unroll
    for (int h = 0; h < PF_HC_FOLD_MAX; h++)
        if (h < a.hc_streams) q.r[h] = r[(size_t)h * a.hc_stream_pitch];
}

__device__ __forceinline__ bool pf_output_commit(const PfKernelArgs &a, int t, int n, float value,
                                                 const PfOutputRegs &q) {
#pragma clang fp contract(off)
    if (!a.hc_residual) {
        a.y[(size_t)t * a.y_pitch + n] = value;
        return pf_finite(value);
    }
    bool ok = true;
    float *r = a.hc_residual + (size_t)t * a.hc_token_pitch + n;
    const float *w = a.hc_inject + (size_t)t * a.hc_streams;
#pragma unroll
    for (int h = 0; h < PF_HC_FOLD_MAX; h++) {
        if (h < a.hc_streams) {
            const float product = w[h] * value;
            const float result = q.r[h] + product;
            r[(size_t)h * a.hc_stream_pitch] = result;
            ok &= pf_finite(result);
        }
    }
    return ok;
}

struct PfHipMoe {
    PfHipMoeDesc desc;
    uint8_t *w[8];
    size_t bytes[8], row_bytes[8], expert_bytes[8], scale_offset[8];
    int k_logical[8], blocks_per_row[8], n_out[8];
    uint64_t *iq2_grid;
    uint32_t *iq2_signed;
    size_t total_bytes;
    bool decode_ready;               // shapes and formats the specialised decode kernels cover
    bool prefill_ready;              // shapes and formats the matrix-core prefill kernels cover
    int stream_decode;               // a streamed layer whose short batches run the tile decode kernels on pool slots: 1 Q4_K
                                     // throughout, 4 the q4 checkpoint profile (0: the general kernels serve every batch)
    float *w_norm2;                  // [experts] squared norm of each router row
    float *router_t;                 // [slab of 64 experts][hidden / 4][64][4] copy of the router
    uint8_t *w_tiled[8];             // tile-ordered second copy of the expert tensors for the prefill path (or null)
    uint8_t *w_itile[8];             // tile-ordered second copy of IQ2_XXS expert tensors for the decode path (or null)
    uint8_t *w_qtile[8];             // tile-ordered second copy of the Q8_0 shared gate and up tensors (or null)
    bool streamed;                   // the routed tensors are not resident: forwards read them from an expert pool
};

// Digit image of a K-vector for wave-uniform (scalar) reads: per 32-group PF_IMG_GROUP dwords (the values' lowest
// base-256 digits as 32 signed bytes, then the next digits, then the highest), then K/32 group steps (float), then K/32
// sums of the integers.  Two digits (16 bits) held the benchmark's tolerance but not that of layers with eight times
// larger weights (1.6 times the bound on the smallest outputs of a row); three leave a margin of 2^8 more.
#define PF_IMG_PLANES 3                       // signed byte digits per value: 24 bits
#define PF_IMG_GROUP (8 * PF_IMG_PLANES)      // dwords of one 32-group's digits
__host__ __device__ constexpr size_t pf_image2_words(size_t K) { return (K / 32) * (PF_IMG_GROUP + 2); }

struct PfHipWork {
    const PfHipMoe *moe;
    size_t cap, bytes;
    uint32_t *ximg, *aimg;
    float *logits, *logit_ssq, *route_weights, *act, *shared_act, *shared_scale, *x, *y;
    uint32_t *ids, *uniq, *error_word, *exact_rows, *route_flags, *slots, *fuse_lines, *fuse_gen;
    uint16_t *x16, *act16, *sact16;  // prefill buffers (allocated when cap exceeds the decode path's batch)
    float *x_scale, *act_scale, *sact_scale, *x_max2, *down;
    uint32_t *counts, *offsets, *pair_to_row, *row_to_pair, *group_bad, *tiles;
    uint8_t *host;                  // pinned host block for the host-pointer forwards of short batches (null: not available)
    uint8_t *host_device;           // the same block as the kernels address it (they write the output rows straight into it)
    int stage_limit;                // profiling: launch only the first so many kernels of a forward; 0 = all
    int force_general;               // tests: run the general kernels even where the decode path applies
    size_t guard, guard_at[40];      // diagnostics (PF_WORK_GUARD=1): bytes of pattern behind each buffer, and where
};

// pf_moe_kernels.hip
void pf_launch_general(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit, int first_stage = 1);
size_t pf_general_lds_bytes(const PfKernelArgs &a);
// pf_moe_route.hip
void pf_launch_route(const PfKernelArgs &a, int tokens, hipStream_t stream);
size_t pf_router_slab_floats(int experts, int hidden);
void pf_launch_router_slabs(const float *d_src, int experts, int hidden, float *d_dst, hipStream_t stream);
int pf_route_exact_device(const float *d_logits, int tokens, int experts, int top_k, int norm,
                          float *d_probs, uint32_t *d_ids, float *d_weights, uint32_t *d_error,
                          unsigned long long *d_bad_row, hipStream_t stream);
// histogram, scan, row tiles and placement (an expert's rows in no particular order) in one launch; false (nothing
// launched) for more pairs or experts than it takes
bool pf_launch_group_fused(const uint32_t *d_ids, int pairs, int experts, int tokens, uint32_t *d_offsets, uint32_t *d_tiles,
                           uint32_t *d_pair_to_row, uint32_t *d_row_to_pair, hipStream_t stream);
void pf_launch_group_place(const uint32_t *d_ids, int pairs, int experts, const uint32_t *d_offsets,
                           uint32_t *d_pair_to_row, uint32_t *d_row_to_pair, hipStream_t stream);
int pf_group_pairs_device(const uint32_t *d_ids, int tokens, int experts, int top_k, uint32_t *d_counts,
                          uint32_t *d_offsets, uint32_t *d_pair_to_row, uint32_t *d_row_to_pair,
                          uint32_t *d_first_bad, hipStream_t stream);
// pf_moe_exact.hip
void pf_launch_exact_matmul(uint32_t type, const uint8_t *d_w, size_t row_bytes, int n_out, int k_logical,
                            const float *d_x, int rows, float *d_y, uint32_t *d_error, const uint64_t *grid,
                            hipStream_t stream);
void pf_launch_exact_decode(uint32_t type, const uint8_t *d_row, int k_storage, float *d_out, uint32_t *d_error,
                            const uint64_t *grid, hipStream_t stream);
void pf_launch_exact_elementwise(int op, const float *d_a, const float *d_b, float *d_out, size_t n, uint32_t *d_error,
                                 hipStream_t stream);
void pf_launch_exact_combine(const float *d_down, const uint64_t *d_pair_to_row, const float *d_weights, const float *d_sa,
                             const float *d_shared, float *d_routed, float *d_y, int tokens, int top_k, int hidden,
                             uint32_t *d_error, hipStream_t stream);
// pf_moe_decode.hip
bool pf_decode_supported(const PfHipMoeDesc &d);
// more experts (or slots) than the fast routing holds in a wave's registers: every token's logits are summed serially
// from the router's slab copy (pf_moe_route.hip)
bool pf_route_needs_slabs(int experts, int top_k);
int pf_decode_tile_layer(const PfHipMoeDesc &d, const uint8_t *const q4k_tiled[8], const uint8_t *const iq2_tiled[8],
                         const uint8_t *const q8_tiled[8]);
void pf_launch_iq2_tile(const uint8_t *d_payload, const uint16_t *d_scales, uint8_t *d_dst, size_t rows, int blocks_per_row,
                        hipStream_t stream);
void pf_launch_q8_tile(const uint8_t *d_payload, const uint16_t *d_scales, uint8_t *d_dst, size_t rows, int blocks_per_row,
                       hipStream_t stream);
void pf_launch_decode(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_dec_router(const PfKernelArgs &a, int tokens, int router_blocks, hipStream_t stream);
// bytes of the activation lines a workspace needs for the one-launch expert stage of a one-token forward (0: the
// layer's shape or formats are not taken)
void pf_decode_fused_scratch(const PfHipMoeDesc &d, size_t *line_bytes);
// launches per forward on the decode path: 2 for one token with the fused expert stage, 4 where the routing runs in a
// launch of its own (three tokens or more on the tile kernels), else 3
int pf_decode_launches(const PfKernelArgs &a, int tokens);
// kernels 2 and 3 of the tile decode path on pool slots, for a Q4_K layer or one in the q4 checkpoint profile (expert
// streaming: kernel 1 ran in an earlier call)
void pf_launch_decode_stream_experts(const PfKernelArgs &a, int tokens, hipStream_t stream);
void pf_launch_iq2_split(const uint8_t *d_gguf, uint8_t *d_payload, uint16_t *d_scales, size_t blocks,
                         hipStream_t stream);
void pf_launch_block_split(const uint8_t *d_gguf, uint8_t *d_payload, uint8_t *d_scales, size_t blocks,
                           int block_bytes, int header_bytes, hipStream_t stream);
// pf_moe_prefill.hip
bool pf_prefill_supported(const PfHipMoeDesc &d);
void pf_launch_prefill(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_q4k_tile(const uint8_t *d_src, uint8_t *d_dst, size_t rows, int blocks_per_row, hipStream_t stream);
void pf_launch_row_norm2(const float *d_w, int rows, int cols, float *d_out, hipStream_t stream);
size_t pf_prefill_half_row(int cols);   // halfs per row of the fp16 form of a matrix with `cols` columns
int pf_prefill_max_tiles(int tokens, int experts, int top_k);
// pf_moe_hc.hip
void pf_launch_hc_read(const float *d_normed, size_t n_token_pitch, size_t n_stream_pitch, const float *d_logits,
                       size_t g_token_pitch, size_t g_stream_pitch, float *d_mixed, size_t m_pitch, int tokens,
                       int streams, int hidden, uint32_t *d_error, hipStream_t stream);
void pf_launch_hc_add(float *d_residual, size_t r_token_pitch, size_t r_stream_pitch, const float *d_block,
                      size_t b_pitch, const float *d_inject, size_t i_pitch, int tokens, int streams, int hidden,
                      uint32_t *d_error, hipStream_t stream);
// pf_moe_api.hip
const uint64_t *pf_device_iq2_grid(void);
const uint32_t *pf_device_iq2_signed(void);
void pf_set_error(const char *what, hipError_t code);
