/* GGUF v3 checkpoints as the source of the MoE block's weights.
 *
 * What the reference spreads over its reader, config and weight catalog, narrowed to
 * the MoE feed-forward path: open and validate a GGUF v3 file (src/gguf.c:31-105,
 * src/gguf_reader.c), read the dimensions the block needs from the metadata
 * (src/qwen4_config.c:152-216 and the checks of :28-45), find and check the eight
 * tensors of one layer (src/qwen4_weights.c:19-56, rows :91-99) and hand them to
 * qwen4_moe_create as views (src/qwen4_forward.c:72-79, :174-187).
 *
 * The reference's reader terminates the process on a malformed file (die(),
 * src/util.c:13-21); every function here returns a status and fills the error
 * record instead, with the reference's message as the detail.  Tensors and metadata
 * of other blocks (attention, recurrent layers, embeddings, n-gram table) are parsed
 * as descriptors and otherwise ignored: a file the reference refuses because of them
 * can be accepted here.
 *
 * The file is mapped read-only for the life of the handle; views returned by
 * pf_gguf_moe_weights borrow the mapping.  qwen4_moe_create copies the bytes to
 * device memory, so a layer created through pf_gguf_moe_create outlives the file
 * handle.  File contents must not change while the handle is open. */
#ifndef PF_GGUF_H
#define PF_GGUF_H
#include "qwen4_moe.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct PfGguf PfGguf;

/* Replaces gguf_open / gguf_close (src/gguf.c:31-112).  Same acceptance rules:
 * little-endian GGUF v3, 1..100000 tensors, at most 100000 metadata entries, ASCII
 * identifier names below 128 bytes without duplicates, general.architecture
 * "qwen4exp", a power-of-two general.alignment (default 32), ranks 1..4, nonzero
 * dimensions, known tensor formats, rows that are whole blocks, aligned offsets,
 * tensors inside the file and not overlapping, the header within the first 128 MiB.
 * Status: QW4_IO when the file cannot be opened or mapped (os_errno is set),
 * QW4_UNSUPPORTED for another architecture, QW4_OVERFLOW for sizes beyond size_t,
 * QW4_OOM, QW4_FORMAT for everything else. */
Qwen4Status pf_gguf_open(const char *path, PfGguf **out, Qwen4Error *err);
void pf_gguf_close(PfGguf *g);

/* Descriptors, sorted by file offset as in the reference (src/gguf.c:92);
 * file_offset is absolute.  NULL when out of range / not found. */
size_t pf_gguf_tensor_count(const PfGguf *g);
const GgufTensor *pf_gguf_tensor(const PfGguf *g, size_t index);
const GgufTensor *pf_gguf_find(const PfGguf *g, const char *name);
size_t pf_gguf_data_offset(const PfGguf *g);
size_t pf_gguf_file_size(const PfGguf *g);
/* The mapped bytes of a tensor of this file (NULL for a foreign descriptor). */
const unsigned char *pf_gguf_tensor_bytes(const PfGguf *g, const GgufTensor *tensor);

/* What the MoE path needs of the reference's Qwen4ConfigView (src/qwen4.h:14-22). */
typedef struct {
    uint32_t blocks, trunk_blocks, mtp_blocks;
    Qwen4MoeConfig moe;          /* of the trunk layers; see pf_gguf_moe_layer_config */
    Qwen4HcShape hc;
    const char *semantic_profile; /* static string: "qwen38-q2-text-f32-v1" or "qwen38-q4-text-f32-v1" */
} PfGgufMoeModel;

/* Replaces the MoE and hyper-connection part of qwen4_config_load
 * (src/qwen4_config.c:281-299): the same keys, types, zero and range checks, the
 * refusal of unknown qwen4exp.* keys, the expert-format profile picked by layer 0's
 * routed tensors and the padded-K rule of the Q2_K down projection, with the
 * reference's statuses, subjects and details.  Keys of other blocks are not read. */
Qwen4Status pf_gguf_moe_model(const PfGguf *g, PfGgufMoeModel *out, Qwen4Error *err);

/* The block's configuration for one layer: the trunk's for layers below trunk_blocks;
 * for the multi-token-prediction layers after them Q4_K gate/up and MXFP4 down at the
 * logical width (src/qwen4_weights.c:97-99, src/qwen4_forward_gpu.m:707).
 * QW4_RANGE for a layer outside the model. */
Qwen4Status pf_gguf_moe_layer_config(const PfGgufMoeModel *model, uint32_t layer,
                                     Qwen4MoeConfig *out, Qwen4Error *err);

/* Replaces the eight MoE rows of the weight catalog and their binding
 * (src/qwen4_weights.c:91-99 through record(), :19-56; src/qwen4_forward.c:72-79):
 * blk.<layer>.ffn_gate_inp / ffn_gate_inp_shexp / ffn_{gate,up,down}_shexp /
 * ffn_{gate,up,down}_exps .weight, each checked for presence (QW4_MISSING), format
 * (QW4_FORMAT), rank and physical shape (QW4_SHAPE) and byte count.  On QW4_OK the
 * views point into the mapping. */
Qwen4Status pf_gguf_moe_weights(const PfGguf *g, const PfGgufMoeModel *model, uint32_t layer,
                                Qwen4MoeWeights *out, Qwen4Error *err);

/* Replaces create_moe (src/qwen4_forward.c:174-183): the layer's views and
 * configuration through qwen4_moe_create, which uploads the tensors. */
Qwen4Status pf_gguf_moe_create(const PfGguf *g, const PfGgufMoeModel *model, uint32_t layer,
                               Qwen4Moe **out, Qwen4Error *err);

#ifdef __cplusplus
}
#endif
#endif
