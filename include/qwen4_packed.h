/* Packed (quantised) linear contract of the MoE path.
 *
 * Layout-compatible with the host-visible part of the reference's
 * src/qwen4_packed.h:6-19 and the two GGUF descriptor types it takes from
 * src/gguf.h:20-25.  Every format the reference registers is executed: F32 (type
 * 0), F16 (1), Q8_0 (8), Q2_K (10), Q4_K (12), IQ2_XXS (16), BF16 (30) and MXFP4
 * (39); unknown type ids are refused with QW4_FORMAT as in the reference
 * (src/qwen4_packed_internal.h:57-63). */
#ifndef PF_QWEN4_PACKED_H
#define PF_QWEN4_PACKED_H
#include "qwen4_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One row of the GGUF block table (src/gguf.h:20, values src/gguf.c:12-16). */
typedef struct {
    uint32_t id;
    const char *name;
    size_t block;   /* elements per block */
    size_t bytes;   /* bytes per block */
} GgufFormat;

/* Tensor descriptor as the GGUF reader produces it (src/gguf.h:21-25).
 * shape[0] is the storage (innermost) dimension, shape[1] the output rows,
 * shape[2] the expert count. */
typedef struct {
    char name[128];
    uint32_t type;
    uint32_t rank;
    size_t shape[4];
    size_t file_offset;
    size_t bytes;
} GgufTensor;

/* Derived geometry of one packed tensor (src/qwen4_packed.h:6-10).
 * Byte address of block b of row n of expert e:
 *   e * expert_bytes + n * row_bytes + b * block_bytes. */
typedef struct {
    uint32_t gguf_type;
    size_t k_storage;
    size_t k_logical;
    size_t n_out;
    size_t n_experts;
    size_t row_bytes;
    size_t expert_bytes;
    size_t tensor_bytes;
} QW4PackedLayout;

typedef struct {
    Qwen4CpuSpan span;
    QW4PackedLayout layout;
} QW4PackedCpuView;

/* Replaces gguf_format (src/gguf.c:11-22) for the ids this build knows about.
 * Returns NULL instead of terminating the process on an unknown id. */
const GgufFormat *gguf_format(uint32_t id);

/* Replaces qw4_packed_layout_init (src/qwen4_packed.c:8-33): host-only, integer,
 * overflow-checked. */
Qwen4Status qw4_packed_layout_init(const GgufTensor *tensor, size_t k_logical,
                                   QW4PackedLayout *out, Qwen4Error *err);

/* Replaces qw4_packed_decode_row (src/qwen4_packed.c:124-143).  The row is
 * uploaded, decoded by a HIP kernel that follows the reference's per-element
 * arithmetic (results are bit-identical), and copied back.  `out` is untouched
 * unless the call returns QW4_OK. */
Qwen4Status qw4_packed_decode_row(const QW4PackedCpuView *weights, size_t expert,
                                  size_t row, float *out, size_t out_elements,
                                  Qwen4Error *err);

/* Replaces qw4_packed_matmul (src/qwen4_packed.c:145-181): y[m,n] = sum over
 * k < k_logical of W_expert[n,k] * x[m,k].  Runs a HIP kernel with one lane per
 * output that multiplies and adds in ascending k without contraction, which is
 * the reference's order: results are bit-identical.  Any nonfinite weight,
 * input, product or partial sum gives QW4_NONFINITE and leaves y untouched. */
Qwen4Status qw4_packed_matmul(const QW4PackedCpuView *weights, size_t expert,
                              Qwen4F32 x, Qwen4F32Mut y, Qwen4Error *err);

#ifdef __cplusplus
}
#endif
#endif
