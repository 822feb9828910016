/* Contract types of the MoE feed-forward path.
 *
 * Layout-compatible with the part of the reference's src/qwen4_types.h that
 * src/qwen4_moe.h and src/qwen4_packed.h use: a translation unit of the
 * reference compiled against this header sees the same enum values and the
 * same struct layouts, so handles and views cross the boundary unchanged.
 * Qwen4HcShape serves the two hyper-connection steps either side of the block
 * (include/qwen4_hc.h).  Types of other blocks (attention, n-gram, recurrent
 * state) are not here. */
#ifndef PF_QWEN4_TYPES_H
#define PF_QWEN4_TYPES_H
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#define QWEN4_CONTRACT_VERSION 1u
#define QWEN4_MAX_RANK 4u

/* Status codes, values 0..20 in the reference's order (src/qwen4_types.h:14-19). */
typedef enum {
    QW4_OK = 0,
    QW4_INVALID_ARGUMENT = 1,
    QW4_MISSING = 2,
    QW4_TYPE = 3,
    QW4_RANGE = 4,
    QW4_SHAPE = 5,
    QW4_STRIDE = 6,
    QW4_FORMAT = 7,
    QW4_UNSUPPORTED = 8,
    QW4_OVERFLOW = 9,
    QW4_CAPACITY = 10,
    QW4_OOM = 11,
    QW4_OWNER = 12,
    QW4_BUSY = 13,
    QW4_STALE = 14,
    QW4_BAD_STATE = 15,
    QW4_NONFINITE = 16,
    QW4_IO = 17,
    QW4_EOF = 18,
    QW4_CANCELLED = 19,
    QW4_GPU_ERROR = 20
} Qwen4Status;

/* Error record (src/qwen4_types.h:20-26).  Every entry point accepts NULL. */
typedef struct {
    Qwen4Status code;
    int os_errno;
    uint64_t file_offset;
    uint64_t row;
    size_t requested_bytes;
    size_t completed_bytes;
    char subject[128];
    char detail[256];
} Qwen4Error;

typedef struct { const unsigned char *data; size_t bytes; } Qwen4CpuSpan;

/* Rank-2 token-major activations.  Dimensions count elements, strides and
 * capacities count BYTES; the last axis is contiguous (src/qwen4_types.h:31-46). */
typedef struct {
    const float *data;
    size_t capacity_bytes;
    size_t rank;
    size_t dim[QWEN4_MAX_RANK];
    size_t stride_bytes[QWEN4_MAX_RANK];
} Qwen4F32;

typedef struct {
    float *data;
    size_t capacity_bytes;
    size_t rank;
    size_t dim[QWEN4_MAX_RANK];
    size_t stride_bytes[QWEN4_MAX_RANK];
} Qwen4F32Mut;

typedef struct {
    uint32_t *data;
    size_t capacity_bytes;
    size_t rows;
    size_t cols;
    size_t row_stride_bytes;
} Qwen4U32Mut;

/* MoE dimensions (src/qwen4_types.h:75-80).  trunk_type holds the GGUF types of
 * the routed gate, up and down tensors; the path reads the types from the weight
 * views and only carries this field along. */
typedef struct {
    uint32_t hidden_size;
    uint32_t experts;
    uint32_t top_k;
    uint32_t intermediate;
    uint32_t shared_intermediate;
    uint32_t down_physical;
    bool norm_topk_prob;
    uint32_t trunk_type[3];
} Qwen4MoeConfig;

/* Hyper-connection dimensions (src/qwen4_types.h:69): `streams` residual streams of
 * `hidden_size` floats per token; low_rank and rms_eps belong to the gate's low-rank
 * projection and are only validated here (nonzero, eps finite and positive). */
typedef struct {
    size_t streams;
    size_t hidden_size;
    size_t low_rank;
    float rms_eps;
} Qwen4HcShape;

#endif
