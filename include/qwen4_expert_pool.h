/* A bounded cache of routed experts read from the model file into device memory: the interface of
 * src/qwen4_expert_pool.h of the reference (same names, arguments and results), with the three regions
 * in HBM instead of page-aligned host memory.
 *
 * An expert is the gate, up and down slice of one (layer, expert).  The pool holds `slots` of them in
 * three device regions, one per matrix, so that a kernel which addresses experts as
 * region + slot * bytes_per_expert reads the pool exactly as it reads a resident expert tensor.  On a
 * miss the least recently used slot that is not pinned is overwritten; experts acquired for the current
 * batch stay pinned until released, so an eviction never pulls one out from under a running kernel.
 * One thread at a time per pool. */
#ifndef PICOFORGE_AMD_QWEN4_EXPERT_POOL_H
#define PICOFORGE_AMD_QWEN4_EXPERT_POOL_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct QW4ExpertPool QW4ExpertPool;
typedef struct { uint64_t offset[3]; } QW4ExpertLayer;   /* file offsets of the layer's gate, up and down tensors */
/* acquire_ns: wall time spent inside qw4_pool_acquire, i.e. how long batches waited for the file. */
typedef struct { uint64_t hits, misses, evictions, bytes_read, acquire_ns; } QW4PoolStats;

/* Replaces qw4_pool_create (src/qwen4_expert_pool.c:41-68).  fd: the model file, open for reading.
 * bytes[m]: one expert's slice of matrix m as the file stores it; expert e of layer l, matrix m, is at
 * layers[l].offset[m] + e * bytes[m].  NULL on failure (bad argument, no device, out of memory). */
QW4ExpertPool *qw4_pool_create(int fd, const QW4ExpertLayer *layers, uint32_t n_layers, uint32_t experts,
                               const size_t bytes[3], uint32_t slots);
void qw4_pool_destroy(QW4ExpertPool *pool);
/* Replaces qw4_pool_acquire (src/qwen4_expert_pool.c:104-135): makes the n experts of `layer` resident
 * and pins them; slots[i] is where experts[i] now lives.  An expert listed twice shares its slot and is
 * pinned twice.  Which slot is taken and what is evicted is decided in list order before anything is
 * read, so hits, evictions and slots do not depend on the reader count.  Returns 0, or -1 when every
 * slot is pinned, an id is out of range or a read fails (then nothing stays pinned by this call and the
 * slots it had taken are forgotten). */
int qw4_pool_acquire(QW4ExpertPool *pool, uint32_t layer, const uint32_t *experts, size_t n, uint32_t *slots);
/* Replaces qw4_pool_set_readers (:85): reads of one acquire that run at once (1 = serial; default 8). */
void qw4_pool_set_readers(QW4ExpertPool *pool, uint32_t readers);
void qw4_pool_release(QW4ExpertPool *pool, const uint32_t *slots, size_t n);
/* The whole pool of one matrix: a DEVICE pointer (the reference returns host memory it wraps in a
 * no-copy GPU buffer) and its size. */
void *qw4_pool_region(const QW4ExpertPool *pool, int matrix, size_t *bytes);
QW4PoolStats qw4_pool_stats(const QW4ExpertPool *pool);

/* Extensions without a counterpart in the reference (its pool holds file bytes and its kernels read them).
 * pf_pool_set_formats tells the pool the three matrices' GGUF types and shapes (rows of k_storage[m] weights,
 * n_out[m] rows per expert; bytes[m] of qw4_pool_create must be one expert's file bytes of that shape) so that
 * every slot holds its expert in the layout this library's kernels read: IQ2_XXS, Q8_0 and MXFP4 are split into
 * payloads and scales on arrival, the other formats stay as the file stores them.  Needed for layers whose routed
 * tensors are in one of those three formats (both checkpoint profiles); before the first acquire only.  0 or -1. */
int pf_pool_set_formats(QW4ExpertPool *pool, const uint32_t gguf_type[3], const size_t k_storage[3], const size_t n_out[3]);
uint32_t pf_pool_slots(const QW4ExpertPool *pool);
size_t pf_pool_scale_offset(const QW4ExpertPool *pool, int matrix);   /* where matrix m's scales start in its region; 0: not split */
uint32_t pf_pool_format(const QW4ExpertPool *pool, int matrix);      /* UINT32_MAX: slots as the file stores them */

#ifdef __cplusplus
}
#endif
#endif
