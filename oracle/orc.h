/* CPU oracle of the MoE feed-forward path: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU algorithm, used as the checker
 * by tests/, by the smoke run and as the timed CPU baseline of bench.py.  The
 * shipped library never links, loads or calls anything in this directory.
 *
 * Every function keeps the reference's evaluation order so that, compiled with
 * -ffp-contract=off -fno-fast-math, its results are bit-identical to the
 * reference's C path.  Types come from include/ (layout-compatible with the
 * reference); functions carry an orc_ prefix so that the oracle, a build of the
 * reference and the product library can be loaded side by side.
 *
 * Every function below is pinned by checks that do not restate its formula:
 * tests/test_oracle_packed.py, tests/test_oracle_moe.py and tests/test_oracle_hc.py
 * (known answers the reference's own tests hold, independent numpy evaluations,
 * closed forms, and the reference's compiled C path bit for bit), and
 * tests/test_golden.py (vectors written by that compiled path). */
#ifndef PF_ORACLE_H
#define PF_ORACLE_H
#include "../include/qwen4_moe.h"
#include "../include/qwen4_hc.h"

typedef struct OrcMoe OrcMoe;
typedef struct OrcMoeWork OrcMoeWork;

/* src/gguf.c:11-22, src/qwen4_packed.c:8-33 */
const GgufFormat *orc_format(uint32_t id);
Qwen4Status orc_packed_layout_init(const GgufTensor *, size_t k_logical, QW4PackedLayout *, Qwen4Error *);
/* src/qwen4_packed.c:54-66 */
float orc_half_value(uint16_t bits);
/* src/qwen4_packed.c:67-122 (F32, F16, Q8_0, Q2_K, Q4_K, IQ2_XXS, BF16, MXFP4) */
float orc_packed_value(const unsigned char *row, size_t column, uint32_t type);
/* src/qwen4_packed.c:124-143 and :145-181 */
Qwen4Status orc_packed_decode_row(const QW4PackedCpuView *, size_t expert, size_t row,
                                  float *out, size_t out_elements, Qwen4Error *);
Qwen4Status orc_packed_matmul(const QW4PackedCpuView *, size_t expert, Qwen4F32 x, Qwen4F32Mut y,
                              Qwen4Error *);
/* src/qwen4_cpu_internal.h:103-107, src/qwen4_base.c:76-99; kind 0 sigmoid, 1 SiLU */
float orc_sigmoid(float x);
float orc_silu(float x);
Qwen4Status orc_activate(int kind, Qwen4F32 x, Qwen4F32Mut out, Qwen4Error *);
/* src/qwen4_moe.c:188-249, :251-303 */
Qwen4Status orc_moe_route(const Qwen4MoeConfig *, Qwen4F32 logits, Qwen4MoeRoutes,
                          Qwen4F32Mut probabilities, Qwen4Error *);
Qwen4Status orc_moe_group_pairs(const Qwen4MoeConfig *, Qwen4U32Mut ids, QW4MoeGrouping, Qwen4Error *);
/* src/qwen4_moe.c:47-76, :80-129, :130-132, :384-431 */
Qwen4Status orc_moe_create(const Qwen4MoeConfig *, const Qwen4MoeWeights *, OrcMoe **, Qwen4Error *);
void orc_moe_destroy(OrcMoe *);
Qwen4Status orc_moe_work_size(const OrcMoe *, size_t token_cap, size_t *bytes, Qwen4Error *);
Qwen4Status orc_moe_work_create(const OrcMoe *, size_t token_cap, size_t byte_budget, OrcMoeWork **,
                                Qwen4Error *);
Qwen4Status orc_moe_work_reset(OrcMoeWork *, Qwen4Error *);
void orc_moe_work_destroy(OrcMoeWork *);
void orc_moe_observe(OrcMoeWork *, QW4MoeObserver, void *);
Qwen4Status orc_moe_forward(const OrcMoe *, Qwen4F32 x, Qwen4F32Mut y, Qwen4MoeRoutes *optional_routes,
                            OrcMoeWork *, Qwen4Error *);
/* src/qwen4_base.c:142-160 and :161-175: the hyper-connection read before the block
 * and the injection after it */
Qwen4Status orc_hc_read(const Qwen4HcShape *, Qwen4F32 normed, Qwen4F32 gate_logits, Qwen4F32Mut mixed,
                        Qwen4Error *);
Qwen4Status orc_hc_add(const Qwen4HcShape *, Qwen4F32Mut residual, Qwen4F32 block_out, Qwen4F32 inject,
                       Qwen4Error *);
#endif
