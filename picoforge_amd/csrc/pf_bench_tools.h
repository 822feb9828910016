/* Measuring tools of bench.py (picoforge_amd/libpf_bench.so): graph-replay timing of forwards
 * through the public entry points of include/pf_moe_hip.h, single-kernel timing of the
 * hyper-connection steps, a copy kernel of known traffic.  Not part of the shipped library. */
#ifndef PF_BENCH_TOOLS_H
#define PF_BENCH_TOOLS_H
#include "../../include/pf_moe_hip.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct PfBenchPlan PfBenchPlan;
const char *pf_bench_last_error(void);

/* A replay of `forwards` forwards.  They are captured as one graph of u forwards (u = the largest
 * multiple of `layers` up to 64, at least `layers`) launched forwards / u times and one graph of the
 * remaining forwards; forward i of a graph runs layer i % layers on input block i % n_inputs of d_x
 * ([tokens, hidden] blocks, dense) into output block i % y_blocks of d_y.  kernel_limit > 0 captures
 * only the first so many kernel launches of every forward. */
int pf_bench_plan_moe(const PfHipMoe *const *moes, PfHipWork *const *works, size_t layers, const float *d_x,
                      size_t n_inputs, float *d_y, size_t y_blocks, size_t tokens, size_t forwards,
                      int kernel_limit, size_t hidden, PfBenchPlan **out);
/* The block between its two hyper-connection steps: fused != 0 one chained enqueue per forward,
 * else read, forward and add as three. */
int pf_bench_plan_hc(const PfHipMoe *moe, PfHipWork *work, const float *d_normed, const float *d_logits,
                     size_t n_inputs, float *d_residual, const float *d_inject, size_t streams, size_t tokens,
                     size_t forwards, int fused, size_t hidden, PfBenchPlan **out);
/* Replays the plan `repeats` times; ms_each[r] = elapsed time of replay r between two events on the
 * plan's stream. */
int pf_bench_plan_run(PfBenchPlan *plan, size_t repeats, float *ms_each);
void pf_bench_plan_destroy(PfBenchPlan *plan);

int pf_bench_hc_time_step(int which, float *d_cube, const float *d_logits, float *d_rows, const float *d_inject,
                          size_t tokens, size_t streams, size_t hidden, size_t iters, uint32_t *d_error_word,
                          float *elapsed_ms);
int pf_bench_copy_probe(size_t bytes, size_t launches);

#ifdef __cplusplus
}
#endif
#endif
