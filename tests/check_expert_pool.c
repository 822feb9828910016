/* Host-only harness of the expert pool (picoforge_amd/csrc/qwen4_expert_pool.c): the HIP shim it calls is replaced by
 * plain memory, so the bookkeeping, the reader threads and their hand-over run on the CPU, under the sanitizers
 * (tests/test_expert_pool_host.py).  200 acquires of one to three experts over two layers through four slots; every
 * acquired slot must hold its expert's three slices as the file stores them. */
#define _DEFAULT_SOURCE
#include "../include/qwen4_expert_pool.h"
#include "../include/pf_moe_hip.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>
#include <fcntl.h>
struct PfHipStage { unsigned char *host; size_t bytes; };
int pf_hip_malloc(void **p, size_t b) { *p = malloc(b); return *p ? 0 : 3; }
void pf_hip_free(void *p) { free(p); }
int pf_hip_memcpy_h2d(void *d, const void *s, size_t b) { memcpy(d, s, b); return 0; }
int pf_hip_stage_create(size_t bytes, PfHipStage **out) { PfHipStage *s = calloc(1, sizeof *s); s->host = malloc(bytes); s->bytes = bytes; *out = s; return 0; }
void pf_hip_stage_destroy(PfHipStage *s) { if (s) { free(s->host); free(s); } }
void *pf_hip_stage_host(PfHipStage *s) { return s->host; }
int pf_hip_pool_store_staged(PfHipStage *st, uint32_t t, size_t k, size_t n, size_t slots, void *region, size_t slot, size_t fb) {
    (void)t; (void)k; (void)n;
    if (slot >= slots || fb > st->bytes) return 1;
    memcpy((unsigned char *)region + slot * fb, st->host, fb);
    return 0;
}
int pf_hip_pool_region_plan(uint32_t a, size_t b, size_t c, size_t d, size_t *e, size_t *f, size_t *g, size_t *h) { (void)a;(void)b;(void)c;(void)d;(void)e;(void)f;(void)g;(void)h; return 1; }
int pf_hip_pool_store(uint32_t a, size_t b, size_t c, size_t d, void *e, size_t f, const void *g) { (void)a;(void)b;(void)c;(void)d;(void)e;(void)f;(void)g; return 1; }
int main(void) {
    const size_t sizes[3] = {96, 64, 160};
    const uint32_t layers = 2, experts = 6, slots = 4;
    size_t total = 4096 + layers * experts * (96 + 64 + 160);
    unsigned char *blob = malloc(total);
    for (size_t i = 0; i < total; i++) blob[i] = (unsigned char)(i * 7 + 3);
    char path[] = "/tmp/pf_pool_XXXXXX";
    int fd = mkstemp(path);
    if (write(fd, blob, total) != (ssize_t)total) return 2;
    QW4ExpertLayer table[2];
    size_t at = 4096;
    for (uint32_t l = 0; l < layers; l++) for (int m = 0; m < 3; m++) { table[l].offset[m] = at; at += experts * sizes[m]; }
    QW4ExpertPool *p = qw4_pool_create(fd, table, layers, experts, sizes, slots);
    if (!p) return 3;
    for (int round = 0; round < 200; round++) {
        uint32_t ids[3] = {(uint32_t)(round % 6), (uint32_t)((round * 5 + 1) % 6), (uint32_t)((round + 3) % 6)}, out[3];
        int n = 1 + round % 3;
        int rc = qw4_pool_acquire(p, (uint32_t)(round & 1), ids, (size_t)n, out);
        if (rc == 0) {
            for (int i = 0; i < n; i++)
                for (int m = 0; m < 3; m++) {
                    size_t bytes; unsigned char *region = qw4_pool_region(p, m, &bytes);
                    if (memcmp(region + out[i] * sizes[m], blob + table[round & 1].offset[m] + ids[i] * sizes[m], sizes[m])) { printf("mismatch round %d\n", round); return 4; }
                }
            qw4_pool_release(p, out, (size_t)n);
        }
    }
    QW4PoolStats st = qw4_pool_stats(p);
    printf("hits %llu misses %llu\n", (unsigned long long)st.hits, (unsigned long long)st.misses);
    qw4_pool_destroy(p);
    close(fd); unlink(path);
    free(blob);
    return st.misses > 100 && st.hits > 10 ? 0 : 5;
}
