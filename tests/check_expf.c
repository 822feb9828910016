/* Compares pf_expf_libm (the expf the HIP kernels evaluate, picoforge_amd/csrc/pf_expf_libm.h)
 * with the host C library's expf, bit for bit.
 *
 *   check_expf [count]   count random bit patterns (default 20 million) plus every float within
 *                        +-1 of the overflow and underflow thresholds
 *   check_expf --all     all 2^32 bit patterns (about half a minute)
 *
 * Prints the first mismatches and "mismatches N"; exit status 0 either way, the caller decides.
 * Build with -ffp-contract=off so that only the fused steps the header writes are fused. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../picoforge_amd/csrc/pf_expf_libm.h"

static unsigned long long checked, bad;
static void one(float x) {
    if (x != x) return;
    const float a = expf(x), m = pf_expf_libm(x);
    checked++;
    if (memcmp(&a, &m, 4)) {
        if (bad < 8) printf("x=%a libm=%a mine=%a\n", x, a, m);
        bad++;
    }
}

int main(int argc, char **argv) {
    if (argc > 1 && !strcmp(argv[1], "--all")) {
        for (unsigned long long b = 0; b < (1ull << 32); b++) {
            const uint32_t u = (uint32_t)b;
            float x;
            memcpy(&x, &u, 4);
            one(x);
        }
    } else {
        unsigned long long n = argc > 1 ? strtoull(argv[1], 0, 10) : 20000000ull, seed = 88172645463325252ull;
        for (unsigned long long i = 0; i < n; i++) {
            seed ^= seed << 13; seed ^= seed >> 7; seed ^= seed << 17;
            const uint32_t u = (uint32_t)(seed >> 20);
            float x;
            memcpy(&x, &u, 4);
            if (!(fabsf(x) < 110.0f)) x = (float)((double)(seed % 2200000) / 10000.0 - 110.0);
            one(x);
        }
        for (float x = -104.97f; x < -102.97f; x = nextafterf(x, 0.0f)) one(x);
        for (float x = 87.72f; x < 89.72f; x = nextafterf(x, 100.0f)) one(x);
        const float special[] = {0.0f, -0.0f, INFINITY, -INFINITY, 89.0f, -104.0f, 1e-30f, -1e-30f, 0x1p-149f, -0x1p-149f};
        for (size_t i = 0; i < sizeof special / sizeof *special; i++) one(special[i]);
    }
    printf("checked %llu mismatches %llu\n", checked, bad);
    return 0;
}
