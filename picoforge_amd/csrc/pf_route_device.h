// Reference-order routing, shared by the routing kernels and the decode path.
//
// Every function here keeps a*b+c as two roundings (contraction is switched off
// inside each body): they restate src/qwen4_packed.c:164-179 (serial logit) and
// src/qwen4_moe.c:219-247 (softmax, k rounds of arg-max, renormalisation).
#pragma once
#include "pf_device.h"
#include <math.h>

__device__ __forceinline__ void pf_wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// (p, id) arg-max over the wave: larger p wins, equal p goes to the lower id,
// which is what an ascending scan with a strict comparison selects.
__device__ __forceinline__ void pf_wave_argmax(float &p, uint32_t &id) {
    for (int m = 1; m < PF_WAVE; m <<= 1) {
        float op = __shfl_xor(p, m);
        uint32_t oid = __shfl_xor(id, m);
        if (op > p || (op == p && oid < id)) { p = op; id = oid; }
    }
}

// One router logit in the reference's order: k ascending, product then sum.
__device__ __forceinline__ float pf_serial_logit(const float *w, const float *x, int K) {
#pragma clang fp contract(off)
    float sum = 0.0f;
    for (int k = 0; k < K; k++) {
        float p = w[k] * x[k];
        sum = sum + p;
    }
    return sum;
}

// Reference-order routing of one token by one wave.  z, p, q: LDS arrays of E
// floats (q is scratch).  Writes ids/weights (top_k entries) and leaves the
// probabilities in p.
__device__ __forceinline__ void pf_route_exact_wave(const float *z, float *p, float *q, int E, int K, bool norm,
                                                    uint32_t *ids_out, float *w_out, int lane) {
#pragma clang fp contract(off)
    float top = -INFINITY;
    for (int e = lane; e < E; e += PF_WAVE) top = fmaxf(top, z[e]);
    top = pf_wave_max(top);
    // exponent in double, rounded once: the correctly rounded expf
    for (int e = lane; e < E; e += PF_WAVE) {
        float shifted = z[e] - top;
        p[e] = (float)exp((double)shifted);
    }
    pf_wave_lds_fence();
    float sum = 0.0f;
    for (int e = 0; e < E; e++) sum = sum + p[e];   // serial, expert ascending
    pf_wave_lds_fence();
    for (int e = lane; e < E; e += PF_WAVE) {
        float v = p[e] / sum;
        p[e] = v;
        q[e] = v;
    }
    pf_wave_lds_fence();
    float chosen = 0.0f;
    for (int slot = 0; slot < K; slot++) {
        float best = -2.0f;
        uint32_t best_id = 0xffffffffu;
        for (int e = lane; e < E; e += PF_WAVE) {
            float v = q[e];
            if (v > best) { best = v; best_id = (uint32_t)e; }
        }
        pf_wave_argmax(best, best_id);
        if ((int)(best_id & (PF_WAVE - 1)) == lane) q[best_id] = -1.0f;
        pf_wave_lds_fence();
        chosen = chosen + best;
        if (lane == 0) { ids_out[slot] = best_id; w_out[slot] = best; }
    }
    pf_wave_lds_fence();
    if (norm && lane == 0)
        for (int slot = 0; slot < K; slot++) w_out[slot] = w_out[slot] / chosen;
    pf_wave_lds_fence();
}
