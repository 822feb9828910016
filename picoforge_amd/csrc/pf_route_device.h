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

// (p, id) arg-max over the wave: larger p wins, equal p goes to the lower id, which is what an
// ascending scan with a strict comparison selects.  p is a probability or negative (no candidate):
// nonnegative floats order like their bit patterns, so the pair travels as one 64-bit key,
// (bits of p) : (~id), through the DPP reduction steps; a lane without a candidate offers key 0.
__device__ __forceinline__ void pf_wave_argmax(float &p, uint32_t &id) {
    uint32_t hi = p < 0.0f ? 0u : __float_as_uint(p), lo = p < 0.0f ? 0u : ~id;
    auto step = [&](auto dpp) {
        const uint32_t mh = (uint32_t)dpp((int)hi), ml = (uint32_t)dpp((int)lo);
        const bool better = mh > hi || (mh == hi && ml > lo);
        hi = better ? mh : hi;
        lo = better ? ml : lo;
    };
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false); });    // quad_perm [1,0,3,2]
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false); });    // quad_perm [2,3,0,1]
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false); });   // row_half_mirror
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false); });   // row_mirror
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0x142, 0xA, 0xF, false); });   // row_bcast:15 into rows 1,3
    step([](int v) { return __builtin_amdgcn_update_dpp(v, v, 0x143, 0xC, 0xF, false); });   // row_bcast:31 into rows 2,3
    hi = (uint32_t)__builtin_amdgcn_readlane((int)hi, 63);
    lo = (uint32_t)__builtin_amdgcn_readlane((int)lo, 63);
    p = (hi | lo) ? __uint_as_float(hi) : -2.0f;
    id = (hi | lo) ? ~lo : 0xffffffffu;
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
    // the C library's expf, bit for bit (pf_expf_libm.h)
    for (int e = lane; e < E; e += PF_WAVE) {
        float shifted = z[e] - top;
        p[e] = pf_expf_libm(shifted);
    }
    pf_wave_lds_fence();
    float sum = 0.0f;
    int e0 = 0;
    for (; e0 + 32 <= E; e0 += 32) {   // serial, expert ascending; the LDS reads of a batch are requested together
        float v[32];
#pragma unroll
        for (int j = 0; j < 32; j++) v[j] = p[e0 + j];
#pragma unroll
        for (int j = 0; j < 32; j++) sum = sum + v[j];
    }
    for (int e = e0; e < E; e++) sum = sum + p[e];
    pf_wave_lds_fence();
    for (int e = lane; e < E; e += PF_WAVE) {
        float v = p[e] / sum;
        p[e] = v;
        q[e] = v;
    }
    pf_wave_lds_fence();
    float chosen = 0.0f, mine = 0.0f;
    uint32_t mine_id = 0;
    for (int slot = 0; slot < K; slot++) {
        float best = -2.0f;
        uint32_t best_id = 0xffffffffu;
        for (int e = lane; e < E; e += PF_WAVE) {
            float v = q[e];
            if (v > best) { best = v; best_id = (uint32_t)e; }
        }
        pf_wave_argmax(best, best_id);
        // no candidate at all (every probability NaN): nothing to strike out, the id stays out of range
        if (best_id != 0xffffffffu && (int)(best_id & (PF_WAVE - 1)) == lane) q[best_id] = -1.0f;
        pf_wave_lds_fence();
        chosen = chosen + best;
        if ((slot & (PF_WAVE - 1)) == lane) { mine = best; mine_id = best_id; }   // lane r keeps slots r, r + 64, ...
        // ids_out / w_out may be global memory: written from registers, 64 slots at a time
        if ((slot & (PF_WAVE - 1)) == PF_WAVE - 1 || slot == K - 1) {
            const int s = (slot & ~(PF_WAVE - 1)) + lane;
            if (s <= slot) {
                ids_out[s] = mine_id;
                w_out[s] = (norm && K <= PF_WAVE) ? mine / chosen : mine;   // chosen is final here when K <= 64
            }
        }
    }
    if (norm && K > PF_WAVE)   // each lane divides the slots it wrote itself
        for (int s = lane; s < K; s += PF_WAVE) w_out[s] = w_out[s] / chosen;
    pf_wave_lds_fence();
}
