// Fast routing of one token by one wave: logits in registers, selection in logit
// space, and a closeness test that sends ambiguous tokens to the reference-order
// path.  Selecting on logits equals selecting on probabilities (src/qwen4_moe.c:233-246)
// whenever adjacent selected logits are further apart than the test's tolerance,
// because exp and the division by a common sum are monotone up to a few ulps.
#pragma once
#include "pf_device.h"

__device__ __forceinline__ float pf_dpp_max_step(float v, const int which) {
    int moved;
    const int bits = __float_as_int(v);
    switch (which) {
    case 0: moved = __builtin_amdgcn_update_dpp(bits, bits, 0xB1, 0xF, 0xF, false); break;   // quad_perm [1,0,3,2]
    case 1: moved = __builtin_amdgcn_update_dpp(bits, bits, 0x4E, 0xF, 0xF, false); break;   // quad_perm [2,3,0,1]
    case 2: moved = __builtin_amdgcn_update_dpp(bits, bits, 0x141, 0xF, 0xF, false); break;  // row_half_mirror
    case 3: moved = __builtin_amdgcn_update_dpp(bits, bits, 0x140, 0xF, 0xF, false); break;  // row_mirror
    case 4: moved = __builtin_amdgcn_update_dpp(bits, bits, 0x142, 0xA, 0xF, false); break;  // row_bcast:15 into rows 1,3
    default: moved = __builtin_amdgcn_update_dpp(bits, bits, 0x143, 0xC, 0xF, false); break; // row_bcast:31 into rows 2,3
    }
    return fmaxf(v, __int_as_float(moved));
}

// Maximum over the wave, returned in every lane (read back from lane 63).
__device__ __forceinline__ float pf_wave_max_fast(float v) {
    v = pf_dpp_max_step(v, 0);
    v = pf_dpp_max_step(v, 1);
    v = pf_dpp_max_step(v, 2);
    v = pf_dpp_max_step(v, 3);
    v = pf_dpp_max_step(v, 4);
    v = pf_dpp_max_step(v, 5);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

struct PfRouteResult {
    uint32_t id;     // lane r < top_k: expert of slot r
    float weight;    // lane r < top_k: route weight of slot r
    bool close;      // uniform: some adjacent pair of the k+1 best logits is within tolerance
    bool bad;        // uniform: a nonfinite logit was seen
};

// z_row, ssq_row: the token's E logits and sums of squared products.  Expert e
// lives in lane e / NPL, register e % NPL, so the lowest lane holding the
// maximum also holds the lowest expert id among equal logits.
template <int NPL>
__device__ __forceinline__ PfRouteResult pf_route_fast_wave(const float *z_row, const float *ssq_row, int E, int K,
                                                            bool norm, int hidden, int lane) {
    float v[NPL], s2[NPL];
    bool bad = false;
#pragma unroll
    for (int j = 0; j < NPL; j++) {
        const int e = lane * NPL + j;
        v[j] = e < E ? z_row[e] : -INFINITY;
        s2[j] = e < E ? ssq_row[e] : 0.0f;
        bad |= e < E && !pf_finite(v[j]);
    }
    bad = __any(bad);
    float total = 0.0f, top_all = 0.0f;
    if (!norm) {   // unnormalised weights need the full softmax denominator
        float m = v[0];
#pragma unroll
        for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
        top_all = pf_wave_max_fast(m);
#pragma unroll
        for (int j = 0; j < NPL; j++) total += expf(v[j] - top_all);   // exp(-inf) = 0 for padding
        total = pf_wave_sum(total);
    }
    const int rounds = K < E ? K + 1 : K;
    uint32_t my_id = 0;
    float my_z = 0.0f, my_s2 = 0.0f;
    for (int r = 0; r < rounds; r++) {
        float m = v[0];
#pragma unroll
        for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
        const float wm = pf_wave_max_fast(m);
        const unsigned long long holders = __ballot(m == wm);
        const int owner = holders ? __ffsll((long long)holders) - 1 : 0;   // no holder: NaN logits, flagged as bad
        int jl = NPL - 1;
#pragma unroll
        for (int j = NPL - 1; j >= 0; j--) jl = v[j] == wm ? j : jl;
        const int jsel = __builtin_amdgcn_readlane(jl, owner);
        float s2sel = s2[0];
#pragma unroll
        for (int j = 1; j < NPL; j++) s2sel = j == jsel ? s2[j] : s2sel;
        s2sel = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s2sel), owner));
#pragma unroll
        for (int j = 0; j < NPL; j++) v[j] = (lane == owner && j == jsel) ? -INFINITY : v[j];
        if (lane == r) {
            my_id = (uint32_t)(owner * NPL + jsel);
            my_z = wm;
            my_s2 = s2sel;
        }
    }
    // closeness of neighbours in the sorted list of the k+1 best
    const float next_z = __shfl_down(my_z, 1), next_s2 = __shfl_down(my_s2, 1);
    const float top = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_z), 0));
    // Noise model of a K-term FP32 sum in any order: standard deviation
    // u * sqrt(K * sum(products^2) / 6); eight of those per logit, plus the
    // rounding of z - max and of the exponential.
    const float u = 5.9604645e-8f, hk = (float)hidden / 6.0f;
    const float tol = 8.0f * u * (sqrtf(hk * my_s2) + sqrtf(hk * next_s2)) + 4e-6f * fmaxf(1.0f, top - next_z);
    const bool close = __any(lane + 1 < rounds && !(my_z - next_z > tol));
    float e = lane < K ? expf(my_z - top) : 0.0f;
    float weight;
    if (norm) weight = e / pf_wave_sum(e);
    else weight = e * expf(top - top_all) / total;   // exp(z - top_all) / total, without overflow
    PfRouteResult out;
    out.id = my_id;
    out.weight = weight;
    out.close = close;
    out.bad = bad;
    return out;
}
