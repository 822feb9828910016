// Fast routing: logits in registers, selection in logit space, and a closeness test that
// sends ambiguous tokens to the reference-order path.  Selecting on logits equals selecting
// on probabilities (src/qwen4_moe.c:233-246) whenever adjacent selected logits are further
// apart than the test's tolerance, because exp and the division by a common sum are
// monotone up to a few ulps.
//
// Two forms: one wave routes a whole token (pf_route_fast_wave), or several waves each
// reduce a contiguous chunk of experts to their best k+1 candidates (pf_route_stage1) and
// one wave merges the candidates (pf_route_stage2).  Expert e of a chunk lives in lane
// e / NPL, register e % NPL, so the lowest lane holding the maximum also holds the lowest
// expert id among equal logits: ties go to the lower id, as an ascending scan with a strict
// comparison decides them.
#pragma once
#include "pf_device.h"
#include "pf_route_device.h"

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

// Expert lane * NPL + j of a row of E values into register j (fill beyond E).  The registers of a lane are
// consecutive in memory: requested as 16-byte pieces where the row allows it, and all before the first is used
// (a bounds test per element would make every element a round trip of its own).
template <int NPL>
__device__ __forceinline__ void pf_load_row(const float *row, int E, int lane, float fill, float (&v)[NPL]) {
    const int base = lane * NPL;
    if (NPL % 4 == 0 && E % 4 == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
#pragma unroll
        for (int j = 0; j < NPL; j += 4) {
            float4 q = make_float4(fill, fill, fill, fill);
            if (base + j < E) q = *reinterpret_cast<const float4 *>(row + base + j);
            v[j] = q.x; v[j + 1] = q.y; v[j + 2] = q.z; v[j + 3] = q.w;
        }
        return;
    }
    float got[NPL];
#pragma unroll
    for (int j = 0; j < NPL; j++) got[j] = row[min(base + j, E - 1)];
#pragma unroll
    for (int j = 0; j < NPL; j++) v[j] = base + j < E ? got[j] : fill;
}

struct PfRouteResult {
    uint32_t id;     // lane r < top_k: expert of slot r
    float weight;    // lane r < top_k: route weight of slot r
    bool close;      // uniform: some adjacent pair of the k+1 best logits is within tolerance
    bool bad;        // uniform: a nonfinite logit was seen
};

// One round of extraction: the largest remaining value of the wave, its holder and register.
template <int NPL>
__device__ __forceinline__ void pf_extract_max(float (&v)[NPL], int lane, float &wm, int &owner, int &jsel) {
    float m = v[0];
#pragma unroll
    for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
    wm = pf_wave_max_fast(m);
    const unsigned long long holders = __ballot(m == wm);
    owner = holders ? __ffsll((long long)holders) - 1 : 0;   // no holder: NaN logits, flagged as bad
    int jl = NPL - 1;
#pragma unroll
    for (int j = NPL - 1; j >= 0; j--) jl = v[j] == wm ? j : jl;
    jsel = NPL == 1 ? 0 : __builtin_amdgcn_readlane(jl, owner);
#pragma unroll
    for (int j = 0; j < NPL; j++) v[j] = (lane == owner && j == jsel) ? -INFINITY : v[j];
}

// Closeness test and route weights from the sorted k+1 best: lane r holds (my_z, my_s2).
// total/top_all: softmax denominator and its reference maximum (only used when !norm).
__device__ __forceinline__ void pf_route_finish_wave(float my_z, float my_s2, int K, int rounds, bool norm, int hidden,
                                                     float total, float top_all, int lane, float &weight, bool &close) {
    const float next_z = __shfl_down(my_z, 1), next_s2 = __shfl_down(my_s2, 1);
    const float top = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_z), 0));
    // Noise model of a K-term FP32 sum in any order: standard deviation
    // u * sqrt(K * sum(products^2) / 6); eight of those per logit, plus the
    // rounding of z - max and of the exponential.
    const float u = 5.9604645e-8f, hk = (float)hidden / 6.0f;
    const float tol = 8.0f * u * (sqrtf(hk * my_s2) + sqrtf(hk * next_s2)) + 4e-6f * fmaxf(1.0f, top - next_z);
    // Far below the maximum exp() reaches the subnormals and zero, where distinct logits give
    // equal probabilities and the reference's tie rule (lower id) decides: serial-order path.
    close = __any((lane + 1 < rounds && !(my_z - next_z > tol)) || (lane < rounds && !(top - my_z < 80.0f)));
    const float e = lane < K ? expf(my_z - top) : 0.0f;
    if (norm) weight = e / pf_wave_sum(e);
    else weight = e * expf(top - top_all) / total;
}

// ---- selection by packed keys -------------------------------------------------------------
// The extraction above costs about a hundred instructions a round.  This one costs a quarter of
// that: every logit becomes one 32-bit key, the order-preserving integer of the float with its low
// ten bits replaced by 1023 - id, so that a plain unsigned maximum names value and expert at once
// and keys are unique.  Each lane sorts its keys once (maxima and minima of a sorting network);
// a round then is the wave's maximum over the lanes' heads and a shift of the winner's list.
// Ten mantissa bits are lost, so the order among the extracted is only approximate: the exact
// logits of the extracted are fetched back from the registers they came from (lane id / NPL,
// register id % NPL) and ranked again exactly (value descending, then id ascending), and one
// more key than needed is extracted: if it has the same truncated value as the last one needed,
// an expert that was not extracted could belong in front of it, and the token is reported as
// close (it is then routed in the reference's serial order).
#define PF_KEY_ID_BITS 10
#define PF_KEY_ID_MASK 1023u

__device__ __forceinline__ uint32_t pf_order_bits(float z) {
    const uint32_t u = __float_as_uint(z);   // -0 sorts just below +0: the exact ranking afterwards treats them as equal
    return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}

__device__ __forceinline__ uint32_t pf_dpp_umax_step(uint32_t v, const int which) {
    int moved;
    const int bits = (int)v;
    // lanes a step does not reach receive 0, the identity of the unsigned maximum (so the move can merge into it)
    switch (which) {
    case 0: moved = __builtin_amdgcn_update_dpp(0, bits, 0xB1, 0xF, 0xF, true); break;   // quad_perm [1,0,3,2]
    case 1: moved = __builtin_amdgcn_update_dpp(0, bits, 0x4E, 0xF, 0xF, true); break;   // quad_perm [2,3,0,1]
    case 2: moved = __builtin_amdgcn_update_dpp(0, bits, 0x141, 0xF, 0xF, true); break;  // row_half_mirror
    case 3: moved = __builtin_amdgcn_update_dpp(0, bits, 0x140, 0xF, 0xF, true); break;  // row_mirror
    case 4: moved = __builtin_amdgcn_update_dpp(0, bits, 0x142, 0xA, 0xF, false); break;  // row_bcast:15 into rows 1,3
    default: moved = __builtin_amdgcn_update_dpp(0, bits, 0x143, 0xC, 0xF, false); break; // row_bcast:31 into rows 2,3
    }
    return max(v, (uint32_t)moved);
}

template <int NPL> struct PfTopk {
    uint32_t key[NPL];   // this lane's keys, largest first; 0 = none left

    // v[j]: logit of expert lane * NPL + j (experts beyond E: any value)
    __device__ __forceinline__ void setup(const float (&v)[NPL], int E, int lane) {
#pragma unroll
        for (int j = 0; j < NPL; j++) {
            const uint32_t id = (uint32_t)(lane * NPL + j);
            key[j] = id < (uint32_t)E ? ((pf_order_bits(v[j]) & ~PF_KEY_ID_MASK) | (PF_KEY_ID_MASK - id)) : 0u;
        }
        // bitonic sorting network, descending
#pragma unroll
        for (int size = 2; size <= NPL; size *= 2) {
#pragma unroll
            for (int stride = size / 2; stride > 0; stride /= 2) {
#pragma unroll
                for (int i = 0; i < NPL; i++) {
                    const int partner = i ^ stride;
                    if (partner > i) {
                        const bool descending = (i & size) == 0;
                        const uint32_t hi = max(key[i], key[partner]), lo = min(key[i], key[partner]);
                        key[i] = descending ? hi : lo;
                        key[partner] = descending ? lo : hi;
                    }
                }
            }
        }
    }

    // the largest key left in the wave, removed from its lane's list; 0 when nothing is left
    __device__ __forceinline__ uint32_t pop() {
        uint32_t m = key[0];
        m = pf_dpp_umax_step(m, 0);
        m = pf_dpp_umax_step(m, 1);
        m = pf_dpp_umax_step(m, 2);
        m = pf_dpp_umax_step(m, 3);
        m = pf_dpp_umax_step(m, 4);
        m = pf_dpp_umax_step(m, 5);
        const uint32_t best = (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
        const bool mine = key[0] == best && best != 0u;
#pragma unroll
        for (int j = 0; j + 1 < NPL; j++) key[j] = mine ? key[j + 1] : key[j];
        key[NPL - 1] = mine ? 0u : key[NPL - 1];
        return best;
    }
};

__device__ __forceinline__ uint32_t pf_key_id(uint32_t key) { return PF_KEY_ID_MASK - (key & PF_KEY_ID_MASK); }

// Lane r < count holds the r-th popped key in my_key (count <= 64: the k + 1 best and one more).  Fetches the
// exact logit and sum of squares of the first count - 1 and ranks them exactly; afterwards lane r < count - 1
// holds the r-th best (id, z, s2).  Returns (uniformly) whether the extra key ties the last one needed.
template <int NPL>
__device__ __forceinline__ bool pf_topk_exact_order(uint32_t my_key, int count, const float (&v)[NPL], const float (&s2)[NPL],
                                                    int lane, uint32_t &id, float &z, float &ssq) {
    const int need = count - 1;
    const bool have = lane < need && my_key != 0u;
    id = have ? pf_key_id(my_key) : 0xffffffffu;
    const int at = have ? (int)id : 0;
    z = -INFINITY;
    ssq = 0.0f;
#pragma unroll
    for (int j = 0; j < NPL; j++) {
        const float vz = __shfl(v[j], at / NPL), vs = __shfl(s2[j], at / NPL);
        if (have && at % NPL == j) { z = vz; ssq = vs; }
    }
    const uint32_t last = (uint32_t)__builtin_amdgcn_readlane((int)my_key, need - 1);
    const uint32_t extra = (uint32_t)__builtin_amdgcn_readlane((int)my_key, need);
    const bool ambiguous = extra != 0u && (extra >> PF_KEY_ID_BITS) == (last >> PF_KEY_ID_BITS);
    // exact rank among the needed ones: how many come before this lane's
    int rank = 0;
    for (int q = 0; q < need; q++) {
        const float zq = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(z), q));
        const uint32_t idq = (uint32_t)__builtin_amdgcn_readlane((int)id, q);
        rank += (zq > z || (zq == z && idq < id)) ? 1 : 0;
    }
    const int to = lane < need ? rank : lane;   // a permutation of the lanes
    id = (uint32_t)__builtin_amdgcn_ds_permute(to * 4, (int)id);
    z = __int_as_float(__builtin_amdgcn_ds_permute(to * 4, __float_as_int(z)));
    ssq = __int_as_float(__builtin_amdgcn_ds_permute(to * 4, __float_as_int(ssq)));
    return ambiguous;
}

template <int NPL>
__device__ __forceinline__ PfRouteResult pf_route_fast_wave(const float *z_row, const float *ssq_row, int E, int K,
                                                            bool norm, int hidden, int lane) {
    float v[NPL], s2[NPL];
    bool bad = false;
    pf_load_row<NPL>(z_row, E, lane, -INFINITY, v);
    pf_load_row<NPL>(ssq_row, E, lane, 0.0f, s2);
#pragma unroll
    for (int j = 0; j < NPL; j++) bad |= lane * NPL + j < E && !pf_finite(v[j]);
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
    PfTopk<NPL> top;
    top.setup(v, E, lane);
    uint32_t my_key = 0;
    for (int r = 0; r <= rounds; r++) {   // one more than needed: see pf_topk_exact_order
        const uint32_t best = top.pop();
        if (lane == r) my_key = best;
    }
    PfRouteResult out;
    float my_z, my_s2;
    const bool ambiguous = pf_topk_exact_order<NPL>(my_key, rounds + 1, v, s2, lane, out.id, my_z, my_s2);
    pf_route_finish_wave(my_z, my_s2, K, rounds, norm, hidden, total, top_all, lane, out.weight, out.close);
    out.close |= ambiguous;
    out.bad = bad;
    return out;
}

// ---- several waves per token -------------------------------------------------------------
// Candidate lists in LDS: for each of `parts` waves, `rounds` entries sorted by (logit
// descending, id ascending); entry = sort key, logit, id, sum of squared products.  part_max
// and part_sum carry the pieces of the softmax denominator.  `first` receives the merged
// k + 1 best.
struct PfRouteCands {
    unsigned long long key[128];
    float z[128];
    uint32_t id[128];
    float s2[128];
    float first_z[16], first_s2[16];
    uint32_t first_id[16];
    float part_max[8], part_sum[8];
    uint32_t bad[8];
};

// Larger key = earlier in the order: the logit as an order-preserving integer (-0 counted as
// +0), then the lower id.  Equal logits among the k + 1 best always take the serial-order
// path, so the id part only makes the order total.
__device__ __forceinline__ unsigned long long pf_route_key(float z, uint32_t id) {
    uint32_t u = __float_as_uint(z + 0.0f);
    u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
    return ((unsigned long long)u << 32) | (uint32_t)~id;
}

// Stage 1 by ranking: every value's rank = how many of the chunk's values have a larger key.
// The other values come as wave-uniform operands (v_readlane), so one comparison and one
// carry-add per pair and no dependent chain across lanes.
template <int NPL>
__device__ __forceinline__ void pf_route_stage1(const float *z_row, const float *ssq_row, int E, int part, int chunk,
                                                int rounds, bool norm, PfRouteCands *c, int lane) {
    const int base = part * chunk, len = min(chunk, E - base);
    float v[NPL], s2[NPL];
    bool bad = false;
#pragma unroll
    for (int j = 0; j < NPL; j++) {
        const int i = lane * NPL + j;
        v[j] = i < len ? z_row[base + i] : -INFINITY;
        s2[j] = i < len ? ssq_row[base + i] : 0.0f;
        bad |= i < len && !pf_finite(v[j]);
    }
    bad = __any(bad);
    if (!norm) {
        float m = v[0], sum = 0.0f;
#pragma unroll
        for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
        m = pf_wave_max_fast(m);
#pragma unroll
        for (int j = 0; j < NPL; j++) sum += expf(v[j] - m);
        sum = pf_wave_sum(sum);
        if (lane == 0) { c->part_max[part] = m; c->part_sum[part] = sum; }
    }
    if (lane == 0) c->bad[part] = bad ? 1u : 0u;
    if (NPL == 1) {   // wider chunks keep the extraction below (the unrolled ranking would spill)
        unsigned long long key[NPL];
        uint32_t hi[NPL];
        int rank[NPL];
#pragma unroll
        for (int j = 0; j < NPL; j++) {
            key[j] = pf_route_key(v[j], (uint32_t)(base + lane * NPL + j));
            hi[j] = (uint32_t)(key[j] >> 32);
            rank[j] = 0;
        }
#pragma unroll
        for (int l = 0; l < PF_WAVE; l++) {
#pragma unroll
            for (int jj = 0; jj < NPL; jj++) {
                const unsigned long long other =
                    ((unsigned long long)(uint32_t)__builtin_amdgcn_readlane((int)hi[jj], l) << 32) |
                    (uint32_t)~(uint32_t)(base + l * NPL + jj);
#pragma unroll
                for (int j = 0; j < NPL; j++) rank[j] += other > key[j] ? 1 : 0;
            }
        }
#pragma unroll
        for (int j = 0; j < NPL; j++) {
            if (rank[j] < rounds) {
                const int at = part * rounds + rank[j];
                c->key[at] = key[j];
                c->z[at] = v[j];
                c->id[at] = v[j] == -INFINITY ? 0xffffffffu : (uint32_t)(base + lane * NPL + j);
                c->s2[at] = s2[j];
            }
        }
        return;
    }
    for (int r = 0; r < rounds; r++) {
        float wm;
        int owner, jsel;
        pf_extract_max<NPL>(v, lane, wm, owner, jsel);
        const int at = part * rounds + r;
        // the holder stores from its own registers: one predicated store per register, no
        // register array indexed by a run-time value
#pragma unroll
        for (int j = 0; j < NPL; j++) {
            if (lane == owner && j == jsel) {
                c->key[at] = pf_route_key(wm, (uint32_t)(base + lane * NPL + j));
                c->z[at] = wm;
                c->id[at] = wm == -INFINITY ? 0xffffffffu : (uint32_t)(base + lane * NPL + j);
                c->s2[at] = s2[j];
            }
        }
    }
}

// Merge by one wave, again by ranking: candidate p and p + 64 sit in lane p (at most 128
// candidates); the other candidates' keys are read from LDS at wave-uniform addresses.
__device__ __forceinline__ PfRouteResult pf_route_stage2(PfRouteCands *c, int parts, int K, int rounds, bool norm,
                                                         int hidden, int lane) {
    const int count = parts * rounds;
    const unsigned long long k0 = lane < count ? c->key[lane] : 0ull;
    const unsigned long long k1 = lane + 64 < count ? c->key[lane + 64] : 0ull;
    float total = 0.0f, top_all = 0.0f;
    bool bad = false;
    for (int w = 0; w < parts; w++) bad |= c->bad[w] != 0;
    if (!norm) {
        top_all = c->part_max[0];
        for (int w = 1; w < parts; w++) top_all = fmaxf(top_all, c->part_max[w]);
        for (int w = 0; w < parts; w++) total += c->part_sum[w] * expf(c->part_max[w] - top_all);
    }
    int r0 = 0, r1 = 0;
#pragma unroll 8
    for (int l = 0; l < count; l++) {
        const unsigned long long other = c->key[l];
        r0 += other > k0 ? 1 : 0;
        r1 += other > k1 ? 1 : 0;
    }
    if (lane < count && r0 < rounds) { c->first_z[r0] = c->z[lane]; c->first_id[r0] = c->id[lane]; c->first_s2[r0] = c->s2[lane]; }
    if (lane + 64 < count && r1 < rounds) {
        c->first_z[r1] = c->z[lane + 64]; c->first_id[r1] = c->id[lane + 64]; c->first_s2[r1] = c->s2[lane + 64];
    }
    pf_wave_lds_fence();
    const int at = lane < rounds ? lane : 0;
    const float my_z = c->first_z[at], my_s2 = c->first_s2[at];
    const uint32_t my_id = c->first_id[at];
    PfRouteResult out;
    pf_route_finish_wave(my_z, my_s2, K, rounds, norm, hidden, total, top_all, lane, out.weight, out.close);
    out.id = my_id;
    out.bad = bad;
    return out;
}
