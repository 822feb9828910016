// Re-routing of a token whose fast routing was flagged as close, by the waves of one workgroup.
//
// The reference selects on probabilities from logits summed serially (src/qwen4_packed.c:164-179,
// src/qwen4_moe.c:219-247).  Only the order among the experts near the top k is in doubt, so only those
// are summed again in the reference's order:
//
//   candidates  every expert whose fast logit is within the token's largest noise tolerance of the
//               smallest of the k best fast logits.  An expert outside lies below k experts by more than
//               the tolerance, exactly summed too, and far enough for its probability to be strictly
//               smaller: it is not selected and ties with nobody selected.
//   exact part  a lane per candidate runs the serial sum (below); the maximum of the exact logits is the
//               reference's maximum (the largest logit is a candidate); p = expf(z - max) with the C
//               library's expf reproduced bit for bit.
//   order       by p descending, then id ascending.  The reference orders by fl(p / sum) with the same
//               tie rule.  Two p four ulps or more apart give quotients that round to different values,
//               equal p stay equal, and closer p can only tie, which goes to the lower id: no change
//               when the larger p has the lower id already.  Two neighbours among the k + 1 first that
//               are fewer than four ulps apart, not equal, with the larger p on the higher id need the
//               sum itself: then, or with more than 64 candidates, or with probabilities near the
//               subnormals, the workgroup routes the token the long way (all logits serially, 64 experts
//               a pass through the same chains, then pf_route_exact_wave).
//
// Route weights need not be bit-exact: normalised ones are p / sum of the chosen p (the common sum
// cancels), the others p over the fast logits' softmax denominator.
#pragma once
#include "pf_device.h"
#include "pf_expf_libm.h"
#include "pf_route_device.h"
#include "pf_route_fast.h"

// The serial sums.  A sum is one chain of dependent additions, k ascending, and the chains of different experts are
// independent, so one wave runs them all, a lane per candidate: one vector instruction a step whatever the number of
// candidates.  (A wave per candidate, with the lanes forming the products side by side and the chain fetching them
// back through v_readlane, costs two instructions a step for a single chain: ten candidates on four SIMDs took 30 us.)
// What the chain must never do is wait for memory, and a lane reading its own row keeps too little on its way (two to
// five 128-byte lines a lane: 22-28 us).  So the other waves of the workgroup bring the candidates' rows in with
// coalesced loads, multiply them by the token's values and leave the products in LDS, a chunk of every row at a time,
// one chunk ahead of the chain (PF_FIX_CHUNK_FLOATS floats of LDS per buffer: chunks of 512 values for up to 16
// candidates, 256 up to 32, 128 up to 64), and the chain reads LDS four pieces ahead.  (With the multiplications in the
// chain's own wave, two instructions a step, 2048 values took 8 us.)
#define PF_FIX_CHUNK_FLOATS 8448   // 16 rows of 512 + 4 (or 32 of 256 + 4, or 64 of 128 + 4) floats, rounded up

// The chain over one chunk: p = this lane's row of the chunk's PRODUCTS in LDS (each w[k] * x[k] rounded, formed by the
// waves that brought the row), pieces = 16-byte pieces in the chunk.  The chain is additions only, one vector instruction
// a step; the LDS reads run a batch of four pieces ahead.
__device__ __forceinline__ float pf_serial_chunk(float sum, const float *p, int pieces) {
#pragma clang fp contract(off)
    const float4 *p4 = reinterpret_cast<const float4 *>(p);
    float4 a[4], b[4];
    auto fetch = [&](float4 (&v)[4], int first) {   // beyond the chunk: its last batch again, not used
        const int at = min(first, pieces - 4);
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = p4[at + j];
    };
    auto batch = [&](const float4 (&v)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            __builtin_amdgcn_sched_barrier(0);
            sum = sum + v[j].x;
            sum = sum + v[j].y;
            sum = sum + v[j].z;
            sum = sum + v[j].w;
        }
    };
    const int whole = pieces / 8 * 8;
    if (whole > 0) {
        fetch(a, 0);
        for (int q = 0; q < whole; q += 8) {
            fetch(b, q + 4);
            batch(a);
            fetch(a, q + 8);
            batch(b);
        }
    }
    for (int j = whole; j < pieces; j++) {   // a last chunk that is not whole batches
        const float4 v = p4[j];
        sum = sum + v.x;
        sum = sum + v.y;
        sum = sum + v.z;
        sum = sum + v.w;
    }
    return sum;
}

// LDS the workgroup needs: the candidates' ids (64 words), four words of hand-over, the token's row (H floats), then
// the two chunk buffers and the long way's 3 E floats.
__host__ __device__ constexpr size_t pf_route_fix_lds_floats(int H, int E) { return 68 + (size_t)H + 2 * PF_FIX_CHUNK_FLOATS + 3 * (size_t)E; }

// Called by every wave of a workgroup of at least two waves (workgroup barriers inside); E <= 64 NPL, K < 63.
// Wave 0 picks the candidates and runs their sums, the others feed it.  router: [E][H] f32 as the file stores it;
// x_row: the token's row; z_row, ssq_row: the token's fast logits and their noise terms.  ids_out / w_out: K entries
// each (LDS or global), written by wave 0.  Returns, in every wave, 1 when the candidates settled it and 2 when the
// token went the long way.
template <int NPL>
__device__ __forceinline__ int pf_route_fix_block(const float *router, const float *x_row, const float *z_row, const float *ssq_row,
                                                  int E, int K, bool norm, int H, float *lds, uint32_t *ids_out, float *w_out,
                                                  int wave, int lane) {
#pragma clang fp contract(off)
    uint32_t *cand = reinterpret_cast<uint32_t *>(lds), *hand = cand + 64;   // hand[0]: candidates (0: the long way), hand[1]: outcome
    float *xs = lds + 68, *stage = xs + H, *z = stage + 2 * PF_FIX_CHUNK_FLOATS, *p = z + E, *q = p + E;
    const int picks = K < E ? K : E;
    const int helpers = (int)blockDim.x - PF_WAVE, me = (int)threadIdx.x - PF_WAVE;   // the waves after the first
    float v[NPL];
    int count = 0;
    for (int k = me; k >= 0 && k < H; k += helpers) xs[k] = x_row[k];
    if (wave == 0) {
        float s2[NPL];
        pf_load_row<NPL>(z_row, E, lane, -INFINITY, v);
        pf_load_row<NPL>(ssq_row, E, lane, 0.0f, s2);
        // the k best fast logits: their smallest, the largest, and the largest noise term of the token
        PfTopk<NPL> top;
        top.setup(v, E, lane);
        uint32_t my_key = 0;
        for (int r = 0; r < picks; r++) {
            const uint32_t best = top.pop();
            if (lane == r) my_key = best;
        }
        float mine = INFINITY, best_z = -INFINITY, worst_s2 = 0.0f;
        const bool have = lane < picks && my_key != 0u;
        const int at = have ? (int)pf_key_id(my_key) : 0;
#pragma unroll
        for (int j = 0; j < NPL; j++) {
            const float vz = __shfl(v[j], at / NPL);
            if (have && at % NPL == j) mine = vz;
            best_z = fmaxf(best_z, v[j]);
            worst_s2 = fmaxf(worst_s2, s2[j]);
        }
        const float kth = -pf_wave_max(-mine);   // the smallest of the k best (as extracted: a lower value only adds candidates)
        best_z = pf_wave_max(best_z);
        worst_s2 = pf_wave_max(worst_s2);
        const float u = 5.9604645e-8f, hk = (float)H / 6.0f;
        const float tol = 16.0f * u * sqrtf(hk * worst_s2) + 4e-6f * fmaxf(1.0f, best_z - kth + 1.0f);
        const float floor_z = kth - tol;
        // rows the chunk loads cannot take in 16-byte pieces go the long way, as do logits beyond exp's range
        const bool hopeless = !(best_z - floor_z < 80.0f) || !pf_finite(best_z) || !pf_finite(kth) || H % 4 != 0 ||
                              (reinterpret_cast<uintptr_t>(router) & 15) != 0;
        // the candidates into a list: position = candidates of lower registers, then of lower lanes in this register
        if (!hopeless) {
            const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
            for (int j = 0; j < NPL; j++) {
                const bool in = lane * NPL + j < E && v[j] >= floor_z;
                const unsigned long long m = __ballot(in);
                const int to = count + __popcll(m & below);
                if (in && to < PF_WAVE) cand[to] = (uint32_t)(lane * NPL + j);
                count += __popcll(m);
            }
            if (count > PF_WAVE || count < picks) count = 0;
        }
        if (lane == 0) hand[0] = (uint32_t)count;
    }
    __syncthreads();
    // Serial sums of n router rows, lane r of wave 0 the r-th: the listed candidates (base < 0) or rows base .. base + n.
    // Every wave calls it (workgroup barriers inside).
    auto staged_sums = [&](int n, int base) -> float {
        float sum = 0.0f;
        const int rows = n <= 16 ? 16 : n <= 32 ? 32 : 64, chunk = 8192 / rows, pitch = chunk + 4;
        const int chunks = (H + chunk - 1) / chunk;
        auto bring = [&](int c) {   // chunk c of every row into its buffer, by the waves after the first
            const int first = c * chunk, pieces = min(chunk, H - first) / 4, total = n * pieces;
            float *buf = stage + (c & 1) * PF_FIX_CHUNK_FLOATS;
            for (int i0 = me; i0 >= 0 && i0 < total; i0 += 4 * helpers) {
                float4 held[4];
                int row[4], piece[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int i = min(i0 + j * helpers, total - 1);
                    row[j] = i / pieces; piece[j] = i - row[j] * pieces;
                    const size_t expert = base < 0 ? cand[row[j]] : (uint32_t)(base + row[j]);
                    held[j] = reinterpret_cast<const float4 *>(router + expert * H + first)[piece[j]];
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {   // the products, each rounded once, as the reference forms them before it adds
                    if (i0 + j * helpers < total) {
                        const float4 xv = reinterpret_cast<const float4 *>(xs + first)[piece[j]];
                        reinterpret_cast<float4 *>(buf + row[j] * pitch)[piece[j]] =
                            float4{held[j].x * xv.x, held[j].y * xv.y, held[j].z * xv.z, held[j].w * xv.w};
                    }
                }
            }
        };
        bring(0);
        __syncthreads();
        for (int c = 0; c < chunks; c++) {
            if (wave != 0) {
                if (c + 1 < chunks) bring(c + 1);
            } else {   // lanes beyond the rows sum the last row again, unused
                const int first = c * chunk, pieces = min(chunk, H - first) / 4;
                sum = pf_serial_chunk(sum, stage + (c & 1) * PF_FIX_CHUNK_FLOATS + min(lane, n - 1) * pitch, pieces);
            }
            __syncthreads();
        }
        return sum;
    };
    const int n = (int)hand[0];
    float zc = 0.0f;
    if (n > 0) zc = staged_sums(n, -1);
    if (wave == 0) {
        bool long_way = n == 0;
        if (!long_way) {
            const bool active = lane < count;
            const uint32_t id = active ? cand[lane] : 0xffffffffu;
            const float mine = active ? zc : -INFINITY;
            const float zmax = pf_wave_max(mine);
            float shifted = mine - zmax;
            const float pc = active ? pf_expf_libm(shifted) : -1.0f;
            // rank by (p descending, id ascending)
            int rank = 0;
            for (int c = 0; c < count; c++) {
                const float po = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pc), c));
                const uint32_t io = (uint32_t)__builtin_amdgcn_readlane((int)id, c);
                rank += (po > pc || (po == pc && io < id)) ? 1 : 0;
            }
            const int to = active ? rank : lane;   // a permutation of the lanes
            const uint32_t sid = (uint32_t)__builtin_amdgcn_ds_permute(to * 4, (int)id);
            const float sp = __int_as_float(__builtin_amdgcn_ds_permute(to * 4, __float_as_int(pc)));
            // Neighbours among the first k + 1.  The reference orders by fl(p / sum): two p that are four ulps or more
            // apart give quotients more than one ulp apart, which round to different values; closer p may tie after the
            // division, and a tie goes to the lower id: that changes nothing when the larger p has the lower id already.
            // So the doubt is a pair fewer than four ulps apart, not equal, whose larger p has the higher id; and
            // nothing may be near the subnormals.
            const float next = __shfl_down(sp, 1);
            const uint32_t next_id = (uint32_t)__shfl_down((int)sid, 1);
            const bool paired = lane < picks && lane + 1 < count;
            const bool near = sp != next && __float_as_uint(sp) - __float_as_uint(next) < 4u;
            const bool doubtful = (paired && near && sid > next_id) || (lane < picks && !(sp > 1e-30f)) || (paired && !(next > 1e-30f));
            long_way = __any(doubtful);
            if (!long_way) {
                const float chosen = pf_wave_sum(lane < picks ? sp : 0.0f);
                float weight;
                if (norm) {
                    weight = sp / chosen;
                } else {   // the softmax denominator from the fast logits (weights are compared within a tolerance)
                    float total = 0.0f;
#pragma unroll
                    for (int j = 0; j < NPL; j++) total += lane * NPL + j < E ? expf(v[j] - zmax) : 0.0f;
                    total = pf_wave_sum(total);
                    weight = sp / total;
                }
                if (lane < picks) { ids_out[lane] = sid; w_out[lane] = weight; }
            }
        }
        if (lane == 0) hand[1] = long_way ? 2u : 1u;
    }
    __syncthreads();
    const int how = (int)hand[1];
    if (how == 2) {   // every logit in serial order, 64 experts a pass, then the reference's routing step by step
        if (H % 4 == 0 && (reinterpret_cast<uintptr_t>(router) & 15) == 0) {
            for (int e0 = 0; e0 < E; e0 += PF_WAVE) {
                const int rows = min(PF_WAVE, E - e0);
                const float ze = staged_sums(rows, e0);
                if (wave == 0 && lane < rows) z[e0 + lane] = ze;
            }
        } else {   // rows that cannot be fetched in 16-byte pieces: a thread per expert
            for (int e = threadIdx.x; e < E; e += blockDim.x) z[e] = pf_serial_logit(router + (size_t)e * H, xs, H);
        }
        __syncthreads();
        if (wave == 0) pf_route_exact_wave(z, p, q, E, K, norm, ids_out, w_out, lane);
    }
    __syncthreads();
    return how;
}
