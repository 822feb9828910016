// Re-routing of a token whose fast routing was flagged as close, by one wave (and one more that fetches ahead).
//
// The reference selects on probabilities from logits summed serially (src/qwen4_packed.c:164-179,
// src/qwen4_moe.c:219-247).  Only the order among the experts near the top k is in doubt, so only those
// are summed again in the reference's order:
//
//   candidates  every expert whose fast logit is within the token's largest noise tolerance of the
//               smallest of the k best fast logits.  An expert outside lies below k experts by more than
//               the tolerance, exactly summed too, and far enough for its probability to be strictly
//               smaller: it is not selected and ties with nobody selected.
//   exact part  a lane per candidate runs the serial sum; the maximum of the exact logits is the
//               reference's maximum (the largest logit is a candidate); p = expf(z - max) with the C
//               library's expf reproduced bit for bit.
//   order       by p descending, then id ascending.  The reference orders by fl(p / sum) with the same
//               tie rule; dividing by a common sum keeps the order of two p that differ by two ulps or
//               more strictly, and keeps equal p equal.  Two neighbours among the k + 1 first that are
//               closer than that without being equal need the sum itself: then, or with more than 64
//               candidates, or with probabilities near the subnormals, the wave routes the token the
//               long way (all logits serially, pf_route_exact_wave).
//
// Route weights need not be bit-exact: normalised ones are p / sum of the chosen p (the common sum
// cancels), the others p over the fast logits' softmax denominator.
#pragma once
#include "pf_device.h"
#include "pf_expf_libm.h"
#include "pf_route_device.h"
#include "pf_route_fast.h"

#define PF_FIX_BATCH 8   // 16-byte pieces of a router row per batch of the serial sum; AHEAD batches are on their way

// Serial sums of router rows, one per lane: row = this lane's row (H floats, any valid row for a lane whose result is
// not used), xs = the token's row in LDS, the same for every lane.  AHEAD (even) * 32 registers hold the row's pieces on
// their way; with XAHEAD the token's values are read from LDS a batch ahead into 2 * 32 registers more (read piece by
// piece as they are needed, the chain waits for an LDS round trip every second piece; read through the scalar cache a
// batch ahead, it waits for an L2 round trip every batch: both measured three times slower than the additions).
template <int AHEAD, bool XAHEAD>
__device__ __forceinline__ float pf_serial_logit_lanes(const float *row, const float *xs, int H) {
#pragma clang fp contract(off)
    static_assert(AHEAD % 2 == 0, "the two buffers of token values alternate with the batches");
    float sum = 0.0f;
    int done = 0;
    if (H % 4 == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
        // The row's pieces are requested AHEAD batches before their turn: the chain of additions never waits for
        // memory once the first batch has landed.  No load sits under a condition (a batch beyond the row reads the
        // row's last batch again and is not used): the loop body is straight-line code, which is what lets the
        // compiler wait for one batch and leave the younger ones on their way.
        const float4 *w4 = reinterpret_cast<const float4 *>(row), *x4 = reinterpret_cast<const float4 *>(xs);
        const int pieces = H / 4, batches = pieces / PF_FIX_BATCH, groups = batches / AHEAD;
        const int last = (batches > 0 ? batches - 1 : 0) * PF_FIX_BATCH;   // first piece of the last whole batch
        float4 ring[AHEAD][PF_FIX_BATCH], xa[PF_FIX_BATCH], xb[PF_FIX_BATCH];
        auto request = [&](float4 (&w)[PF_FIX_BATCH], int first) {   // one address per batch, the pieces at fixed offsets from it
            const float4 *src = w4 + min(first, last);
#pragma unroll
            for (int j = 0; j < PF_FIX_BATCH; j++) w[j] = src[j];
        };
        auto request_x = [&](float4 (&x)[PF_FIX_BATCH], int first) {
            const float4 *src = x4 + min(first, last);
#pragma unroll
            for (int j = 0; j < PF_FIX_BATCH; j++) x[j] = src[j];
        };
        // The chain is the additions alone (4 ns each for a wave alone on its SIMD): a piece's products are formed
        // one by one between the additions of the piece before it, where the chain would wait anyway (left to itself
        // the compiler forms each product right before its addition, through one register: two dependent operations
        // a step; all four products ahead of the four additions: 5.4 ns a step).
        auto batch = [&](const float4 (&w)[PF_FIX_BATCH], const float4 (&x)[PF_FIX_BATCH]) {
            float p0 = w[0].x * x[0].x, p1 = w[0].y * x[0].y, p2 = w[0].z * x[0].z, p3 = w[0].w * x[0].w;
#pragma unroll
            for (int j = 0; j < PF_FIX_BATCH; j++) {
                const int n = j + 1 < PF_FIX_BATCH ? j + 1 : j;   // the last piece forms its own products again, unused
                __builtin_amdgcn_sched_barrier(0);
                sum = sum + p0;
                __builtin_amdgcn_sched_barrier(0);
                const float n0 = w[n].x * x[n].x;
                __builtin_amdgcn_sched_barrier(0);
                sum = sum + p1;
                __builtin_amdgcn_sched_barrier(0);
                const float n1 = w[n].y * x[n].y;
                __builtin_amdgcn_sched_barrier(0);
                sum = sum + p2;
                __builtin_amdgcn_sched_barrier(0);
                const float n2 = w[n].z * x[n].z;
                __builtin_amdgcn_sched_barrier(0);
                sum = sum + p3;
                __builtin_amdgcn_sched_barrier(0);
                const float n3 = w[n].w * x[n].w;
                __builtin_amdgcn_sched_barrier(0);
                p0 = n0; p1 = n1; p2 = n2; p3 = n3;
            }
        };
        auto step = [&](int r, int first) {   // batch `first` from ring slot r; r's parity names the buffer its token values are in
            if (XAHEAD) {
                if (r % 2 == 0) { request_x(xb, first + PF_FIX_BATCH); batch(ring[r], xa); }
                else { request_x(xa, first + PF_FIX_BATCH); batch(ring[r], xb); }
            } else {
                request_x(xa, first);
                batch(ring[r], xa);
            }
        };
        if (batches > 0) {
#pragma unroll
            for (int r = 0; r < AHEAD; r++) request(ring[r], r * PF_FIX_BATCH);
            if (XAHEAD) request_x(xa, 0);
        }
        for (int g = 0; g < groups; g++) {
#pragma unroll
            for (int r = 0; r < AHEAD; r++) {
                const int first = (g * AHEAD + r) * PF_FIX_BATCH;
                step(r, first);
                request(ring[r], first + AHEAD * PF_FIX_BATCH);
            }
        }
#pragma unroll
        for (int r = 0; r < AHEAD; r++)   // the batches of the last, partial group are in the ring already
            if (groups * AHEAD + r < batches) step(r, (groups * AHEAD + r) * PF_FIX_BATCH);
        done = batches * PF_FIX_BATCH * 4;
    }
    for (int k = done; k < H; k++) {   // rows of other widths or alignments, and what is left of a row beyond whole batches
        const float p = row[k] * xs[k];
        sum = sum + p;
    }
    return sum;
}

// LDS the workgroup needs: the token's row (H floats), then 3 E floats (the long way's arrays; meanwhile the
// candidates' ids sit in the first 64 words of them and their count in the first word of the third array).
__host__ __device__ constexpr size_t pf_route_fix_lds_floats(int H, int E) { return (size_t)H + 3 * (size_t)(E > 64 ? E : 64); }

// Called by every wave of the workgroup (two workgroup barriers inside); E <= 64 NPL, K < 63.  Wave 0 routes; wave 1,
// where the workgroup has one, touches every 128-byte line of the candidates' router rows as soon as they are known,
// so that the serial sums, which keep only AHEAD lines a lane on their way, find them in the L2.  router: [E][H] f32
// as the file stores it; x_row: the token's row; z_row, ssq_row: the token's fast logits and their noise terms.
// ids_out / w_out: K entries each (LDS or global), written by wave 0.  Returns, in wave 0, 1 when the candidates
// settled it and 2 when the token went the long way.
template <int NPL, int AHEAD, bool XAHEAD>
__device__ __forceinline__ int pf_route_fix_block(const float *router, const float *x_row, const float *z_row, const float *ssq_row,
                                                  int E, int K, bool norm, int H, float *lds, uint32_t *ids_out, float *w_out,
                                                  int wave, int lane) {
#pragma clang fp contract(off)
    const int wide = E > 64 ? E : 64;
    float *xs = lds, *z = lds + H, *p = z + wide, *q = p + wide;
    uint32_t *cand = reinterpret_cast<uint32_t *>(z), *shared_count = reinterpret_cast<uint32_t *>(q);
    const int picks = K < E ? K : E;
    float v[NPL], s2[NPL];
    int count = 0;
    {   // the token's row into LDS: by the other waves where there are any, all pieces requested before the first is stored
        const int helpers = (int)blockDim.x > PF_WAVE ? (int)blockDim.x - PF_WAVE : PF_WAVE;
        const int me = (int)blockDim.x > PF_WAVE ? (int)threadIdx.x - PF_WAVE : lane;
        if (me >= 0 && H % 4 == 0 && (reinterpret_cast<uintptr_t>(x_row) & 15) == 0) {
            const float4 *src = reinterpret_cast<const float4 *>(x_row);
            for (int i0 = me; i0 < H / 4; i0 += 8 * helpers) {
                float4 held[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    held[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    if (i0 + j * helpers < H / 4) held[j] = src[i0 + j * helpers];
                }
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (i0 + j * helpers < H / 4) reinterpret_cast<float4 *>(xs)[i0 + j * helpers] = held[j];
            }
        } else if (me >= 0) {
            for (int k = me; k < H; k += helpers) xs[k] = x_row[k];
        }
    }
    if (wave == 0) {
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
        const bool hopeless = !(best_z - floor_z < 80.0f) || !pf_finite(best_z) || !pf_finite(kth);
        // the candidates into lanes: position = candidates of lower registers, then of lower lanes in this register
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
        if (lane == 0) *shared_count = (uint32_t)count;   // 0: the long way
    }
    __syncthreads();
    int how = 0;
    if (wave == 1) {
        const int n = (int)*shared_count, lines = (H + 31) / 32;
        uint32_t sink = 0;
        for (int i0 = lane; i0 < n * lines; i0 += 16 * PF_WAVE) {   // line-major: the rows' first lines first
            uint32_t got[16];   // sixteen loads a lane on their way before the first is looked at
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int i = i0 + j * PF_WAVE;
                got[j] = 0u;
                if (i < n * lines) got[j] = __float_as_uint(router[(size_t)cand[i % n] * H + (i / n) * 32]);
            }
#pragma unroll
            for (int j = 0; j < 16; j++) sink ^= got[j];
        }
        if (sink == 0x7fc54321u) shared_count[1] = sink;   // keeps the loads alive; the word is never read
    } else if (wave == 0) {
        bool long_way = count == 0;
        if (!long_way) {
            const bool active = lane < count;
            const uint32_t id = active ? cand[lane] : 0xffffffffu;
            const float zc = pf_serial_logit_lanes<AHEAD, XAHEAD>(router + (size_t)(active ? id : 0u) * H, xs, H);
            const float zmax = pf_wave_max(active ? zc : -INFINITY);
            float shifted = zc - zmax;
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
            // neighbours among the first k + 1: equal, or apart by more than the division can close; nothing near the subnormals
            const float next = __shfl_down(sp, 1);
            const bool paired = lane < picks && lane + 1 < count;
            const bool doubtful = (paired && !(sp == next || sp - next > 1e-6f * sp)) || (lane < picks && !(sp > 1e-30f)) ||
                                  (paired && !(next > 1e-30f));
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
                how = 1;
            }
        }
        if (long_way) {   // every logit in serial order, then the reference's routing step by step
            pf_wave_lds_fence();
            for (int e0 = 0; e0 < E; e0 += PF_WAVE) {
                const int e = e0 + lane;
                const float ze = pf_serial_logit_lanes<AHEAD, XAHEAD>(router + (size_t)(e < E ? e : 0) * H, xs, H);
                if (e < E) z[e] = ze;
            }
            pf_wave_lds_fence();
            pf_route_exact_wave(z, p, q, E, K, norm, ids_out, w_out, lane);
            how = 2;
        }
    }
    __syncthreads();
    return how;
}
