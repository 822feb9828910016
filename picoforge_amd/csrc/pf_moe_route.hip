// Routing (softmax, top-k, renormalisation) and expert grouping kernels.
//
// Two routing paths exist.  The fast one keeps a token's logits in the registers
// of one wave and selects in logit space.  It also measures how close the k+1
// best logits are; when two of them are closer than the rounding noise a
// differently ordered logit sum could have, the token is routed again by the
// exact path, which recomputes its logits in the reference's serial order
// (src/qwen4_packed.c:164-179) and follows src/qwen4_moe.c:219-247 step by step.
#include "pf_moe_internal.h"
#include "pf_route_device.h"
#include "pf_route_fast.h"

#define ROUTE_MAX_FAST_EXPERTS 1024

// ---- fast routing inside a forward (general path) --------------------------------
template <int NPL>
__global__ void __launch_bounds__(64) pf_k_route_fast(PfKernelArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x, E = a.experts, K = a.top_k;
    PfRouteResult r = pf_route_fast_wave<NPL>(a.logits + (size_t)t * E, a.logit_ssq + (size_t)t * E, E, K,
                                              a.norm_topk != 0, a.hidden, lane);
    if (r.bad && lane == 0) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    if (lane < K) {
        a.ids[(size_t)t * K + lane] = r.id;
        a.route_weights[(size_t)t * K + lane] = r.weight;
    }
    if (lane == 0) a.route_flags[t] = r.close ? 1u : 0u;
}

// Serial-order recomputation for flagged tokens, in two kernels so that a token's logits
// spread over many compute units: one wave per (token, slab of 64 experts), lane e owns expert e
// and the sum runs over k in order, as the reference's.  The router copy is laid out for this,
// [slab][hidden / 4][64 experts][4 consecutive k]: four steps of a wave are one 1 KB load at a
// uniform base plus the lane's offset, and the token's values are scalar operands.  The sum is
// one dependent chain; the loads are not: they are requested well ahead of the chain (a wave can
// have 63 of them on their way, 252 steps).
__global__ void __launch_bounds__(64) pf_k_route_fix_logits(PfKernelArgs a) {
#pragma clang fp contract(off)
    const int t = blockIdx.x, E = a.experts, H = a.hidden, lane = threadIdx.x;
    const int e = blockIdx.y * PF_WAVE + lane;
    if (!a.route_flags[t]) return;
    const float *__restrict__ xs = a.x + (size_t)t * a.x_pitch;
    const float4 *__restrict__ w = reinterpret_cast<const float4 *>(a.router_t) + (size_t)blockIdx.y * ((H + 3) / 4) * PF_WAVE + lane;
    float sum = 0.0f;
    float4 w0[16], w1[16], w2[16];
    const int batches = H / 64;   // 64 steps = 16 loads
    auto load = [&](float4 (&dst)[16], int b) {
        if (b >= batches) return;
        const float4 *row = w + (size_t)(16 * b) * PF_WAVE;
#pragma unroll
        for (int j = 0; j < 16; j++) dst[j] = row[j * PF_WAVE];
    };
    auto chain = [&](const float4 (&src)[16], int b) {
        if (b >= batches) return;
        const float *x = xs + 64 * b;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const float p0 = src[j].x * x[4 * j];
            sum = sum + p0;
            const float p1 = src[j].y * x[4 * j + 1];
            sum = sum + p1;
            const float p2 = src[j].z * x[4 * j + 2];
            sum = sum + p2;
            const float p3 = src[j].w * x[4 * j + 3];
            sum = sum + p3;
        }
    };
    // three batches rotate: two are on their way while one is summed
    load(w0, 0);
    load(w1, 1);
    for (int b = 0; b < batches; b += 3) {
        load(w2, b + 2);
        chain(w0, b);
        load(w0, b + 3);
        chain(w1, b + 1);
        load(w1, b + 4);
        chain(w2, b + 2);
    }
    const float *tail = reinterpret_cast<const float *>(w);
    for (int k = 64 * batches; k < H; k++) {   // the lane's k-quad at 256 (k / 4) floats
        const float p = tail[(size_t)(k / 4) * 4 * PF_WAVE + (k & 3)] * xs[k];
        sum = sum + p;
    }
    if (e < E) a.logits[(size_t)t * E + e] = sum;
}

// router [experts][hidden] -> [slab][ceil(hidden / 4)][64][4] (expert 64 * slab + lane, four
// consecutive columns together; zeros beyond the last expert and the last column), once at upload
size_t pf_router_slab_floats(int experts, int hidden) {
    return (size_t)((experts + PF_WAVE - 1) / PF_WAVE) * ((hidden + 3) / 4) * 4 * PF_WAVE;
}

__global__ void pf_k_router_slabs(const float *src, int experts, int hidden, float *dst, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t quads = (size_t)(hidden + 3) / 4;
    const int c = (int)(i & 3), lane = (int)((i >> 2) % PF_WAVE);
    const size_t quad = (i / (4 * PF_WAVE)) % quads, slab = i / (4 * PF_WAVE * quads);
    const size_t e = slab * PF_WAVE + lane, k = 4 * quad + c;
    dst[i] = (e < (size_t)experts && k < (size_t)hidden) ? src[e * hidden + k] : 0.0f;
}

void pf_launch_router_slabs(const float *d_src, int experts, int hidden, float *d_dst, hipStream_t stream) {
    const size_t total = pf_router_slab_floats(experts, hidden);
    hipLaunchKernelGGL(pf_k_router_slabs, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, d_src, experts, hidden,
                       d_dst, total);
}

__global__ void __launch_bounds__(64) pf_k_route_fix_select(PfKernelArgs a) {
    extern __shared__ float lds[];
    const int t = blockIdx.x, E = a.experts;
    if (!a.route_flags[t]) return;
    float *z = lds, *p = z + E, *q = p + E;
    for (int e = threadIdx.x; e < E; e += PF_WAVE) z[e] = a.logits[(size_t)t * E + e];
    pf_wave_lds_fence();
    pf_route_exact_wave(z, p, q, E, a.top_k, a.norm_topk != 0, a.ids + (size_t)t * a.top_k,
                        a.route_weights + (size_t)t * a.top_k, threadIdx.x);
    if (threadIdx.x == 0) atomicAdd(a.exact_rows, 1u);
}

// Every token through the exact path (expert counts the fast kernel cannot hold).
__global__ void pf_k_flag_all(uint32_t *flags, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) flags[i] = 1u;
}

void pf_launch_route(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    const int npl = (a.experts + PF_WAVE - 1) / PF_WAVE;
    if (a.experts > ROUTE_MAX_FAST_EXPERTS || a.top_k >= PF_WAVE)
        hipLaunchKernelGGL(pf_k_flag_all, dim3((tokens + 255) / 256), dim3(256), 0, stream, a.route_flags, tokens);
    else if (npl <= 1) hipLaunchKernelGGL(pf_k_route_fast<1>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 2) hipLaunchKernelGGL(pf_k_route_fast<2>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 4) hipLaunchKernelGGL(pf_k_route_fast<4>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 8) hipLaunchKernelGGL(pf_k_route_fast<8>, dim3(tokens), dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(pf_k_route_fast<16>, dim3(tokens), dim3(64), 0, stream, a);
    hipLaunchKernelGGL(pf_k_route_fix_logits, dim3(tokens, (a.experts + PF_WAVE - 1) / PF_WAVE), dim3(PF_WAVE), 0, stream, a);
    hipLaunchKernelGGL(pf_k_route_fix_select, dim3(tokens), dim3(PF_WAVE), 3 * (size_t)a.experts * sizeof(float), stream,
                       a);
}

// ---- qwen4_moe_route on caller-provided logits ----------------------------------
__global__ void pf_k_logits_finite(const float *z, size_t n, int experts, uint32_t *error, unsigned long long *bad_row) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && !pf_finite(z[i])) {
        atomicOr(error, PF_HIP_ERR_NONFINITE);
        atomicMin(bad_row, (unsigned long long)(i / experts));
    }
}

__global__ void __launch_bounds__(64) pf_k_route_exact(const float *logits, int E, int K, int norm, float *probs,
                                                       uint32_t *ids, float *weights) {
    extern __shared__ float lds[];
    const int t = blockIdx.x, lane = threadIdx.x;
    float *z = lds, *p = z + E, *q = p + E;
    for (int e = lane; e < E; e += PF_WAVE) z[e] = logits[(size_t)t * E + e];
    pf_wave_lds_fence();
    pf_route_exact_wave(z, p, q, E, K, norm != 0, ids + (size_t)t * K, weights + (size_t)t * K, lane);
    for (int e = lane; e < E; e += PF_WAVE) probs[(size_t)t * E + e] = p[e];
}

int pf_route_exact_device(const float *d_logits, int tokens, int experts, int top_k, int norm, float *d_probs,
                          uint32_t *d_ids, float *d_weights, uint32_t *d_error, unsigned long long *d_bad_row,
                          hipStream_t stream) {
    const size_t n = (size_t)tokens * experts;
    if (n == 0) return PF_HIP_OK;
    hipLaunchKernelGGL(pf_k_logits_finite, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, d_logits, n,
                       experts, d_error, d_bad_row);
    uint32_t err = 0;
    if (hipMemcpyAsync(&err, d_error, 4, hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
        return PF_HIP_E_RUNTIME;
    if (err) return PF_HIP_OK;   // caller reads the error word; nothing was written
    const size_t lds = 3 * (size_t)experts * sizeof(float);
    if (lds > 64 * 1024) return PF_HIP_E_UNSUPPORTED;
    hipLaunchKernelGGL(pf_k_route_exact, dim3(tokens), dim3(64), lds, stream, d_logits, experts, top_k, norm,
                       d_probs, d_ids, d_weights);
    return hipGetLastError() == hipSuccess ? PF_HIP_OK : PF_HIP_E_RUNTIME;
}

__global__ void pf_k_fill_u32(uint32_t *p, int n, uint32_t value) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

// ---- grouping: stable counting sort of (token, slot) pairs by expert ------------
// first_bad = min over offending (token, slot) of 2 * pair + kind, kind 0 = id out
// of range, 1 = id repeated within the token: the error a scan in pair order
// meets first (src/qwen4_moe.c:277-284)
__global__ void pf_k_group_check(const uint32_t *ids, int tokens, int E, int K, uint32_t *first_bad) {
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    const uint32_t *row = ids + (size_t)t * K;
    for (int s = 0; s < K; s++) {
        const uint32_t pair = (uint32_t)(t * K + s);
        if (row[s] >= (uint32_t)E) { atomicMin(first_bad, 2u * pair); return; }
        for (int j = 0; j < s; j++)
            if (row[j] == row[s]) { atomicMin(first_bad, 2u * pair + 1u); return; }
    }
}

__global__ void pf_k_group_count(const uint32_t *ids, int pairs, int E, uint32_t *counts) {
    int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p < pairs && ids[p] < (uint32_t)E) atomicAdd(&counts[ids[p]], 1u);
}

// one block: exclusive scan of counts[E] into offsets[E+1]
__global__ void __launch_bounds__(256) pf_k_group_scan(const uint32_t *counts, int E, uint32_t *offsets) {
    __shared__ uint32_t part[256];
    const int tid = threadIdx.x, per = (E + 255) / 256, lo = tid * per, hi = min(E, lo + per);
    uint32_t s = 0;
    for (int e = lo; e < hi; e++) s += counts[e];
    part[tid] = s;
    __syncthreads();
    if (tid == 0) {
        uint32_t run = 0;
        for (int i = 0; i < 256; i++) { uint32_t v = part[i]; part[i] = run; run += v; }
        offsets[E] = run;
    }
    __syncthreads();
    uint32_t run = part[tid];
    for (int e = lo; e < hi; e++) { offsets[e] = run; run += counts[e]; }
}

// one wave per expert walks the pairs in order: rank = earlier pairs of the
// same expert, so placement is stable without ordered atomics.  The ids pass through LDS in
// pieces; a lane looks at four consecutive pairs per step (one 16-byte LDS read), two steps'
// reads are requested together.
#define PLACE_PIECE 8192
__global__ void __launch_bounds__(256) pf_k_group_place(const uint32_t *ids, int pairs, int E, const uint32_t *offsets,
                                                        uint32_t *pair_to_row, uint32_t *row_to_pair) {
    __shared__ __align__(16) uint32_t staged[PLACE_PIECE];
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = pf_lane();
    const bool active = e < E && offsets[min(e, E - 1) + 1] != offsets[min(e, E - 1)];
    uint32_t base = e < E ? offsets[e] : 0u;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int piece = 0; piece < pairs; piece += PLACE_PIECE) {
        const int len = min(PLACE_PIECE, pairs - piece), padded = (len + 511) & ~511;
        __syncthreads();
        // all of a thread's loads are requested before the first is stored (the piece starts on a
        // 16-byte boundary of ids; its ragged end is read id by id)
        uint4 held[PLACE_PIECE / 4 / 256];
#pragma unroll
        for (int j = 0; j < PLACE_PIECE / 4 / 256; j++) {
            const int i = 4 * ((int)threadIdx.x + 256 * j);
            uint4 v = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
            if (i + 4 <= len) {
                v = *reinterpret_cast<const uint4 *>(ids + piece + i);
            } else if (i < len) {
                v.x = ids[piece + i];
                if (i + 1 < len) v.y = ids[piece + i + 1];
                if (i + 2 < len) v.z = ids[piece + i + 2];
            }
            held[j] = v;
        }
#pragma unroll
        for (int j = 0; j < PLACE_PIECE / 4 / 256; j++) {
            const int i = 4 * ((int)threadIdx.x + 256 * j);
            if (i < padded) *reinterpret_cast<uint4 *>(staged + i) = held[j];
        }
        __syncthreads();
        if (!active) continue;
        // step: 256 pairs, lane l holds pairs 4l .. 4l + 3 of it
        auto place = [&](const uint4 &v, int p0) {
            const bool h0 = v.x == (uint32_t)e, h1 = v.y == (uint32_t)e, h2 = v.z == (uint32_t)e, h3 = v.w == (uint32_t)e;
            const int mine = (int)h0 + (int)h1 + (int)h2 + (int)h3;
            const unsigned long long any = __ballot(mine != 0);
            if (!any) return;
            // pairs of lower lanes come first, then this lane's own earlier ones
            const unsigned long long m0 = __ballot(h0), m1 = __ballot(h1), m2 = __ballot(h2), m3 = __ballot(h3);
            uint32_t row = base + __popcll(m0 & below) + __popcll(m1 & below) + __popcll(m2 & below) + __popcll(m3 & below);
            const int p = piece + p0 + 4 * lane;
            if (h0) { pair_to_row[p] = row; row_to_pair[row] = (uint32_t)p; row++; }
            if (h1) { pair_to_row[p + 1] = row; row_to_pair[row] = (uint32_t)(p + 1); row++; }
            if (h2) { pair_to_row[p + 2] = row; row_to_pair[row] = (uint32_t)(p + 2); row++; }
            if (h3) { pair_to_row[p + 3] = row; row_to_pair[row] = (uint32_t)(p + 3); }
            base += __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3);
        };
        const uint4 *quads = reinterpret_cast<const uint4 *>(staged);
        for (int p0 = 0; p0 < padded; p0 += 512) {
            const uint4 va = quads[p0 / 4 + lane], vb = quads[p0 / 4 + 64 + lane];
            place(va, p0);
            place(vb, p0 + 256);
        }
    }
}

void pf_launch_group_place(const uint32_t *d_ids, int pairs, int experts, const uint32_t *d_offsets,
                           uint32_t *d_pair_to_row, uint32_t *d_row_to_pair, hipStream_t stream) {
    hipLaunchKernelGGL(pf_k_group_place, dim3((experts + 3) / 4), dim3(256), 0, stream, d_ids, pairs, experts, d_offsets,
                       d_pair_to_row, d_row_to_pair);
}

int pf_group_pairs_device(const uint32_t *d_ids, int tokens, int experts, int top_k, uint32_t *d_counts,
                          uint32_t *d_offsets, uint32_t *d_pair_to_row, uint32_t *d_row_to_pair, uint32_t *d_first_bad,
                          hipStream_t stream) {
    const int pairs = tokens * top_k;
    hipLaunchKernelGGL(pf_k_fill_u32, dim3(1), dim3(64), 0, stream, d_first_bad, 1, 0xffffffffu);
    hipLaunchKernelGGL(pf_k_fill_u32, dim3((experts + 255) / 256), dim3(256), 0, stream, d_counts, experts, 0u);
    if (tokens > 0) {
        hipLaunchKernelGGL(pf_k_group_check, dim3((tokens + 255) / 256), dim3(256), 0, stream, d_ids, tokens, experts,
                           top_k, d_first_bad);
        hipLaunchKernelGGL(pf_k_group_count, dim3((pairs + 255) / 256), dim3(256), 0, stream, d_ids, pairs, experts,
                           d_counts);
    }
    hipLaunchKernelGGL(pf_k_group_scan, dim3(1), dim3(256), 0, stream, d_counts, experts, d_offsets);
    if (tokens > 0)
        hipLaunchKernelGGL(pf_k_group_place, dim3((experts + 3) / 4), dim3(256), 0, stream, d_ids, pairs, experts,
                           d_offsets, d_pair_to_row, d_row_to_pair);
    return hipGetLastError() == hipSuccess ? PF_HIP_OK : PF_HIP_E_RUNTIME;
}
