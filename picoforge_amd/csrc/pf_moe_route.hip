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
// spread over many compute units: one wave per (token, 64 experts), lane e owns expert e and
// the sum runs over k in order, as the reference's, on the transposed router copy
// [hidden][experts]: every step is one coalesced 256-byte load at a wave-uniform base plus the
// lane's offset.  Then one wave per token selects.
__global__ void __launch_bounds__(64) pf_k_route_fix_logits(PfKernelArgs a) {
#pragma clang fp contract(off)
    const int t = blockIdx.x, E = a.experts, H = a.hidden;
    int e = blockIdx.y * PF_WAVE + threadIdx.x;
    if (!a.route_flags[t]) return;
    const float *__restrict__ xs = a.x + (size_t)t * a.x_pitch;
    const float *__restrict__ wt = a.router_t;
    const bool live = e < E;
    e = min(e, E - 1);   // every lane keeps loading: the token's values are shared through v_readlane
    // The sum is one dependent chain; the loads are not.  They are requested 128 at a time, one
    // batch ahead of the chain, so that the chain rarely waits for memory.  The token's values
    // travel the same way, 64 per register, and reach the chain through v_readlane.
    float sum = 0.0f, wa[128], wb[128], xa[2], xb[2];
    const int batches = H / 128, lane = threadIdx.x;
    const uint32_t lane_bytes = 4u * (uint32_t)e;   // uniform row base + 32-bit lane offset: no per-load address arithmetic
    auto load = [&](float (&dst)[128], float (&xdst)[2], int b) {
        const char *row = reinterpret_cast<const char *>(wt + (size_t)(128 * b) * E);
        xdst[0] = xs[128 * b + lane];
        xdst[1] = xs[128 * b + 64 + lane];
#pragma unroll
        for (int j = 0; j < 128; j++) {
            dst[j] = *reinterpret_cast<const float *>(row + lane_bytes);
            row += 4 * (size_t)E;
        }
    };
    auto chain = [&](const float (&src)[128], const float (&xsrc)[2]) {
#pragma unroll
        for (int j = 0; j < 128; j++) {
            const float xj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xsrc[j >> 6]), j & 63));
            const float p = src[j] * xj;
            sum = sum + p;
        }
    };
    if (batches > 0) load(wa, xa, 0);
    for (int b = 0; b < batches; b += 2) {
        if (b + 1 < batches) load(wb, xb, b + 1);
        chain(wa, xa);
        if (b + 2 < batches) load(wa, xa, b + 2);
        if (b + 1 < batches) chain(wb, xb);
    }
    for (int k = 128 * batches; k < H; k++) {
        const float p = (wt + (size_t)k * E)[e] * xs[k];
        sum = sum + p;
    }
    if (live) a.logits[(size_t)t * E + e] = sum;
}

// router [experts][hidden] -> [hidden][experts], once at upload
__global__ void pf_k_transpose(const float *src, int rows, int cols, float *dst) {
    __shared__ float tile[32][33];
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32, tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int j = ty; j < 32; j += 8)
        if (r0 + j < rows && c0 + tx < cols) tile[j][tx] = src[(size_t)(r0 + j) * cols + c0 + tx];
    __syncthreads();
    for (int j = ty; j < 32; j += 8)
        if (c0 + j < cols && r0 + tx < rows) dst[(size_t)(c0 + j) * rows + r0 + tx] = tile[tx][j];
}

void pf_launch_transpose(const float *d_src, int rows, int cols, float *d_dst, hipStream_t stream) {
    hipLaunchKernelGGL(pf_k_transpose, dim3((cols + 31) / 32, (rows + 31) / 32), dim3(256), 0, stream, d_src, rows, cols,
                       d_dst);
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
// same expert, so placement is stable without ordered atomics
__global__ void __launch_bounds__(256) pf_k_group_place(const uint32_t *ids, int pairs, int E, const uint32_t *offsets,
                                                        uint32_t *pair_to_row, uint32_t *row_to_pair) {
    __shared__ uint32_t staged[8192];   // the ids pass through LDS in pieces: the scan then waits on no global load
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = pf_lane();
    const bool active = e < E && offsets[min(e, E - 1) + 1] != offsets[min(e, E - 1)];
    uint32_t base = e < E ? offsets[e] : 0u;
    for (int piece = 0; piece < pairs; piece += 8192) {
        const int len = min(8192, pairs - piece);
        __syncthreads();
        for (int i = threadIdx.x; i < len; i += blockDim.x) staged[i] = ids[piece + i];
        __syncthreads();
        if (!active) continue;
        for (int p0 = 0; p0 < len; p0 += PF_WAVE) {
            const int p = p0 + lane;
            const bool hit = p < len && staged[p] == (uint32_t)e;
            const unsigned long long mask = __ballot(hit);
            if (hit) {
                const uint32_t row = base + __popcll(mask & ((1ull << lane) - 1ull));
                pair_to_row[piece + p] = row;
                row_to_pair[row] = (uint32_t)(piece + p);
            }
            base += __popcll(mask);
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
