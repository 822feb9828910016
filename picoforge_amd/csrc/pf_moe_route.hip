// Routing (softmax, top-k, renormalisation) and expert grouping kernels.
//
// Two routing paths exist.  The fast one keeps a token's logits in the registers
// of one wave and sums the exponentials with a tree.  It also measures how close
// the k+1 best logits are; when two of them are closer than the rounding noise a
// differently ordered logit sum could have, the token is routed again by the
// exact path, which recomputes its logits in the reference's serial order
// (src/qwen4_packed.c:164-179) and follows src/qwen4_moe.c:219-247 step by step.
#include "pf_moe_internal.h"
// Reference-order arithmetic: a*b+c must stay two roundings.  HIP's __fmul_rn and
// __fadd_rn are plain operators compiled with contraction allowed, so they fuse
// after inlining; the helpers below are compiled with contraction off instead.
#pragma clang fp contract(off)
static __device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
static __device__ __forceinline__ float add_rn(float a, float b) { return a + b; }
static __device__ __forceinline__ float sub_rn(float a, float b) { return a - b; }
static __device__ __forceinline__ float div_rn(float a, float b) { return a / b; }
#include <math.h>

#define ROUTE_MAX_FAST_EXPERTS 1024

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// (p, id) arg-max over the wave: larger p wins, equal p goes to the lower id,
// which is what an ascending scan with a strict comparison selects.
__device__ __forceinline__ void wave_argmax(float &p, uint32_t &id) {
    for (int m = 1; m < PF_WAVE; m <<= 1) {
        float op = __shfl_xor(p, m);
        uint32_t oid = __shfl_xor(id, m);
        if (op > p || (op == p && oid < id)) { p = op; id = oid; }
    }
}

// Reference-order routing of one token by one wave.  z, p, q: LDS arrays of E
// floats (q is scratch).  Writes ids/weights (top_k entries) and leaves the
// probabilities in p.
__device__ void route_exact_wave(const float *z, float *p, float *q, int E, int K, bool norm, uint32_t *ids_out,
                                 float *w_out, int lane) {
    float top = -INFINITY;
    for (int e = lane; e < E; e += PF_WAVE) top = fmaxf(top, z[e]);
    top = pf_wave_max(top);
    // exponent in double, rounded once: the correctly rounded expf
    for (int e = lane; e < E; e += PF_WAVE) p[e] = (float)exp((double)sub_rn(z[e], top));
    wave_lds_fence();
    float sum = 0.0f;
    for (int e = 0; e < E; e++) sum = add_rn(sum, p[e]);   // serial, expert ascending
    wave_lds_fence();
    for (int e = lane; e < E; e += PF_WAVE) {
        float v = div_rn(p[e], sum);
        p[e] = v;
        q[e] = v;
    }
    wave_lds_fence();
    float chosen = 0.0f;
    for (int slot = 0; slot < K; slot++) {
        float best = -2.0f;
        uint32_t best_id = 0xffffffffu;
        for (int e = lane; e < E; e += PF_WAVE) {
            float v = q[e];
            if (v > best) { best = v; best_id = (uint32_t)e; }
        }
        wave_argmax(best, best_id);
        if ((int)(best_id & (PF_WAVE - 1)) == lane) q[best_id] = -1.0f;
        wave_lds_fence();
        chosen = add_rn(chosen, best);
        if (lane == 0) { ids_out[slot] = best_id; w_out[slot] = best; }
    }
    if (norm && lane == 0)
        for (int slot = 0; slot < K; slot++) w_out[slot] = div_rn(w_out[slot], chosen);
}

// ---- fast routing inside a forward --------------------------------------------
template <int NPL>
__global__ void __launch_bounds__(64) pf_k_route_fast(PfKernelArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x, E = a.experts, K = a.top_k;
    const float *zr = a.logits + (size_t)t * E, *sr = a.logit_ssq + (size_t)t * E;
    float z[NPL], s2[NPL], p[NPL];
    float top = -INFINITY;
    bool bad = false;
#pragma unroll
    for (int i = 0; i < NPL; i++) {
        const int e = lane + PF_WAVE * i;
        const bool in = e < E;
        z[i] = in ? zr[e] : -INFINITY;
        s2[i] = in ? sr[e] : 0.0f;
        bad |= in && !pf_finite(z[i]);
        top = fmaxf(top, z[i]);
    }
    if (bad) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    top = pf_wave_max(top);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NPL; i++) {
        p[i] = (lane + PF_WAVE * i < E) ? expf(z[i] - top) : -1.0f;
        sum += fmaxf(p[i], 0.0f);
    }
    sum = pf_wave_sum(sum);
#pragma unroll
    for (int i = 0; i < NPL; i++) if (p[i] >= 0.0f) p[i] = p[i] / sum;
    // k rounds, plus one more to see the runner-up's logit
    const int rounds = K < E ? K + 1 : K;
    float chosen = 0.0f, prev_z = 0.0f, prev_s2 = 0.0f, my_w = 0.0f;
    uint32_t my_id = 0;
    bool close = false;
    for (int r = 0; r < rounds; r++) {
        float best = -2.0f;
        uint32_t best_id = 0xffffffffu;
#pragma unroll
        for (int i = 0; i < NPL; i++)
            if (p[i] > best) { best = p[i]; best_id = (uint32_t)(lane + PF_WAVE * i); }
        wave_argmax(best, best_id);
        const int owner = best_id & (PF_WAVE - 1), slot_i = best_id >> 6;
        float zo = 0.0f, so = 0.0f;
#pragma unroll
        for (int i = 0; i < NPL; i++)
            if (i == slot_i) {
                zo = z[i];
                so = s2[i];
                if (lane == owner) p[i] = -1.0f;
            }
        zo = __shfl(zo, owner);
        so = __shfl(so, owner);
        if (r > 0) {
            // Noise model of a K-term FP32 sum in any order: standard deviation
            // u * sqrt(K * sum(products^2) / 6); eight of those per logit, plus the
            // rounding of z - max and of the exponential.
            const float u = 5.9604645e-8f, hk = (float)a.hidden / 6.0f;
            float tol = 8.0f * u * (sqrtf(hk * so) + sqrtf(hk * prev_s2)) + 4e-6f * fmaxf(1.0f, top - zo);
            close |= !(prev_z - zo > tol);
        }
        prev_z = zo;
        prev_s2 = so;
        if (r < K) {
            chosen += best;
            if (lane == r) { my_id = best_id; my_w = best; }   // top_k <= 64: lane s keeps slot s
        }
    }
    if (lane < K) {
        a.ids[(size_t)t * K + lane] = my_id;
        a.route_weights[(size_t)t * K + lane] = a.norm_topk ? my_w / chosen : my_w;
    }
    if (lane == 0) a.route_flags[t] = close ? 1u : 0u;
}

// Serial-order recomputation for flagged tokens: thread e owns expert e.
__global__ void __launch_bounds__(256) pf_k_route_fix(PfKernelArgs a) {
    extern __shared__ float lds[];
    const int t = blockIdx.x, E = a.experts, H = a.hidden;
    if (!a.route_flags[t]) return;
    float *xs = lds, *z = lds + H, *p = z + E, *q = p + E;
    const float *x = a.x + (size_t)t * a.x_pitch;
    for (int k = threadIdx.x; k < H; k += blockDim.x) xs[k] = x[k];
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const float *w = reinterpret_cast<const float *>(a.w[0]) + (size_t)e * H;
        float sum = 0.0f;
        for (int k = 0; k < H; k++) sum = add_rn(sum, mul_rn(w[k], xs[k]));
        z[e] = sum;
        a.logits[(size_t)t * E + e] = sum;
    }
    __syncthreads();
    if (threadIdx.x < PF_WAVE) {
        route_exact_wave(z, p, q, E, a.top_k, a.norm_topk != 0, a.ids + (size_t)t * a.top_k,
                         a.route_weights + (size_t)t * a.top_k, threadIdx.x);
        if (threadIdx.x == 0) atomicAdd(a.exact_rows, 1u);
    }
}

// Every token through the exact path (expert counts the fast kernel cannot hold).
__global__ void pf_k_flag_all(uint32_t *flags, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) flags[i] = 1u;
}

void pf_launch_route(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    uint32_t *flags = a.route_flags;
    const int npl = (a.experts + PF_WAVE - 1) / PF_WAVE;
    if (a.experts > ROUTE_MAX_FAST_EXPERTS || a.top_k > PF_WAVE)
        hipLaunchKernelGGL(pf_k_flag_all, dim3((tokens + 255) / 256), dim3(256), 0, stream, flags, tokens);
    else if (npl <= 1) hipLaunchKernelGGL(pf_k_route_fast<1>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 2) hipLaunchKernelGGL(pf_k_route_fast<2>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 4) hipLaunchKernelGGL(pf_k_route_fast<4>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 8) hipLaunchKernelGGL(pf_k_route_fast<8>, dim3(tokens), dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(pf_k_route_fast<16>, dim3(tokens), dim3(64), 0, stream, a);
    const size_t lds = ((size_t)a.hidden + 3 * (size_t)a.experts) * sizeof(float);
    hipLaunchKernelGGL(pf_k_route_fix, dim3(tokens), dim3(256), lds, stream, a);
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
    wave_lds_fence();
    route_exact_wave(z, p, q, E, K, norm != 0, ids + (size_t)t * K, weights + (size_t)t * K, lane);
    wave_lds_fence();
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
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = pf_lane();
    if (e >= E) return;
    uint32_t base = offsets[e];
    if (offsets[e + 1] == base) return;
    for (int p0 = 0; p0 < pairs; p0 += PF_WAVE) {
        const int p = p0 + lane;
        const bool hit = p < pairs && ids[p] == (uint32_t)e;
        const unsigned long long mask = __ballot(hit);
        if (hit) {
            const uint32_t row = base + __popcll(mask & ((1ull << lane) - 1ull));
            pair_to_row[p] = row;
            row_to_pair[row] = (uint32_t)p;
        }
        base += __popcll(mask);
    }
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
