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
#include "pf_route_fix.h"

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
    if (lane == 0 && r.close) {   // onto the list of tokens to route again in serial order: [0] count, then the tokens
        const uint32_t at = atomicAdd(a.route_flags, 1u);
        a.route_flags[1 + at] = (uint32_t)t;
    }
}

// Serial-order recomputation for flagged tokens, in two kernels so that a token's logits
// spread over many compute units: one workgroup per (token, slab of 64 experts), lane e of its
// first wave owns expert e and the sum runs over k in order, as the reference's.  The router copy
// is laid out for this, [slab][hidden / 4][64 experts][4 consecutive k]: four steps of the wave
// are one 1 KB piece.  The sum is one dependent chain of 2 x hidden operations; what it must never
// do is wait for memory, so two more waves stream the slab's pieces into an eight-batch LDS ring
// (16 pieces = 64 steps per batch, six batches ahead: about 100 KB on their way) and the token's
// row sits in LDS too, read as broadcasts.  One workgroup barrier per batch hands a batch over and
// frees the one before it.
#define FIX_RING 8
#define FIX_AHEAD 6    // batches on their way or waiting in the ring beyond the one being handed over
#define FIX_BATCH 16   // 1 KB pieces per batch
__global__ void __launch_bounds__(192) pf_k_route_fix_logits(PfKernelArgs a) {
#pragma clang fp contract(off)
    extern __shared__ __align__(16) unsigned char fix_lds[];   // the ring, then the token's row
    const int E = a.experts, H = a.hidden, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = blockIdx.y * PF_WAVE + lane;
    float4 *ring = reinterpret_cast<float4 *>(fix_lds);
    float *xs = reinterpret_cast<float *>(fix_lds + FIX_RING * FIX_BATCH * 1024);
    const float4 *__restrict__ w = reinterpret_cast<const float4 *>(a.router_t) + (size_t)blockIdx.y * ((H + 3) / 4) * PF_WAVE;
    const int batches = H / 64;
    const uint32_t listed = a.route_flags[0];
    for (uint32_t item = blockIdx.x; item < listed; item += gridDim.x) {   // the workgroup's share of the listed tokens
    const int t = (int)a.route_flags[1 + item];
    const float *__restrict__ row = a.x + (size_t)t * a.x_pitch;
    __syncthreads();   // the previous token's row has been used up
    for (int k = threadIdx.x; k < H; k += blockDim.x) xs[k] = row[k];
    __syncthreads();
    if (wave >= 1) {   // two loaders: wave 1 the even batches, wave 2 the odd ones, three batches each on their way
        const int mine = wave - 1;
        auto issue = [&](int b) {   // batch b into slot b % FIX_RING: piece j lands at [slot][j][lane]
            const float4 *src = w + (size_t)(FIX_BATCH * b) * PF_WAVE + lane;
            unsigned char *dst = fix_lds + (size_t)(b % FIX_RING) * FIX_BATCH * 1024;
#pragma unroll
            for (int j = 0; j < FIX_BATCH; j++)
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(src + j * PF_WAVE),
                                                 reinterpret_cast<uint32_t *>(dst + j * 1024), 16, 0, 0);
        };
        for (int b = mine; b < FIX_AHEAD && b < batches; b += 2) issue(b);
        for (int s = 0; s < batches; s++) {
            if ((s & 1) == mine) {
                // batch s has landed when only this wave's younger batches (s + 2, s + 4) are outstanding
                if (s + 4 < batches) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * FIX_BATCH) : "memory");
                else if (s + 2 < batches) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(FIX_BATCH) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __builtin_amdgcn_s_barrier();   // hands batch s over; batch s - 1 has been consumed
            if ((s & 1) == mine && s + FIX_AHEAD < batches) issue(s + FIX_AHEAD);
        }
        continue;
    }
    float sum = 0.0f;
    for (int s = 0; s < batches; s++) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const float4 *slot = ring + (size_t)(s % FIX_RING) * FIX_BATCH * PF_WAVE + lane;
        const float4 *x4 = reinterpret_cast<const float4 *>(xs + 64 * s);
        float4 wv[FIX_BATCH], xv[FIX_BATCH];
#pragma unroll
        for (int j = 0; j < FIX_BATCH; j++) { wv[j] = slot[j * PF_WAVE]; xv[j] = x4[j]; }
#pragma unroll
        for (int j = 0; j < FIX_BATCH; j++) {
            const float p0 = wv[j].x * xv[j].x;
            sum = sum + p0;
            const float p1 = wv[j].y * xv[j].y;
            sum = sum + p1;
            const float p2 = wv[j].z * xv[j].z;
            sum = sum + p2;
            const float p3 = wv[j].w * xv[j].w;
            sum = sum + p3;
        }
    }
    const float *tail = reinterpret_cast<const float *>(w + lane);
    for (int k = 64 * batches; k < H; k++) {   // the lane's k-quad at 256 (k / 4) floats
        const float p = tail[(size_t)(k / 4) * 4 * PF_WAVE + (k & 3)] * xs[k];
        sum = sum + p;
    }
    if (e < E) a.logits[(size_t)t * E + e] = sum;
    }
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
    const int E = a.experts;
    float *z = lds, *p = z + E, *q = p + E;
    const uint32_t listed = a.route_flags[0];
    for (uint32_t item = blockIdx.x; item < listed; item += gridDim.x) {
        const int t = (int)a.route_flags[1 + item];
        for (int e = threadIdx.x; e < E; e += PF_WAVE) z[e] = a.logits[(size_t)t * E + e];
        pf_wave_lds_fence();
        pf_route_exact_wave(z, p, q, E, a.top_k, a.norm_topk != 0, a.ids + (size_t)t * a.top_k,
                            a.route_weights + (size_t)t * a.top_k, threadIdx.x);
        if (threadIdx.x == 0) atomicAdd(a.exact_rows, 1u);
    }
}

// The listed tokens, one wave each: only the experts whose order is in doubt are summed again in serial order
// (pf_route_fix.h); a token that this does not settle is routed the long way by the same wave.  exact_rows[0]
// counts the listed tokens, exact_rows[1] those that went the long way.
template <int NPL>
__global__ void __launch_bounds__(1024) pf_k_route_fix(PfKernelArgs a) {
    extern __shared__ float fix_floats[];
    const int E = a.experts, K = a.top_k, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t listed = a.route_flags[0];
    for (uint32_t item = blockIdx.x; item < listed; item += gridDim.x) {
        const int t = (int)a.route_flags[1 + item];
        const int how = pf_route_fix_block<NPL>(reinterpret_cast<const float *>(a.w[0]), a.x + (size_t)t * a.x_pitch,
                                                a.logits + (size_t)t * E, a.logit_ssq + (size_t)t * E, E, K, a.norm_topk != 0,
                                                a.hidden, fix_floats, a.ids + (size_t)t * K, a.route_weights + (size_t)t * K,
                                                wave, lane);
        if (threadIdx.x == 0) {
            atomicAdd(a.exact_rows, 1u);
            if (how == 2) atomicAdd(a.exact_rows + 1, 1u);
        }
    }
}

// Every token through the exact path (expert counts the fast kernel cannot hold): the full list.
__global__ void pf_k_flag_all(uint32_t *list, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) list[0] = (uint32_t)n;
    if (i < n) list[1 + i] = (uint32_t)i;
}

template <int NPL>
static void launch_route_fix(const PfKernelArgs &a, int workers, size_t lds, hipStream_t stream) {
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_route_fix<NPL>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  144 * 1024);
        configured = true;
    }
    hipLaunchKernelGGL(pf_k_route_fix<NPL>, dim3(workers), dim3(1024), lds, stream, a);
}

bool pf_route_needs_slabs(int experts, int top_k) { return experts > ROUTE_MAX_FAST_EXPERTS || top_k >= PF_WAVE - 1; }

void pf_launch_route(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    const int npl = (a.experts + PF_WAVE - 1) / PF_WAVE;
    if (pf_route_needs_slabs(a.experts, a.top_k))   // the fast routing keeps top_k + 2 keys, one per lane
        hipLaunchKernelGGL(pf_k_flag_all, dim3((tokens + 255) / 256), dim3(256), 0, stream, a.route_flags, tokens);
    else if (npl <= 1) hipLaunchKernelGGL(pf_k_route_fast<1>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 2) hipLaunchKernelGGL(pf_k_route_fast<2>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 4) hipLaunchKernelGGL(pf_k_route_fast<4>, dim3(tokens), dim3(64), 0, stream, a);
    else if (npl <= 8) hipLaunchKernelGGL(pf_k_route_fast<8>, dim3(tokens), dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(pf_k_route_fast<16>, dim3(tokens), dim3(64), 0, stream, a);
    // the listed tokens are few: a fixed number of workgroups walks the list
    const int workers = tokens < 256 ? tokens : 256;
    if (!pf_route_needs_slabs(a.experts, a.top_k)) {
        const size_t lds = pf_route_fix_lds_floats(a.hidden, a.experts) * sizeof(float);
        if (npl <= 1) launch_route_fix<1>(a, workers, lds, stream);
        else if (npl <= 2) launch_route_fix<2>(a, workers, lds, stream);
        else if (npl <= 4) launch_route_fix<4>(a, workers, lds, stream);
        else if (npl <= 8) launch_route_fix<8>(a, workers, lds, stream);
        else launch_route_fix<16>(a, workers, lds, stream);
        return;
    }
    // more experts than a wave's registers hold: every token is listed and all its logits are summed serially
    const size_t fix_lds = (size_t)FIX_RING * FIX_BATCH * 1024 + (size_t)a.hidden * sizeof(float);
    static bool configured = false;   // more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_route_fix_logits),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        configured = true;
    }
    hipLaunchKernelGGL(pf_k_route_fix_logits, dim3(workers, (a.experts + PF_WAVE - 1) / PF_WAVE), dim3(3 * PF_WAVE), fix_lds, stream, a);
    hipLaunchKernelGGL(pf_k_route_fix_select, dim3(workers), dim3(PF_WAVE), 3 * (size_t)a.experts * sizeof(float), stream,
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

// ---- grouping in one launch (the prefill path) ---------------------------------------------------------
// One workgroup of 1024 threads: counts the pairs per expert in LDS, scans the counts (offsets, and the row tiles:
// tiles[0] = count, tiles[1 + i] = expert | tile index << 16; the shared expert = expert E with every token, as
// pf_k_pf_scan_tiles lists them), and hands every pair the next free row of its expert through an LDS cursor.  The rows
// of an expert are therefore in no particular order (pf_k_group_place keeps them in pair order): every row of the
// grouped products is computed on its own and found again through pair_to_row, so the order changes no result, and a
// walk over all pairs per expert, which the order costs, took three times as long as everything else here.
#define GROUP_FUSED_MAX_PAIRS 32768
#define GROUP_FUSED_MAX_EXPERTS 2047
__global__ void __launch_bounds__(1024) pf_k_group_fused(const uint32_t *ids, int pairs, int E, int tokens, uint32_t *offsets,
                                                         uint32_t *tiles, uint32_t *pair_to_row, uint32_t *row_to_pair) {
    extern __shared__ __align__(16) uint32_t fused_lds[];
    __shared__ uint32_t wave_rows[16], wave_tiles[16];
    const int tid = threadIdx.x, quads = pairs / 4;
    uint32_t *counts = fused_lds, *cursor = counts + (E + 1);
    for (int e = tid; e <= E; e += 1024) counts[e] = 0;
    __syncthreads();
    // four pairs a thread and step (ids on a 16-byte boundary), the ragged end pair by pair
    for (int q = tid; q < quads; q += 1024) {
        const uint4 v = reinterpret_cast<const uint4 *>(ids)[q];
        if (v.x < (uint32_t)E) atomicAdd(&counts[v.x], 1u);
        if (v.y < (uint32_t)E) atomicAdd(&counts[v.y], 1u);
        if (v.z < (uint32_t)E) atomicAdd(&counts[v.z], 1u);
        if (v.w < (uint32_t)E) atomicAdd(&counts[v.w], 1u);
    }
    for (int p = 4 * quads + tid; p < pairs; p += 1024) {
        const uint32_t id = ids[p];
        if (id < (uint32_t)E) atomicAdd(&counts[id], 1u);
    }
    __syncthreads();
    // exclusive scan of the counts (rows) and of the row-tile counts, thread t owning `per` consecutive experts
    const int per = (E + 1 + 1023) / 1024, lo = tid * per, hi = min(E + 1, lo + per);
    uint32_t rows = 0, ntiles = 0;
    for (int e = lo; e < hi; e++) {
        const uint32_t c = e < E ? counts[e] : (uint32_t)tokens;
        if (e < E) rows += c;
        ntiles += (c + 31u) / 32u;
    }
    // inclusive scan over the 1024 threads: within a wave by shuffles, then the sixteen waves' totals through LDS
    const int lane = pf_lane(), wave = tid >> 6;
    uint32_t run_rows = rows, run_tiles = ntiles;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up_rows = __shfl_up(run_rows, d), up_tiles = __shfl_up(run_tiles, d);
        if (lane >= d) { run_rows += up_rows; run_tiles += up_tiles; }
    }
    if (lane == 63) { wave_rows[wave] = run_rows; wave_tiles[wave] = run_tiles; }
    __syncthreads();
    for (int w = 0; w < wave; w++) { run_rows += wave_rows[w]; run_tiles += wave_tiles[w]; }
    if (tid == 1023) {
        offsets[E] = run_rows;
        tiles[0] = run_tiles;
    }
    uint32_t row = run_rows - rows, at = run_tiles - ntiles;
    for (int e = lo; e < hi; e++) {
        const uint32_t c = e < E ? counts[e] : (uint32_t)tokens, n = (c + 31u) / 32u;
        if (e < E) {
            cursor[e] = row;
            offsets[e] = row;
            row += c;
        }
        for (uint32_t i = 0; i < n; i++) tiles[1 + at + i] = (uint32_t)e | (i << 16);
        at += n;
    }
    __syncthreads();
    auto place = [&](uint32_t id, int p) {
        if (id >= (uint32_t)E) return;
        const uint32_t r = atomicAdd(&cursor[id], 1u);
        pair_to_row[p] = r;
        row_to_pair[r] = (uint32_t)p;
    };
    for (int q = tid; q < quads; q += 1024) {
        const uint4 v = reinterpret_cast<const uint4 *>(ids)[q];
        place(v.x, 4 * q); place(v.y, 4 * q + 1); place(v.z, 4 * q + 2); place(v.w, 4 * q + 3);
    }
    for (int p = 4 * quads + tid; p < pairs; p += 1024) place(ids[p], p);
}

bool pf_launch_group_fused(const uint32_t *d_ids, int pairs, int experts, int tokens, uint32_t *d_offsets, uint32_t *d_tiles,
                           uint32_t *d_pair_to_row, uint32_t *d_row_to_pair, hipStream_t stream) {
    if (pairs <= 0 || pairs > GROUP_FUSED_MAX_PAIRS || experts > GROUP_FUSED_MAX_EXPERTS || (reinterpret_cast<uintptr_t>(d_ids) & 15)) return false;
    const size_t lds = 2 * ((size_t)experts + 1) * sizeof(uint32_t);
    hipLaunchKernelGGL(pf_k_group_fused, dim3(1), dim3(1024), lds, stream, d_ids, pairs, experts, tokens, d_offsets, d_tiles,
                       d_pair_to_row, d_row_to_pair);
    return true;
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
