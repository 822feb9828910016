// The two hyper-connection steps either side of the MoE block (src/qwen4_base.c:142-175):
//
//   mixed[t, j]        = (sum over streams h of normed[t, h, j] * sigmoid(logits[t, h, j])) / streams
//   residual[t, h, j] += inject[t, h] * block[t, j]
//
// Both are streaming kernels bound by HBM: the read moves 2 * streams + 1 floats per output
// element, the add 2 * streams + 1 per block element.  A thread owns four adjacent columns (one
// 16-byte access per stream) where the shapes allow it, one column otherwise.  Every product and
// sum is rounded on its own, streams in ascending order, as the reference's loops do, and the
// sigmoid's exponential is the C library's expf bit for bit, so both steps give the reference's
// bits on a host whose C library computes expf that way; nonfinite
// inputs or results set the error word instead of stopping the call.
#include "pf_moe_internal.h"
#include <math.h>

// src/qwen4_cpu_internal.h:103-106 with the C library's expf reproduced bit for bit
__device__ __forceinline__ float hc_sigmoid(float x) { return pf_sigmoid_libm(x); }

template <int V> struct HcVec;
template <> struct HcVec<1> { typedef float type; };
template <> struct HcVec<4> { typedef float4 type; };

// S: the stream count when it is known at compile time (all loads of a thread are then requested
// before the first sigmoid), 0 for any count.
template <int V, int S>
__global__ void __launch_bounds__(256) pf_k_hc_read(const float *normed, size_t n_token_pitch, size_t n_stream_pitch,
                                                    const float *logits, size_t g_token_pitch, size_t g_stream_pitch,
                                                    float *mixed, size_t m_pitch, int streams, int hidden,
                                                    uint32_t *error_word) {
#pragma clang fp contract(off)
    typedef typename HcVec<V>::type Vec;
    const int t = blockIdx.y, j = (blockIdx.x * blockDim.x + threadIdx.x) * V;
    bool bad = false;
    if (j < hidden) {
        const float *n = normed + (size_t)t * n_token_pitch + j, *g = logits + (size_t)t * g_token_pitch + j;
        float sum[V];
#pragma unroll
        for (int c = 0; c < V; c++) sum[c] = 0.0f;
        auto add_stream = [&](const Vec &nv, const Vec &gv) {
            const float *nf = (const float *)&nv, *gf = (const float *)&gv;
#pragma unroll
            for (int c = 0; c < V; c++) {
                if (!pf_finite(nf[c]) || !pf_finite(gf[c])) sum[c] = NAN;
                const float term = nf[c] * hc_sigmoid(gf[c]);
                sum[c] = sum[c] + term;
            }
        };
        if (S) {
            Vec nv[S ? S : 1], gv[S ? S : 1];
#pragma unroll
            for (int h = 0; h < S; h++) {
                nv[h] = *(const Vec *)(n + (size_t)h * n_stream_pitch);
                gv[h] = *(const Vec *)(g + (size_t)h * g_stream_pitch);
            }
#pragma unroll
            for (int h = 0; h < S; h++) add_stream(nv[h], gv[h]);
        } else {
            for (int h = 0; h < streams; h++)
                add_stream(*(const Vec *)(n + (size_t)h * n_stream_pitch), *(const Vec *)(g + (size_t)h * g_stream_pitch));
        }
        Vec out;
        float *of = (float *)&out;
        const float count = (float)streams;
#pragma unroll
        for (int c = 0; c < V; c++) {   // a flagged element is written as zero: what consumes the rows next sees finite input
            const bool ok = pf_finite(sum[c]);
            bad |= !ok;
            of[c] = ok ? sum[c] / count : 0.0f;
        }
        *(Vec *)(mixed + (size_t)t * m_pitch + j) = out;
    }
    if (__any(bad) && pf_lane() == 0) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
}

// The read for a few tokens: one thread per (stream, column) so that every sigmoid of a token is
// evaluated at once; a workgroup covers 64 columns and up to 16 streams, the terms meet in LDS and
// the threads of the first stream add them in stream order.
#define HC_WIDE_STREAMS 16
__global__ void __launch_bounds__(64 * HC_WIDE_STREAMS) pf_k_hc_read_wide(const float *normed, size_t n_token_pitch,
                                                                          size_t n_stream_pitch, const float *logits,
                                                                          size_t g_token_pitch, size_t g_stream_pitch,
                                                                          float *mixed, size_t m_pitch, int streams,
                                                                          int hidden, uint32_t *error_word) {
#pragma clang fp contract(off)
    __shared__ float term[HC_WIDE_STREAMS][64];
    const int c = threadIdx.x, hh = threadIdx.y, t = blockIdx.y, j = blockIdx.x * 64 + c;
    float sum = 0.0f;
    for (int h0 = 0; h0 < streams; h0 += blockDim.y) {
        const int h = h0 + hh;
        float v = 0.0f;
        if (h < streams && j < hidden) {
            const float nv = normed[(size_t)t * n_token_pitch + (size_t)h * n_stream_pitch + j];
            const float gv = logits[(size_t)t * g_token_pitch + (size_t)h * g_stream_pitch + j];
            v = pf_finite(nv) && pf_finite(gv) ? nv * hc_sigmoid(gv) : NAN;
        }
        term[hh][c] = v;
        __syncthreads();
        if (hh == 0) {
            const int n = min((int)blockDim.y, streams - h0);
            for (int k = 0; k < n; k++) sum = sum + term[k][c];
        }
        __syncthreads();
    }
    bool bad = false;
    if (hh == 0 && j < hidden) {
        bad = !pf_finite(sum);
        mixed[(size_t)t * m_pitch + j] = bad ? 0.0f : sum / (float)streams;
    }
    if (__any(bad) && pf_lane() == 0) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
}

template <int V>
__global__ void __launch_bounds__(256) pf_k_hc_add(float *residual, size_t r_token_pitch, size_t r_stream_pitch,
                                                   const float *block, size_t b_pitch, const float *inject,
                                                   size_t i_pitch, int streams, int hidden, uint32_t *error_word) {
#pragma clang fp contract(off)
    typedef typename HcVec<V>::type Vec;
    const int t = blockIdx.y, j = (blockIdx.x * blockDim.x + threadIdx.x) * V;
    bool bad = false;
    if (j < hidden) {
        const Vec bv = *(const Vec *)(block + (size_t)t * b_pitch + j);
        const float *bf = (const float *)&bv;
#pragma unroll
        for (int c = 0; c < V; c++) bad |= !pf_finite(bf[c]);
        float *r = residual + (size_t)t * r_token_pitch + j;
        for (int h = 0; h < streams; h++) {
            const float w = inject[(size_t)t * i_pitch + h];
            Vec rv = *(const Vec *)(r + (size_t)h * r_stream_pitch);
            float *rf = (float *)&rv;
            bad |= !pf_finite(w);
#pragma unroll
            for (int c = 0; c < V; c++) {
                bad |= !pf_finite(rf[c]);
                const float product = w * bf[c];
                rf[c] = rf[c] + product;
                bad |= !pf_finite(rf[c]);
            }
            *(Vec *)(r + (size_t)h * r_stream_pitch) = rv;
        }
    }
    if (__any(bad) && pf_lane() == 0) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
}

#define GRID_ROWS 65535
static bool quad_ok(const void *p, size_t a, size_t b) { return (uintptr_t)p % 16 == 0 && a % 4 == 0 && b % 4 == 0; }

void pf_launch_hc_read(const float *d_normed, size_t n_token_pitch, size_t n_stream_pitch, const float *d_logits,
                       size_t g_token_pitch, size_t g_stream_pitch, float *d_mixed, size_t m_pitch, int tokens,
                       int streams, int hidden, uint32_t *d_error, hipStream_t stream) {
    if (tokens <= 0 || hidden <= 0) return;
    const bool quad = hidden % 4 == 0 && quad_ok(d_normed, n_token_pitch, n_stream_pitch) &&
                      quad_ok(d_logits, g_token_pitch, g_stream_pitch) && quad_ok(d_mixed, m_pitch, 0);
    if ((size_t)tokens * hidden <= 65536 && tokens <= GRID_ROWS) {   // too few columns to occupy the device at four per thread
        const int rows = streams < HC_WIDE_STREAMS ? streams : HC_WIDE_STREAMS;
        hipLaunchKernelGGL(pf_k_hc_read_wide, dim3((hidden + 63) / 64, tokens), dim3(64, rows), 0, stream, d_normed,
                           n_token_pitch, n_stream_pitch, d_logits, g_token_pitch, g_stream_pitch, d_mixed, m_pitch,
                           streams, hidden, d_error);
        return;
    }
    for (int t0 = 0; t0 < tokens; t0 += GRID_ROWS) {   // the token axis of a launch grid is 16 bits wide
        const int n = tokens - t0 < GRID_ROWS ? tokens - t0 : GRID_ROWS;
        const float *nn = d_normed + (size_t)t0 * n_token_pitch, *gg = d_logits + (size_t)t0 * g_token_pitch;
        float *mm = d_mixed + (size_t)t0 * m_pitch;
        if (quad && streams == 4)
            hipLaunchKernelGGL((pf_k_hc_read<4, 4>), dim3((hidden / 4 + 255) / 256, n), dim3(256), 0, stream, nn,
                               n_token_pitch, n_stream_pitch, gg, g_token_pitch, g_stream_pitch, mm, m_pitch, streams,
                               hidden, d_error);
        else if (quad)
            hipLaunchKernelGGL((pf_k_hc_read<4, 0>), dim3((hidden / 4 + 255) / 256, n), dim3(256), 0, stream, nn,
                               n_token_pitch, n_stream_pitch, gg, g_token_pitch, g_stream_pitch, mm, m_pitch, streams,
                               hidden, d_error);
        else
            hipLaunchKernelGGL((pf_k_hc_read<1, 0>), dim3((hidden + 255) / 256, n), dim3(256), 0, stream, nn,
                               n_token_pitch, n_stream_pitch, gg, g_token_pitch, g_stream_pitch, mm, m_pitch, streams,
                               hidden, d_error);
    }
}

void pf_launch_hc_add(float *d_residual, size_t r_token_pitch, size_t r_stream_pitch, const float *d_block,
                      size_t b_pitch, const float *d_inject, size_t i_pitch, int tokens, int streams, int hidden,
                      uint32_t *d_error, hipStream_t stream) {
    if (tokens <= 0 || hidden <= 0) return;
    const bool quad = hidden % 4 == 0 && quad_ok(d_residual, r_token_pitch, r_stream_pitch) &&
                      quad_ok(d_block, b_pitch, 0);
    for (int t0 = 0; t0 < tokens; t0 += GRID_ROWS) {
        const int n = tokens - t0 < GRID_ROWS ? tokens - t0 : GRID_ROWS;
        float *rr = d_residual + (size_t)t0 * r_token_pitch;
        const float *bb = d_block + (size_t)t0 * b_pitch, *ii = d_inject + (size_t)t0 * i_pitch;
        if (quad)
            hipLaunchKernelGGL(pf_k_hc_add<4>, dim3((hidden / 4 + 255) / 256, n), dim3(256), 0, stream, rr,
                               r_token_pitch, r_stream_pitch, bb, b_pitch, ii, i_pitch, streams, hidden, d_error);
        else
            hipLaunchKernelGGL(pf_k_hc_add<1>, dim3((hidden + 255) / 256, n), dim3(256), 0, stream, rr, r_token_pitch,
                               r_stream_pitch, bb, b_pitch, ii, i_pitch, streams, hidden, d_error);
    }
}
