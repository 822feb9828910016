// General MoE kernels for gfx950: any admitted shape and format combination.
//
// One wave computes one output row product; activations of the current token
// are staged in LDS (zero-padded to the stored row length, so the stored padding
// of a row multiplies zeros).  Shapes that the specialised decode and prefill
// kernels cover are dispatched there instead.
//
// Device layout of the tensors: F32, F16, BF16, Q4_K and Q2_K keep GGUF's bytes.
// IQ2_XXS, Q8_0 and MXFP4 tensors are split at upload into the blocks' payloads
// (64, 32 and 16 bytes; all blocks, row-major) followed by the blocks' scales
// (half, half, one byte), so that payload loads are aligned.
#include "pf_moe_internal.h"

// ---- row products: packed row . x (LDS) -----------------------------------------

__device__ __forceinline__ float dot_row_f32(const uint8_t *row, const float *x, int K, int lane) {
    const float *w = reinterpret_cast<const float *>(row);
    float acc = 0.0f;
    if ((K & 3) == 0) {
        for (int k = lane * 4; k < K; k += 4 * PF_WAVE) {
            float4 a = *reinterpret_cast<const float4 *>(w + k);
            acc = fmaf(a.x, x[k], acc);
            acc = fmaf(a.y, x[k + 1], acc);
            acc = fmaf(a.z, x[k + 2], acc);
            acc = fmaf(a.w, x[k + 3], acc);
        }
    } else {
        for (int k = lane; k < K; k += PF_WAVE) acc = fmaf(w[k], x[k], acc);
    }
    return acc;
}

// Lane l takes 16 nibble bytes of block l/8: the low nibbles are 16 weights of
// group 2j, the high nibbles 16 weights of group 2j+1 (j = (l%8)/2).
__device__ __forceinline__ float dot_row_q4k(const uint8_t *row, const float *x, int nblk, int lane) {
    const int r = lane & 7, j = r >> 1, half = r & 1;
    float acc = 0.0f;
    for (int b = lane >> 3; b < nblk; b += 8) {
        const uint8_t *blk = row + (size_t)b * 144;
        const uint4 hdr = *reinterpret_cast<const uint4 *>(blk);
        const uint4 q = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * r);
        const float d = pf_half_bits_to_float(hdr.x & 0xffffu);
        const float dmin = pf_half_bits_to_float(hdr.x >> 16);
        const uint32_t sc[3] = {hdr.y, hdr.z, hdr.w};
        uint32_t s0, m0, s1, m1;
        pf_q4k_scale_min(sc, 2 * j, s0, m0);
        pf_q4k_scale_min(sc, 2 * j + 1, s1, m1);
        const float *xl = x + 256 * b + 64 * j + 16 * half, *xh = xl + 32;
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
        float ql = 0.0f, qh = 0.0f, sl = 0.0f, sh = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t byte = (qw[w] >> (8 * c)) & 255u;
                const float a = xl[4 * w + c], bb = xh[4 * w + c];
                ql = fmaf((float)(byte & 15u), a, ql);
                qh = fmaf((float)(byte >> 4), bb, qh);
                sl += a;
                sh += bb;
            }
        }
        acc += d * ((float)s0 * ql + (float)s1 * qh) - dmin * ((float)m0 * sl + (float)m1 * sh);
    }
    return acc;
}

// The same product on the tile-ordered copy (pf_decode_addr.h: per 32-row tile and 256-block the 32 headers, then per
// 64-weight run the rows' halves): row n of the expert whose tiles start at `expert`.  Layers that keep only this
// copy of their Q4_K tensors are read through it.
__device__ __forceinline__ float dot_row_q4k_tiled(const uint8_t *expert, int n, const float *x, int nblk, int lane) {
    const int r = lane & 7, j = r >> 1, half = r & 1, row_in_tile = n & 31;
    float acc = 0.0f;
    for (int b = lane >> 3; b < nblk; b += 8) {
        const uint8_t *chunk = expert + pf_q4t_chunk_at(0, 0, n >> 5, nblk, b);
        const uint4 hdr = *reinterpret_cast<const uint4 *>(chunk + pf_q4t_header_at(row_in_tile));
        const uint4 q = *reinterpret_cast<const uint4 *>(chunk + pf_q4t_piece_at(j, half, row_in_tile));
        const float d = pf_half_bits_to_float(hdr.x & 0xffffu);
        const float dmin = pf_half_bits_to_float(hdr.x >> 16);
        const uint32_t sc[3] = {hdr.y, hdr.z, hdr.w};
        uint32_t s0, m0, s1, m1;
        pf_q4k_scale_min(sc, 2 * j, s0, m0);
        pf_q4k_scale_min(sc, 2 * j + 1, s1, m1);
        const float *xl = x + 256 * b + 64 * j + 16 * half, *xh = xl + 32;
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
        float ql = 0.0f, qh = 0.0f, sl = 0.0f, sh = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t byte = (qw[w] >> (8 * c)) & 255u;
                const float a = xl[4 * w + c], bb = xh[4 * w + c];
                ql = fmaf((float)(byte & 15u), a, ql);
                qh = fmaf((float)(byte >> 4), bb, qh);
                sl += a;
                sh += bb;
            }
        }
        acc += d * ((float)s0 * ql + (float)s1 * qh) - dmin * ((float)m0 * sl + (float)m1 * sh);
    }
    return acc;
}

// Lane l takes group l (32 weights, one aligned 8-byte payload word) per pass.
__device__ __forceinline__ float dot_row_iq2(const uint8_t *payload, const uint16_t *scales, const float *x, int nblk,
                                             int lane, const uint64_t *grid) {
    const int ngroups = nblk * 8;
    float acc = 0.0f;
    for (int gi = lane; gi < ngroups; gi += PF_WAVE) {
        const uint2 p = *reinterpret_cast<const uint2 *>(payload + 8 * (size_t)gi);
        const float d = pf_half_bits_to_float(scales[gi >> 3]);
        const uint32_t idx = p.x, word = p.y;
        const float scale = d * (float)(2u * (word >> 28) + 1u) * 0.125f;
        const float *xg = x + 32 * gi;
        float gacc = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 4; slot++) {
            const uint64_t mags = grid[(idx >> (8 * slot)) & 255u];
            uint32_t signs = (word >> (7 * slot)) & 127u;
            signs |= pf_parity7(signs) << 7;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float m = (float)(uint32_t)((mags >> (8 * e)) & 255u);
                const float xv = xg[8 * slot + e];
                gacc = fmaf((signs >> e) & 1u ? -m : m, xv, gacc);
            }
        }
        acc = fmaf(scale, gacc, acc);
    }
    return acc;
}

// The same product on the tile-ordered copy (pf_decode_addr.h: per 32-row tile and 256-block the rows' 16-byte pieces of
// each 64-weight run, two groups a piece, then the rows' block scales): row n of the expert whose tiles start at
// `expert`.  Pool slots of a streamed layer are kept in this order for the decode kernels; longer batches read them here.
__device__ __forceinline__ float dot_row_iq2_tiled(const uint8_t *expert, int n, const float *x, int nblk, int lane,
                                                   const uint64_t *grid) {
    const int ngroups = nblk * 8, row_in_tile = n & 31;
    float acc = 0.0f;
    for (int gi = lane; gi < ngroups; gi += PF_WAVE) {
        const uint8_t *chunk = expert + pf_i2t_chunk_at(0, 0, n >> 5, nblk, gi >> 3);
        const uint2 p = *reinterpret_cast<const uint2 *>(chunk + pf_i2t_piece_at((gi & 7) >> 1, row_in_tile) + 8 * (gi & 1));
        const float d = pf_half_bits_to_float(*reinterpret_cast<const uint16_t *>(chunk + pf_i2t_scale_at(row_in_tile)));
        const uint32_t idx = p.x, word = p.y;
        const float scale = d * (float)(2u * (word >> 28) + 1u) * 0.125f;
        const float *xg = x + 32 * gi;
        float gacc = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 4; slot++) {
            const uint64_t mags = grid[(idx >> (8 * slot)) & 255u];
            uint32_t signs = (word >> (7 * slot)) & 127u;
            signs |= pf_parity7(signs) << 7;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float m = (float)(uint32_t)((mags >> (8 * e)) & 255u);
                const float xv = xg[8 * slot + e];
                gacc = fmaf((signs >> e) & 1u ? -m : m, xv, gacc);
            }
        }
        acc = fmaf(scale, gacc, acc);
    }
    return acc;
}

// F16 / BF16 rows: two values per lane and step.
template <bool BF>
__device__ __forceinline__ float dot_row_16(const uint8_t *row, const float *x, int K, int lane) {
    const uint16_t *w = reinterpret_cast<const uint16_t *>(row);
    float acc = 0.0f;
    for (int k = lane; k < K; k += PF_WAVE) {
        const float v = BF ? __uint_as_float((uint32_t)w[k] << 16) : pf_half_bits_to_float(w[k]);
        acc = fmaf(v, x[k], acc);
    }
    return acc;
}

// Q8_0, device layout: 32 code bytes per block (aligned), the half scales apart.  Lane l takes block l.
__device__ __forceinline__ float dot_row_q8(const uint8_t *payload, const uint16_t *scales, const float *x, int nblk,
                                            int lane) {
    float acc = 0.0f;
    for (int b = lane; b < nblk; b += PF_WAVE) {
        const uint4 lo = *reinterpret_cast<const uint4 *>(payload + 32 * (size_t)b);
        const uint4 hi = *reinterpret_cast<const uint4 *>(payload + 32 * (size_t)b + 16);
        const uint32_t q[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        const float *xb = x + 32 * b;
        float g = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; w++)
#pragma unroll
            for (int c = 0; c < 4; c++) g = fmaf((float)(int)(int8_t)(q[w] >> (8 * c)), xb[4 * w + c], g);
        acc = fmaf(pf_half_bits_to_float(scales[b]), g, acc);
    }
    return acc;
}

// MXFP4, device layout: 16 nibble bytes per block (aligned), the scale bytes apart.  Low nibbles are
// values 0..15 of the block, high nibbles 16..31.
__device__ __forceinline__ float dot_row_mxfp4(const uint8_t *payload, const uint8_t *scales, const float *x, int nblk,
                                               int lane) {
    float acc = 0.0f;
    for (int b = lane; b < nblk; b += PF_WAVE) {
        const uint4 p = *reinterpret_cast<const uint4 *>(payload + 16 * (size_t)b);
        const uint32_t q[4] = {p.x, p.y, p.z, p.w};
        const float *xb = x + 32 * b;
        float g = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t byte = (q[w] >> (8 * c)) & 255u;
                g = fmaf(pf_e2m1_value(byte & 15u), xb[4 * w + c], g);
                g = fmaf(pf_e2m1_value(byte >> 4), xb[16 + 4 * w + c], g);
            }
        acc = fmaf(pf_e8m0_scale(scales[b]), g, acc);
    }
    return acc;
}

// Q2_K (GGUF bytes): lane l takes the group of 16 values l of the row: 16 code bytes of one bit plane,
// one scale | min << 4 byte.  Group g of a block: half g / 8, plane (g % 8) / 2, bytes (g % 2) * 16 ...
__device__ __forceinline__ float dot_row_q2k(const uint8_t *row, const float *x, int nblk, int lane) {
    float acc = 0.0f;
    for (int gi = lane; gi < nblk * 16; gi += PF_WAVE) {
        const uint8_t *blk = row + (size_t)(gi >> 4) * 84;
        const int g = gi & 15, plane = (g & 7) >> 1;
        const uint32_t *p = reinterpret_cast<const uint32_t *>(blk + 16 + (g >> 3) * 32 + (g & 1) * 16);   // 4-byte aligned
        const uint32_t q[4] = {p[0], p[1], p[2], p[3]};
        const uint32_t sm = blk[g], dd = *reinterpret_cast<const uint32_t *>(blk + 80);
        const float *xg = x + 16 * gi;
        float dotq = 0.0f, sumx = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float xv = xg[4 * w + c];
                dotq = fmaf((float)((q[w] >> (8 * c + 2 * plane)) & 3u), xv, dotq);
                sumx += xv;
            }
        acc += pf_half_bits_to_float(dd & 0xffffu) * (float)(sm & 15u) * dotq -
               pf_half_bits_to_float(dd >> 16) * (float)(sm >> 4) * sumx;
    }
    return acc;
}

// Row n of expert e of tensor t against x (LDS, padded to the stored length).
__device__ __forceinline__ float dot_tensor_row(const PfKernelArgs &a, int t, size_t e, size_t n, const float *x,
                                                int lane, const uint64_t *grid) {
    const uint8_t *row = a.w[t] + e * a.expert_bytes[t] + n * a.row_bytes[t];
    float v;
    const size_t first_block = (e * a.n_out[t] + n) * a.blocks_per_row[t];   // of the row, for the formats stored split
    const uint8_t *scales = a.w[t] + a.scale_offset[t];
    switch (a.type[t]) {
    case PF_F32: v = dot_row_f32(row, x, a.k_logical[t], lane); break;
    case PF_F16: v = dot_row_16<false>(row, x, a.k_logical[t], lane); break;
    case PF_BF16: v = dot_row_16<true>(row, x, a.k_logical[t], lane); break;
    case PF_Q4_K:
        v = a.w[t] ? dot_row_q4k(row, x, a.blocks_per_row[t], lane)
                   : dot_row_q4k_tiled(a.wt[t] + e * a.expert_bytes[t], (int)n, x, a.blocks_per_row[t], lane);
        break;
    case PF_Q2_K: v = dot_row_q2k(row, x, a.blocks_per_row[t], lane); break;
    case PF_Q8_0:
        v = dot_row_q8(row, reinterpret_cast<const uint16_t *>(scales) + first_block, x, a.blocks_per_row[t], lane);
        break;
    case PF_MXFP4: v = dot_row_mxfp4(row, scales + first_block, x, a.blocks_per_row[t], lane); break;
    default:
        v = a.w[t] ? dot_row_iq2(row, reinterpret_cast<const uint16_t *>(scales) + first_block, x, a.blocks_per_row[t], lane, grid)
                   : dot_row_iq2_tiled(a.wi[t] + e * pf_i2t_expert_bytes(a.n_out[t], a.blocks_per_row[t]), (int)n, x,
                                       a.blocks_per_row[t], lane, grid);
    }
    return pf_wave_sum(v);
}

__device__ __forceinline__ void stage_grid(uint64_t *grid_lds, const uint64_t *grid_global) {
    for (int i = threadIdx.x; i < 256; i += blockDim.x) grid_lds[i] = grid_global[i];
}

// copies `count` floats and zero-fills up to `padded`
__device__ __forceinline__ bool stage_row(float *dst, const float *src, int count, int padded) {
    bool bad = false;
    for (int k = threadIdx.x; k < padded; k += blockDim.x) {
        float v = k < count ? src[k] : 0.0f;
        dst[k] = v;
        bad |= !pf_finite(v);
    }
    return bad;
}

// ---- stage 1: everything that depends on x only -------------------------------
// Units per token: experts router rows, shared_inter fused shared gate/up rows,
// one shared-router row.  One wave per unit.
__global__ void __launch_bounds__(256) pf_k_pre(PfKernelArgs a) {
    extern __shared__ float lds[];
    __shared__ uint64_t grid[256];
    const int H = a.hidden, t = blockIdx.y, lane = pf_lane(), wave = threadIdx.x >> 6;
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) a.route_flags[0] = 0;   // the routing's list starts empty
    if (stage_row(lds, a.x + (size_t)t * a.x_pitch, H, H)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    stage_grid(grid, a.iq2_grid);
    __syncthreads();
    const int unit = blockIdx.x * 4 + wave, E = a.experts, Is = a.shared_inter;
    if (unit < E) {
        // router logit and the sum of squared products used by the tie guard
        const float *w = reinterpret_cast<const float *>(a.w[0]) + (size_t)unit * H;
        float acc = 0.0f, sq = 0.0f;
        for (int k = lane; k < H; k += PF_WAVE) {
            float p = w[k] * lds[k];
            acc += p;
            sq = fmaf(p, p, sq);
        }
        acc = pf_wave_sum(acc);
        sq = pf_wave_sum(sq);
        if (lane == 0) {
            a.logits[(size_t)t * E + unit] = acc;
            a.logit_ssq[(size_t)t * E + unit] = sq;
        }
    } else if (unit < E + Is) {
        const int n = unit - E;
        float g = dot_tensor_row(a, 4, 0, n, lds, lane, grid);
        float u = dot_tensor_row(a, 5, 0, n, lds, lane, grid);
        float v = pf_silu(g) * u;
        if (lane == 0) {
            a.shared_act[(size_t)t * Is + n] = v;
            if (!pf_finite(v)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
        }
    } else if (unit == E + Is) {
        float z = dot_tensor_row(a, 7, 0, 0, lds, lane, grid);
        float s = pf_sigmoid(z);
        if (lane == 0) {
            a.shared_scale[t] = s;
            if (!pf_finite(z)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
        }
    }
}

// ---- stage 3: routed gate/up + SwiGLU ----------------------------------------
// grid (ceil(inter/4), pairs); pair p = token * top_k + slot.
__global__ void __launch_bounds__(256) pf_k_gate_up(PfKernelArgs a) {
    extern __shared__ float lds[];
    __shared__ uint64_t grid[256];
    const int H = a.hidden, pair = blockIdx.y, t = pair / a.top_k, lane = pf_lane(), wave = threadIdx.x >> 6;
    stage_row(lds, a.x + (size_t)t * a.x_pitch, H, H);
    stage_grid(grid, a.iq2_grid);
    __syncthreads();
    const int n = blockIdx.x * 4 + wave;
    if (n >= a.inter) return;
    const uint32_t e = a.ids[pair], at = a.slots ? a.slots[pair] : e;   // where the expert's rows are
    if (e >= (uint32_t)a.experts || (a.slots && at >= a.pool_slots)) {
        if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS);
        return;
    }
    float g = dot_tensor_row(a, 1, at, n, lds, lane, grid);
    float u = dot_tensor_row(a, 2, at, n, lds, lane, grid);
    float v = pf_silu(g) * u;
    if (lane == 0) {
        a.act[(size_t)pair * a.inter + n] = v;
        if (!pf_finite(v)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
}

// ---- stage 4: routed down products, slot-ordered weighted sum, shared branch ----
// grid (ceil(hidden/4), tokens).  LDS holds the token's top_k activation rows
// (each padded to the stored row length of the down tensor) and its shared row.
__global__ void __launch_bounds__(256) pf_k_down_combine(PfKernelArgs a) {
    extern __shared__ float lds[];
    __shared__ uint64_t grid[256];
    const int I = a.inter, Ip = a.down_physical, Is = a.shared_inter, K = a.top_k, t = blockIdx.y;
    const int lane = pf_lane(), wave = threadIdx.x >> 6;
    for (int s = 0; s < K; s++) stage_row(lds + s * Ip, a.act + ((size_t)t * K + s) * I, I, Ip);
    float *sact = lds + K * Ip;
    stage_row(sact, a.shared_act + (size_t)t * Is, Is, Is);
    stage_grid(grid, a.iq2_grid);
    __syncthreads();
    const int n = blockIdx.x * 4 + wave;
    if (n >= a.hidden) return;
    float sum = 0.0f;
    for (int s = 0; s < K; s++) {
        const uint32_t e = a.ids[(size_t)t * K + s], at = a.slots ? a.slots[(size_t)t * K + s] : e;
        if (e >= (uint32_t)a.experts || (a.slots && at >= a.pool_slots)) {
            if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS);
            return;
        }
        float dsum = dot_tensor_row(a, 3, at, n, lds + s * Ip, lane, grid);
        sum += a.route_weights[(size_t)t * K + s] * dsum;   // slot order, as src/qwen4_moe.c:362-372
    }
    float sh = dot_tensor_row(a, 6, 0, n, sact, lane, grid);
    float y = sum + a.shared_scale[t] * sh;
    if (lane == 0) {
        PfOutputRegs out_regs;
        pf_output_prefetch(a, t, n, out_regs);
        if (!pf_output_commit(a, t, n, y, out_regs)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
}

size_t pf_general_lds_bytes(const PfKernelArgs &a) {
    const size_t down = ((size_t)a.top_k * a.down_physical + a.shared_inter) * sizeof(float);
    const size_t x = (size_t)a.hidden * sizeof(float);
    return down > x ? down : x;
}

void pf_launch_general(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit, int first_stage) {
    // stage_limit (profiling, expert streaming): launch only the first so many of the four stages; 0 = all.
    // first_stage: the stage to start at (expert streaming resumes at 3 once the routed experts are resident).
    const int units = a.experts + a.shared_inter + 1, last = stage_limit ? stage_limit : 4;
    const size_t x_lds = (size_t)a.hidden * sizeof(float);
    if (first_stage <= 1 && last >= 1) hipLaunchKernelGGL(pf_k_pre, dim3((units + 3) / 4, tokens), dim3(256), x_lds, stream, a);
    if (first_stage <= 2 && last >= 2) pf_launch_route(a, tokens, stream);
    if (first_stage <= 3 && last >= 3)
        hipLaunchKernelGGL(pf_k_gate_up, dim3((a.inter + 3) / 4, tokens * a.top_k), dim3(256), x_lds, stream, a);
    if (last < 4) return;
    const size_t act_lds = ((size_t)a.top_k * a.down_physical + a.shared_inter) * sizeof(float);
    hipLaunchKernelGGL(pf_k_down_combine, dim3((a.hidden + 3) / 4, tokens), dim3(256), act_lds, stream, a);
}
