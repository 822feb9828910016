// Prefill path: a chunk of tokens through one MoE layer as grouped matrix products on the
// matrix cores.
//
//   pf_k_rows_to_half   f32 rows -> power-of-two scaled fp16 pairs (high + low part) and the
//                       per-32-group sums, the scale, max^2, finite check
//   pf_k_pf_router      router logits [T, E] (+ the shared router as column E) by FP32 MFMA
//   routing, grouping   the kernels of pf_moe_route.hip (serial-order re-route of close tokens,
//                       histogram / scan / stable placement)
//   pf_k_pf_gemm        grouped product over the rows of each expert (the shared expert is
//                       expert E with every token) on v_mfma_f32_32x32x16_f16; gate/up with
//                       the SwiGLU epilogue, or down
//   pf_k_pf_combine     slot-ordered weighted sum of the down rows, then the shared branch
//
// Numerics.  A Q4_K weight is d * (scale * code) - dmin * min (src/qwen4_packed.c:86-93) with
// 6-bit scale and min and a 4-bit code, so scale * code <= 945 and min <= 63 are integers that
// fp16 holds exactly.  The matrix cores therefore multiply exact integer weight operands:
// P = sum_k (scale * code)_k x_k over a 256-block and Q = sum_g min_g * (sum of x over group g),
// and the block's d and dmin are applied in FP32: acc += d * P - dmin * Q.  Activations are
// scaled per row by a power of two so that the largest magnitude lies in [0.5, 1) and split
// into two fp16 parts x = hi + lo (22 significant bits); every product is exact in the FP32
// accumulators, so the result differs from the reference's serial FP32 sum by accumulation
// order and the 2^-22 activation rounding only.
#include "pf_moe_internal.h"

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define A_PITCH 264   // halfs per LDS row of a 256-wide activation tile: 528 bytes, 33 sixteen-byte slots
#define S_PITCH 24    // halfs per LDS row of the group sums (16 used)

// halfs per row of a converted matrix: high parts, low parts, per 256-block 8 + 8 group sums
__host__ __device__ constexpr size_t pf_half_row(int cols) { return 2 * (size_t)cols + (size_t)cols / 16; }

// ---- rows to scaled fp16 pairs ------------------------------------------------------------------
// One workgroup per row (cols a multiple of 256).  scale = 2^e with max|row| / scale in
// [0.5, 1) (1 for a zero row).  Thread j converts the eight values 8j..8j+7; four neighbouring
// threads form one 32-group.
__global__ void __launch_bounds__(256) pf_k_rows_to_half(const float *src, size_t src_pitch, int cols, half_t *dst,
                                                         float *scale_out, float *max2_out, uint32_t *error_word) {
    __shared__ float part[4];
    const size_t row = blockIdx.x;
    const float *s = src + row * src_pitch;
    float m = 0.0f;
    bool bad = false;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = s[c];
        bad |= !pf_finite(v);
        m = fmaxf(m, fabsf(v));
    }
    m = pf_wave_max(m);
    if (pf_lane() == 0) part[threadIdx.x >> 6] = m;
    if (__any(bad) && pf_lane() == 0) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
    __syncthreads();
    m = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    int e = (__float_as_int(m) >> 23) & 255;                  // m in [2^(e-127), 2^(e-126))
    e = (e == 0 || e == 255) ? 126 : min(e, 252);             // zero, subnormal or nonfinite row: scale 1
    const float scale = __int_as_float((e + 1) << 23);        // 2^(e-126)
    const float inv = __int_as_float((253 - e) << 23);        // 2^(126-e)
    half_t *out = dst + row * pf_half_row(cols);
    for (int j = threadIdx.x; j < cols / 8; j += blockDim.x) {
        const float4 a = reinterpret_cast<const float4 *>(s)[2 * j], b = reinterpret_cast<const float4 *>(s)[2 * j + 1];
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        half8v hi, lo;
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const float x = v[c] * inv;
            const half_t h = (half_t)x, l = (half_t)(x - (float)h);
            hi[c] = h;
            lo[c] = l;
            sum += (float)h + (float)l;
        }
        *reinterpret_cast<half8v *>(out + 8 * j) = hi;
        *reinterpret_cast<half8v *>(out + cols + 8 * j) = lo;
        sum += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sum), 0xB1, 0xF, 0xF, true));   // quad xor 1
        sum += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sum), 0x4E, 0xF, 0xF, true));   // quad xor 2
        if ((j & 3) == 0) {
            const int g = j >> 2;
            const half_t sh = (half_t)sum, sl = (half_t)(sum - (float)sh);
            out[2 * cols + 16 * (g >> 3) + (g & 7)] = sh;
            out[2 * cols + 16 * (g >> 3) + 8 + (g & 7)] = sl;
        }
    }
    if (threadIdx.x == 0) {
        scale_out[row] = scale;
        if (max2_out) max2_out[row] = m * m;
    }
}

// squared norm of every router row (once, at upload)
__global__ void __launch_bounds__(64) pf_k_row_norm2(const float *w, int cols, float *out) {
    const float *r = w + (size_t)blockIdx.x * cols;
    float s = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 64) s = fmaf(r[c], r[c], s);
    s = pf_wave_sum(s);
    if (threadIdx.x == 0) out[blockIdx.x] = s;
}

void pf_launch_row_norm2(const float *d_w, int rows, int cols, float *d_out, hipStream_t stream) {
    hipLaunchKernelGGL(pf_k_row_norm2, dim3(rows), dim3(64), 0, stream, d_w, cols, d_out);
}

// ---- router logits by FP32 MFMA ----------------------------------------------------------------
// Workgroup = one 32-token x 32-expert tile, its four waves a quarter of the columns each (the
// partial tiles are added in wave order); operands straight from global memory (the lines a
// lane touches are consumed over the following iterations from the vector cache).
// Column E is the shared router.  Also writes the routing tolerance's bound on the sum of
// squared products, max(x)^2 * |w_e|^2.
__global__ void __launch_bounds__(256) pf_k_pf_router(PfKernelArgs a, int tokens) {
    __shared__ float partial[3][16][64];
    const int H = a.hidden, E = a.experts, lane = pf_lane(), wave = threadIdx.x >> 6;
    const int t0 = blockIdx.x * 32, e0 = blockIdx.y * 32;
    const int i = lane & 31, kk = lane >> 5;
    const int t = min(t0 + i, tokens - 1), e = min(e0 + i, E);
    // the four waves share the tile and split the columns into quarters (hidden is a multiple of 32)
    const int q0 = wave * (H / 32), q1 = q0 + H / 32;
    const float4 *xp = reinterpret_cast<const float4 *>(a.x + (size_t)t * a.x_pitch) + kk;
    const float4 *wp = reinterpret_cast<const float4 *>(e < E ? a.w[0] + (size_t)e * H * 4 : a.w[7]) + kk;
    float16v acc = {0};
#pragma unroll 4
    for (int q = q0; q < q1; q++) {
        const float4 xv = xp[2 * q], wv = wp[2 * q];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.x, wv.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.y, wv.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.z, wv.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv.w, wv.w, acc, 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) partial[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = ((acc[r] + partial[0][r][lane]) + partial[1][r][lane]) + partial[2][r][lane];
    const int col = e0 + i;   // this lane's expert
    const float wn = col < E ? a.w_norm2[col] : 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = t0 + 8 * (r >> 2) + 4 * kk + (r & 3);
        if (row >= tokens || col > E) continue;
        const float z = acc[r];
        if (col < E) {
            a.logits[(size_t)row * E + col] = z;
            a.logit_ssq[(size_t)row * E + col] = a.x_max2[row] * wn;
        } else {
            a.shared_scale[row] = pf_sigmoid(z);
            if (!pf_finite(z)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
        }
    }
}

// ---- grouped product ------------------------------------------------------------------------------
enum { PF_GEMM_GATE_UP = 0, PF_GEMM_DOWN = 1 };

struct Q4Raw { uint4 hdr; uint4 q[4]; };   // one lane's share of a row's 144-byte block: header + 16 bytes per 64 weights

__device__ __forceinline__ void q4_load(Q4Raw &r, const uint8_t *block, int h) {
    r.hdr = *reinterpret_cast<const uint4 *>(block);
#pragma unroll
    for (int j = 0; j < 4; j++) r.q[j] = *reinterpret_cast<const uint4 *>(block + 16 + 32 * j + 16 * h);
}

// 6-bit scale and min of group g from the 12 packed bytes (src/qwen4_packed.c:88-91)
__device__ __forceinline__ void q4_scale_min(const Q4Raw &r, int g, uint32_t &sc, uint32_t &mn) {
    const uint32_t w[3] = {r.hdr.y, r.hdr.z, r.hdr.w};
    const int sh = 8 * (g & 3);
    if (g < 4) {
        sc = (w[0] >> sh) & 63u;
        mn = (w[1] >> sh) & 63u;
    } else {
        const uint32_t hi = (w[2] >> sh) & 255u, lo_s = (w[0] >> sh) & 255u, lo_m = (w[1] >> sh) & 255u;
        sc = (hi & 15u) | ((lo_s & 192u) >> 2);
        mn = (hi >> 4) | ((lo_m & 192u) >> 2);
    }
}

// eight codes (two dwords of nibbles, nibble position nib) times the group's scale, exact in fp16:
// a nibble under the exponent byte 0x64 reads as 1024 + q, and (1024 + q) * s - 1024 * s = q * s
// (the high nibbles stay in place: 1024 + 16 q against s / 16 and 64 s, both exact for a 6-bit s;
// the caller passes the pair of constants that belongs to the nibble position)
__device__ __forceinline__ half8v q4_scaled_codes(uint32_t w0, uint32_t w1, int nib, half2v s2, half2v c1024) {
    const uint32_t mask = nib ? 0xF0F0F0F0u : 0x0F0F0F0Fu;
    const uint32_t q0 = w0 & mask, q1 = w1 & mask;
    const uint32_t bias = 0x64646464u;
    const half2v p0 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q0, 0x04010400u));
    const half2v p1 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q0, 0x04030402u));
    const half2v p2 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q1, 0x04010400u));
    const half2v p3 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q1, 0x04030402u));
    const half2v v0 = p0 * s2 - c1024, v1 = p1 * s2 - c1024, v2 = p2 * s2 - c1024, v3 = p3 * s2 - c1024;
    return half8v{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
}

// One pass: MT row tiles of 32 rows against this wave's two 32-row weight tiles, all K.
// Lane (n = lane % 32, h = lane / 32) owns weight row n of its tiles and, per 64 weights, the
// 16 bytes [16h, 16h + 16) of the 32-byte nibble run: chunk c = 2h + c2 (c2 = 0, 1) of nibble
// position nib is k = 64j + 32 nib + 8c + 0..7, one MFMA per (c2, nib) and activation part.
//
// The activation tile of a 256-block travels from global memory straight into LDS (16 bytes per
// lane, 64 consecutive chunks per wave instruction), one block ahead of the products, into the
// other of two buffers.  Chunk p of a buffer: [0, 1056) high parts, row p / 33, column chunk
// p % 33 (the 33rd is padding); [1056, 2112) low parts likewise; [2112, 2208) group sums, row
// q / 3, chunk q % 3 (the third is padding); the rest, the padding and the rows beyond the
// tile's last read the matrix's all-zero row (index zero_row).
#define TILE_LOADS 35                      // wave instructions per tile
#define TILE_HALFS (TILE_LOADS * 64 * 8)   // 35 840 bytes
#define TILE_LOW (1056 * 8)                // half offsets of the low parts and of the sums in a buffer
#define TILE_SUMS (2112 * 8)

__device__ __forceinline__ uint32_t tile_source(int p, const uint32_t *src_row, uint32_t a_pitch, int a_cols,
                                                uint32_t zero_row) {
    int m, c, base;
    if (p < 2112) {
        const int q = p < 1056 ? p : p - 1056;
        m = q / 33; c = q % 33;
        base = p < 1056 ? 0 : a_cols;
        if (c == 32) m = 32;
    } else {
        const int q = p - 2112;
        m = q / 3; c = q % 3;
        base = 2 * a_cols;
        if (c == 2) m = 32;
    }
    const uint32_t row = m < 32 ? src_row[m] : zero_row;   // src_row holds zero_row beyond the tile's rows
    return row * a_pitch + (uint32_t)base + (row == zero_row ? 0u : 8u * (uint32_t)c);
}

template <int MT>
__device__ __forceinline__ void gemm_pass(half_t *tiles, const uint32_t *src_row, const half_t *a16, int a_cols,
                                          uint32_t zero_row, const uint8_t *wrow0, const uint8_t *wrow1, int kblocks,
                                          float16v (&acc)[2][MT]) {
    static_assert(MT == 1, "one 32-row tile per pass");
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5;
    const uint32_t a_pitch = (uint32_t)pf_half_row(a_cols);
    // this wave's loads of a tile: instruction i = wave + 4 ii covers chunks [64 i, 64 i + 64)
    uint32_t source[9];
#pragma unroll
    for (int ii = 0; ii < 9; ii++) source[ii] = tile_source(64 * (wave + 4 * ii) + lane, src_row, a_pitch, a_cols, zero_row);
    auto issue_tile = [&](int kb, half_t *buffer) {
#pragma unroll
        for (int ii = 0; ii < 9; ii++) {
            const int i = wave + 4 * ii;
            if (i >= TILE_LOADS) break;
            const uint32_t step = 64 * i < 2112 ? 256u : 16u;   // halfs per 256-block in this region (uniform per load)
            __builtin_amdgcn_global_load_lds(a16 + source[ii] + step * (uint32_t)kb, buffer + 512 * i, 16, 0, 0);
        }
    };
    // One 256-block: wait for its bytes, start the next block's, multiply.  The weight bytes
    // alternate between two register sets (cur / next) from block to block.
    auto block_step = [&](int kb, const Q4Raw &cur0, const Q4Raw &cur1, Q4Raw &next0, Q4Raw &next1) {
        half_t *tile_h = tiles + (kb & 1) * TILE_HALFS, *tile_l = tile_h + TILE_LOW, *tile_s = tile_h + TILE_SUMS;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's part of the tile and its weight bytes have arrived
        __syncthreads();                                    // every wave's part; and the other buffer has been consumed
        if (kb + 1 < kblocks) {   // next block's bytes travel while this one is multiplied
            issue_tile(kb + 1, tiles + ((kb + 1) & 1) * TILE_HALFS);
            q4_load(next0, wrow0 + 144 * (kb + 1), h);
            q4_load(next1, wrow1 + 144 * (kb + 1), h);
        }
        const half_t *row_h = tile_h + n * A_PITCH + 16 * h, *row_l = tile_l + n * A_PITCH + 16 * h;
        // first activation fragments, requested before the scale arithmetic
        half8v ah = *reinterpret_cast<const half8v *>(row_h), al = *reinterpret_cast<const half8v *>(row_l);
        const half8v as = *reinterpret_cast<const half8v *>(tile_s + n * S_PITCH + 8 * h);
        // the hardware conversion is exact for every binary16 value, subnormals included
        const half2v dm0 = __builtin_bit_cast(half2v, cur0.hdr.x), dm1 = __builtin_bit_cast(half2v, cur1.hdr.x);
        const float d0 = (float)dm0.x, m0 = (float)dm0.y, d1 = (float)dm1.x, m1 = (float)dm1.y;
        half8v min0, min1;
        half2v s2[2][8], c2k[2][8];
#pragma unroll
        for (int g = 0; g < 8; g++) {
            // even groups sit in the low nibbles (1024 + q, times s, minus 1024 s), odd groups in
            // the high ones (1024 + 16 q, times s / 16, minus 64 s)
            const half_t unit = (g & 1) ? (half_t)0.0625f : (half_t)1.0f;
            const int bias_shift = (g & 1) ? 6 : 10;
            uint32_t sc, mn;
            q4_scale_min(cur0, g, sc, mn);
            min0[g] = (half_t)(int)mn;
            const half_t s0 = (half_t)(int)sc * unit;
            s2[0][g] = half2v{s0, s0};
            c2k[0][g] = half2v{(half_t)(int)(sc << bias_shift), (half_t)(int)(sc << bias_shift)};
            q4_scale_min(cur1, g, sc, mn);
            min1[g] = (half_t)(int)mn;
            const half_t s1 = (half_t)(int)sc * unit;
            s2[1][g] = half2v{s1, s1};
            c2k[1][g] = half2v{(half_t)(int)(sc << bias_shift), (half_t)(int)(sc << bias_shift)};
        }
        // Q: the eight minima against the eight group sums (high parts in k 0..7, low parts in k 8..15)
        const float16v zero = {0};
        const float16v q0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(as, min0, zero, 0, 0, 0);
        const float16v q1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(as, min1, zero, 0, 0, 0);
        // P: scale * code against both activation parts; step s = (j, nib, c2) covers
        // k = 64 j + 32 nib + 16 h + 8 c2 + 0..7, and its fragments are requested one step ahead
        float16v part0 = zero, part1 = zero;
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const int j = s >> 2, nib = (s >> 1) & 1, c2 = s & 1, g = 2 * j + nib;
            half8v nh = ah, nl = al;
            if (s < 15) {
                const int sn = s + 1, kn = 64 * (sn >> 2) + 32 * ((sn >> 1) & 1) + 8 * (sn & 1);
                nh = *reinterpret_cast<const half8v *>(row_h + kn);
                nl = *reinterpret_cast<const half8v *>(row_l + kn);
            }
            const uint4 w0 = cur0.q[j], w1 = cur1.q[j];
            const half8v b0 = q4_scaled_codes(c2 ? w0.z : w0.x, c2 ? w0.w : w0.y, nib, s2[0][g], c2k[0][g]);
            const half8v b1 = q4_scaled_codes(c2 ? w1.z : w1.x, c2 ? w1.w : w1.y, nib, s2[1][g], c2k[1][g]);
            part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b0, part0, 0, 0, 0);
            part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b1, part1, 0, 0, 0);
            part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b0, part0, 0, 0, 0);
            part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b1, part1, 0, 0, 0);
            ah = nh;
            al = nl;
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc[0][0][r] = fmaf(d0, part0[r], fmaf(-m0, q0[r], acc[0][0][r]));
            acc[1][0][r] = fmaf(d1, part1[r], fmaf(-m1, q1[r], acc[1][0][r]));
        }
    };
    Q4Raw a0, a1, b0, b1;
    q4_load(a0, wrow0, h);
    q4_load(a1, wrow1, h);
    issue_tile(0, tiles);
    for (int kb = 0; kb < kblocks; kb += 2) {
        block_step(kb, a0, a1, b0, b1);
        if (kb + 1 < kblocks) block_step(kb + 1, b0, b1, a0, a1);
    }
}

struct GemmTarget {   // what one workgroup of the grouped product works on
    bool shared;
    int first, count, inter, kblocks, a_cols, slab;
    uint32_t zero_row;   // index of the all-zero row that ends the fp16 form of the activation matrix
    const uint8_t *w0, *w1;
    const half_t *a16;
    const float *a_scale;
};

template <int MODE, int MT>
__device__ __forceinline__ void gemm_rows(const PfKernelArgs &a, const GemmTarget &g, int m0, int rows_here, half_t *tiles,
                                          uint32_t *src_row, float *row_scale) {
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5, K = a.top_k;
    for (int m = threadIdx.x; m < 32 * MT; m += 256) {
        uint32_t src = g.zero_row;
        float sc = 0.0f;
        if (m < rows_here) {
            if (MODE == PF_GEMM_GATE_UP) src = g.shared ? (uint32_t)(m0 + m) : a.row_to_pair[g.first + m0 + m] / (uint32_t)K;
            else src = g.shared ? (uint32_t)(m0 + m) : (uint32_t)(g.first + m0 + m);
            sc = g.a_scale[src];
        }
        src_row[m] = src;
        row_scale[m] = sc;
    }
    float16v acc[2][MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) { acc[0][mt] = float16v{0}; acc[1][mt] = float16v{0}; }
    __syncthreads();   // src_row is read by every wave's tile loads
    gemm_pass<MT>(tiles, src_row, g.a16, g.a_cols, g.zero_row, g.w0, g.w1, g.kblocks, acc);
    // epilogue: the lane holds column n of its two tiles; register r of tile mt is row
    // 32 mt + 8 (r / 4) + 4 h + r % 4
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = 32 * mt + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m >= rows_here) continue;
            const float rs = row_scale[m];
            if (MODE == PF_GEMM_GATE_UP) {
                const int unit = 128 * g.slab + 32 * wave + n;
                if (unit >= g.inter) continue;
                const float gate = acc[0][mt][r] * rs, up = acc[1][mt][r] * rs;
                const float v = pf_silu(gate) * up;
                if (g.shared) a.shared_act[(size_t)(m0 + m) * g.inter + unit] = v;
                else a.act[(size_t)(g.first + m0 + m) * g.inter + unit] = v;
            } else {
                const int r0 = 256 * g.slab + 64 * wave + n;
                float *out = a.down + (size_t)(g.first + m0 + m) * a.hidden;
                if (r0 < a.hidden) out[r0] = acc[0][mt][r] * rs;
                if (r0 + 32 < a.hidden) out[r0 + 32] = acc[1][mt][r] * rs;
            }
        }
    }
}

// Histogram of the routed pairs.  counts[] is zero on entry: the workspace starts zeroed and
// pf_k_pf_scan_tiles clears it again once it has been read.
__global__ void pf_k_pf_count(const uint32_t *ids, int pairs, int E, uint32_t *counts) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p < pairs && ids[p] < (uint32_t)E) atomicAdd(&counts[ids[p]], 1u);
}

// One workgroup: exclusive scan of counts[E] into offsets[E + 1], and the row tiles: every
// expert's rows (the shared expert = expert E with all tokens) cut into tiles of 32; tiles[0] =
// count, tiles[1 + i] = expert | (tile index within the expert) << 16.  Leaves counts[] zero.
__global__ void __launch_bounds__(256) pf_k_pf_scan_tiles(uint32_t *counts, int E, int tokens, uint32_t *offsets,
                                                          uint32_t *tiles) {
    __shared__ uint32_t rows_before[256], tiles_before[256];
    const int tid = threadIdx.x, per = (E + 1 + 255) / 256, lo = tid * per, hi = min(E + 1, lo + per);
    uint32_t rows = 0, ntiles = 0;
    for (int e = lo; e < hi; e++) {
        const uint32_t c = e < E ? counts[e] : (uint32_t)tokens;
        if (e < E) rows += c;
        ntiles += (c + 31u) / 32u;
    }
    rows_before[tid] = rows;
    tiles_before[tid] = ntiles;
    __syncthreads();
    if (tid == 0) {
        uint32_t run_rows = 0, run_tiles = 0;
        for (int i = 0; i < 256; i++) {
            const uint32_t r = rows_before[i], n = tiles_before[i];
            rows_before[i] = run_rows;
            tiles_before[i] = run_tiles;
            run_rows += r;
            run_tiles += n;
        }
        offsets[E] = run_rows;
        tiles[0] = run_tiles;
    }
    __syncthreads();
    uint32_t row = rows_before[tid], at = tiles_before[tid];
    for (int e = lo; e < hi; e++) {
        const uint32_t c = e < E ? counts[e] : (uint32_t)tokens, n = (c + 31u) / 32u;
        if (e < E) {
            offsets[e] = row;
            row += c;
            counts[e] = 0;
        }
        for (uint32_t i = 0; i < n; i++) tiles[1 + at + i] = (uint32_t)e | (i << 16);
        at += n;
    }
}

// Workgroup (row tile, slab): 4 waves, each with two 32-row weight tiles (gate + up of 32 units,
// or 2 x 32 down rows) against the tile's 32 rows.
template <int MODE>
__global__ void __launch_bounds__(256) pf_k_pf_gemm(PfKernelArgs a, int tokens, int slabs) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    half_t *tiles = reinterpret_cast<half_t *>(lds_raw);   // two buffers of TILE_HALFS
    __shared__ uint32_t src_row[32];
    __shared__ float row_scale[32];
    const int E = a.experts, lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31;
    // Workgroups go to the eight XCDs round robin by index.  The slabs of one row tile read the
    // same activation rows, so they are given indices eight apart: one XCD, one L2.
    const uint32_t xcd = blockIdx.x % 8, turn = blockIdx.x / 8, tile = (turn / slabs) * 8 + xcd;
    if (tile >= a.tiles[0]) return;
    const uint32_t entry = a.tiles[1 + tile];
    const int expert = entry & 0xffffu, m0 = 32 * (int)(entry >> 16);
    GemmTarget g;
    g.slab = turn % slabs;
    g.shared = expert == E;
    const int P = tokens * a.top_k;
    g.first = g.shared ? P : (int)a.offsets[expert];
    g.count = g.shared ? tokens : (int)a.offsets[expert + 1] - g.first;
    if (g.count <= m0) return;
    g.inter = g.shared ? a.shared_inter : a.inter;
    const size_t ex = g.shared ? 0 : (size_t)expert;
    if (MODE == PF_GEMM_GATE_UP) {
        const int tg = g.shared ? 4 : 1;
        if (128 * g.slab >= g.inter) return;
        const int u = min(128 * g.slab + 32 * wave + n, g.inter - 1);
        g.w0 = a.w[tg] + ex * a.expert_bytes[tg] + (size_t)u * a.row_bytes[tg];
        g.w1 = a.w[tg + 1] + ex * a.expert_bytes[tg + 1] + (size_t)u * a.row_bytes[tg + 1];
        g.kblocks = a.hidden / 256; g.a_cols = a.hidden;
        g.a16 = reinterpret_cast<const half_t *>(a.x16); g.a_scale = a.x_scale;
        g.zero_row = a.token_cap;
    } else {
        const int td = g.shared ? 6 : 3, r0 = 256 * g.slab + 64 * wave + n;
        g.w0 = a.w[td] + ex * a.expert_bytes[td] + (size_t)min(r0, a.hidden - 1) * a.row_bytes[td];
        g.w1 = a.w[td] + ex * a.expert_bytes[td] + (size_t)min(r0 + 32, a.hidden - 1) * a.row_bytes[td];
        g.kblocks = g.inter / 256; g.a_cols = g.inter;
        g.a16 = reinterpret_cast<const half_t *>(g.shared ? a.sact16 : a.act16);
        g.a_scale = g.shared ? a.sact_scale : a.act_scale;
        g.zero_row = g.shared ? a.token_cap : a.token_cap * (uint32_t)a.top_k;
    }
    gemm_rows<MODE, 1>(a, g, m0, min(32, g.count - m0), tiles, src_row, row_scale);
}

// ---- combine ---------------------------------------------------------------------------------------
// y[t] = sum over slots in order of weight * down row, then + sigmoid * shared down row
// (src/qwen4_moe.c:362-372)
__global__ void __launch_bounds__(256) pf_k_pf_combine(PfKernelArgs a, int tokens) {
    const int t = blockIdx.x, H = a.hidden, K = a.top_k, P = tokens * K;
    __shared__ uint32_t rows[64];
    __shared__ float weights[64];
    if ((int)threadIdx.x < K) {
        rows[threadIdx.x] = a.pair_to_row[(size_t)t * K + threadIdx.x];
        weights[threadIdx.x] = a.route_weights[(size_t)t * K + threadIdx.x];
    }
    __syncthreads();
    const float ss = a.shared_scale[t];
    bool bad = false;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float sum = 0.0f;
        for (int s = 0; s < K; s++) {
            const float term = weights[s] * a.down[(size_t)rows[s] * H + c];
            sum += term;
        }
        const float y = sum + ss * a.down[(size_t)(P + t) * H + c];
        bad |= !pf_finite(y);
        a.y[(size_t)t * a.y_pitch + c] = y;
    }
    if (__any(bad) && pf_lane() == 0) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
}

// ---- dispatch --------------------------------------------------------------------------------------
bool pf_prefill_supported(const PfHipMoeDesc &d) {
    for (int j = 1; j <= 6; j++)
        if (d.type[j] != PF_Q4_K) return false;
    if (d.hidden % 256 || d.inter % 256 || d.shared_inter % 256 || d.down_physical != d.inter) return false;
    if (d.top_k > 64 || d.top_k >= d.experts || d.experts >= 65535) return false;
    return true;
}

size_t pf_prefill_half_row(int cols) { return pf_half_row(cols); }
// sum over experts of ceil(rows / 32) <= pairs / 32 + experts, plus the shared expert's tiles
int pf_prefill_max_tiles(int tokens, int experts, int top_k) {
    return (int)(((size_t)tokens * top_k) / 32 + experts + (tokens + 31) / 32 + 1);
}

template <int MODE>
static void launch_gemm(const PfKernelArgs &a, int tokens, int slabs, hipStream_t stream) {
    const size_t lds = 2 * (size_t)TILE_HALFS * sizeof(half_t);
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_pf_gemm<MODE>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        configured = true;
    }
    // the tile count is only known on the device: launch its upper bound, surplus workgroups exit at once
    const int max_tiles = pf_prefill_max_tiles(tokens, a.experts, a.top_k);
    hipLaunchKernelGGL((pf_k_pf_gemm<MODE>), dim3((max_tiles + 7) / 8 * 8 * slabs), dim3(256), lds, stream, a, tokens, slabs);
}

void pf_launch_prefill(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    const int H = a.hidden, E = a.experts, K = a.top_k, I = a.inter, Is = a.shared_inter, P = tokens * K;
    const int last = stage_limit ? stage_limit : 4;
    // stage 1: fp16 parts of x, router logits
    hipLaunchKernelGGL(pf_k_rows_to_half, dim3(tokens), dim3(256), 0, stream, a.x, a.x_pitch, H, (half_t *)a.x16, a.x_scale,
                       a.x_max2, a.error_word);
    hipLaunchKernelGGL(pf_k_pf_router, dim3((tokens + 31) / 32, (E + 1 + 31) / 32), dim3(256), 0, stream, a, tokens);
    if (last < 2) return;
    // stage 2: routes and grouping
    pf_launch_route(a, tokens, stream);
    hipLaunchKernelGGL(pf_k_pf_count, dim3((P + 255) / 256), dim3(256), 0, stream, a.ids, P, E, a.counts);
    hipLaunchKernelGGL(pf_k_pf_scan_tiles, dim3(1), dim3(256), 0, stream, a.counts, E, tokens, a.offsets, a.tiles);
    pf_launch_group_place(a.ids, P, E, a.offsets, a.pair_to_row, a.row_to_pair, stream);
    if (last < 3) return;
    // stage 3: gate/up + SwiGLU, then fp16 parts of the activation rows
    const int gi = I > Is ? I : Is;
    launch_gemm<PF_GEMM_GATE_UP>(a, tokens, (gi + 127) / 128, stream);
    hipLaunchKernelGGL(pf_k_rows_to_half, dim3(P), dim3(256), 0, stream, a.act, (size_t)I, I, (half_t *)a.act16, a.act_scale,
                       (float *)nullptr, a.error_word);
    hipLaunchKernelGGL(pf_k_rows_to_half, dim3(tokens), dim3(256), 0, stream, a.shared_act, (size_t)Is, Is,
                       (half_t *)a.sact16, a.sact_scale, (float *)nullptr, a.error_word);
    if (last < 4) return;
    // stage 4: down and combine
    launch_gemm<PF_GEMM_DOWN>(a, tokens, (H + 255) / 256, stream);
    hipLaunchKernelGGL(pf_k_pf_combine, dim3(tokens), dim3(256), 0, stream, a, tokens);
}
