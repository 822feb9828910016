// Reference-order kernels: per-element decode and the serial product.
//
// One lane owns one output and walks k upwards, multiplying and adding without
// contraction, exactly as src/qwen4_packed.c:164-179 does on the CPU; the decode
// is the per-element arithmetic of src/qwen4_packed.c:67-122 (all eight formats).  Results are
// bit-identical to the reference.  These kernels serve qw4_packed_matmul,
// qw4_packed_decode_row and the tie fallback of the router; they are not the
// throughput path.
#include "pf_moe_internal.h"
// Reference-order arithmetic: a*b+c must stay two roundings.  HIP's __fmul_rn and
// __fadd_rn are plain operators compiled with contraction allowed, so they fuse
// after inlining; the helpers below are compiled with contraction off instead.
#pragma clang fp contract(off)
static __device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
static __device__ __forceinline__ float add_rn(float a, float b) { return a + b; }
static __device__ __forceinline__ float sub_rn(float a, float b) { return a - b; }
static __device__ __forceinline__ float div_rn(float a, float b) { return a / b; }

__device__ __forceinline__ float exact_value(uint32_t type, const uint8_t *row, int column, const uint64_t *grid) {
    if (type == PF_F32) {
        const uint8_t *p = row + 4 * (size_t)column;
        uint32_t bits = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
        return __uint_as_float(bits);
    }
    if (type == PF_BF16) {
        const uint8_t *p = row + 2 * (size_t)column;
        return __uint_as_float(((uint32_t)p[0] | ((uint32_t)p[1] << 8)) << 16);
    }
    if (type == PF_F16) {
        const uint8_t *p = row + 2 * (size_t)column;
        return pf_half_bits_to_float((uint32_t)p[0] | ((uint32_t)p[1] << 8));
    }
    if (type == PF_Q8_0) {   // src/qwen4_packed.c:80-85
        const uint8_t *b = row + (size_t)(column >> 5) * 34;
        const int code = (int)(int8_t)b[2 + (column & 31)];
        return mul_rn(pf_half_bits_to_float((uint32_t)b[0] | ((uint32_t)b[1] << 8)), (float)code);
    }
    if (type == PF_MXFP4) {  // src/qwen4_packed.c:94-101
        const uint8_t *b = row + (size_t)(column >> 5) * 17;
        const int l = column & 31;
        const uint32_t code = (b[1 + (l & 15)] >> ((l >> 4) * 4)) & 15u;
        return mul_rn(pf_e2m1_value(code), pf_e8m0_scale(b[0]));
    }
    const int lane = column & 255, blk = column >> 8;
    if (type == PF_Q2_K) {   // src/qwen4_packed.c:116-121
        const uint8_t *b = row + (size_t)blk * 84;
        const uint32_t sm = b[lane >> 4];
        const uint32_t code = (b[16 + (lane >> 7) * 32 + (lane & 31)] >> (2 * ((lane & 127) >> 5))) & 3u;
        const float d = pf_half_bits_to_float((uint32_t)b[80] | ((uint32_t)b[81] << 8));
        const float dmin = pf_half_bits_to_float((uint32_t)b[82] | ((uint32_t)b[83] << 8));
        return sub_rn(mul_rn(mul_rn(d, (float)(sm & 15u)), (float)code), mul_rn(dmin, (float)(sm >> 4)));
    }
    if (type == PF_Q4_K) {
        const uint8_t *b = row + (size_t)blk * 144, *sc = b + 4;
        const int g = lane >> 5;
        uint32_t scale, minimum;
        if (g < 4) {
            scale = sc[g] & 63u;
            minimum = sc[g + 4] & 63u;
        } else {
            scale = (sc[g + 4] & 15u) | ((sc[g - 4] & 192u) >> 2);
            minimum = (uint32_t)(sc[g + 4] >> 4) | ((sc[g] & 192u) >> 2);
        }
        const uint32_t code = (b[16 + (g >> 1) * 32 + (lane & 31)] >> ((g & 1) * 4)) & 15u;
        const float d = pf_half_bits_to_float((uint32_t)b[0] | ((uint32_t)b[1] << 8));
        const float dmin = pf_half_bits_to_float((uint32_t)b[2] | ((uint32_t)b[3] << 8));
        return sub_rn(mul_rn(mul_rn(d, (float)scale), (float)code), mul_rn(dmin, (float)minimum));
    }
    // IQ2_XXS
    const uint8_t *b = row + (size_t)blk * 66, *grp = b + 2 + (lane >> 5) * 8;
    const int slot = (lane & 31) >> 3, pos = lane & 7;
    const uint32_t word = (uint32_t)grp[4] | ((uint32_t)grp[5] << 8) | ((uint32_t)grp[6] << 16) |
                          ((uint32_t)grp[7] << 24);
    uint32_t signs = (word >> (7 * slot)) & 127u;
    signs |= pf_parity7(signs) << 7;
    const uint32_t magnitude = (uint32_t)((grid[grp[slot]] >> (8 * pos)) & 255u);
    const float d = pf_half_bits_to_float((uint32_t)b[0] | ((uint32_t)b[1] << 8));
    const float scale = mul_rn(mul_rn(d, (float)(2u * (word >> 28) + 1u)), 0.125f);
    const float v = mul_rn(scale, (float)magnitude);
    return (signs >> pos) & 1u ? -v : v;
}

__global__ void pf_k_exact_matmul(uint32_t type, const uint8_t *w, size_t row_bytes, int n_out, int k_logical,
                                  const float *x, int rows, float *y, uint32_t *error, const uint64_t *grid) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * n_out) return;
    const int m = (int)(i / n_out), n = (int)(i % n_out);
    const uint8_t *row = w + (size_t)n * row_bytes;
    const float *in = x + (size_t)m * k_logical;
    float sum = 0.0f;
    bool bad = false;
    for (int k = 0; k < k_logical; k++) {
        const float v = exact_value(type, row, k, grid);
        const float p = mul_rn(v, in[k]);
        sum = add_rn(sum, p);
        bad |= !pf_finite(v) || !pf_finite(in[k]) || !pf_finite(p) || !pf_finite(sum);
    }
    y[i] = sum;
    if (bad) atomicOr(error, PF_HIP_ERR_NONFINITE);
}

__global__ void pf_k_exact_decode(uint32_t type, const uint8_t *row, int k_storage, float *out, uint32_t *error,
                                  const uint64_t *grid) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= k_storage) return;
    const float v = exact_value(type, row, k, grid);
    out[k] = v;
    if (!pf_finite(v)) atomicOr(error, PF_HIP_ERR_NONFINITE);
}

void pf_launch_exact_matmul(uint32_t type, const uint8_t *d_w, size_t row_bytes, int n_out, int k_logical,
                            const float *d_x, int rows, float *d_y, uint32_t *d_error, const uint64_t *grid,
                            hipStream_t stream) {
    const size_t n = (size_t)rows * n_out;
    if (n == 0) return;
    hipLaunchKernelGGL(pf_k_exact_matmul, dim3((unsigned)((n + 63) / 64)), dim3(64), 0, stream, type, d_w, row_bytes,
                       n_out, k_logical, d_x, rows, d_y, d_error, grid);
}

void pf_launch_exact_decode(uint32_t type, const uint8_t *d_row, int k_storage, float *d_out, uint32_t *d_error,
                            const uint64_t *grid, hipStream_t stream) {
    hipLaunchKernelGGL(pf_k_exact_decode, dim3((k_storage + 255) / 256), dim3(256), 0, stream, type, d_row, k_storage,
                       d_out, d_error, grid);
}

// ---- the block's elementwise steps in the reference's order --------------------------------------
// op 0: SiLU (src/qwen4_base.c:76-91 with divisor and multiplier 1), op 1: sigmoid, op 2: a[j] *= b[j]
// (src/qwen4_moe.c:327-330).  A nonfinite input or result sets the error word.
__global__ void pf_k_exact_elementwise(int op, const float *a, const float *b, float *out, size_t n, uint32_t *error) {
    const size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const float v = a[j];
    float r;
    if (op == 2) r = mul_rn(v, b[j]);
    else {
        r = pf_sigmoid_libm(div_rn(v, 1.0f));
        if (op == 0) r = mul_rn(v, r);
        r = mul_rn(r, 1.0f);
    }
    out[j] = r;
    if (!pf_finite(r) || (op != 2 && !pf_finite(v))) atomicOr(error, PF_HIP_ERR_NONFINITE);
}

// src/qwen4_moe.c:350-368: per (row, col) the slot-order sum of weight * down row, then the gated shared
// row added.  routed receives the first sum (the observer's stage 11), y the finished value.
__global__ void pf_k_exact_combine(const float *down, const uint64_t *pair_to_row, const float *weights, const float *sa,
                                   const float *shared, float *routed, float *y, int tokens, int top_k, int hidden,
                                   uint32_t *error) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)tokens * hidden) return;
    const size_t row = i / hidden, col = i % hidden;
    float sum = 0.0f;
    bool bad = false;
    for (int slot = 0; slot < top_k; slot++) {
        const size_t pair = row * top_k + slot;
        const float term = mul_rn(weights[pair], down[pair_to_row[pair] * hidden + col]);
        sum = add_rn(sum, term);
        bad |= !pf_finite(term) || !pf_finite(sum);
    }
    routed[i] = sum;
    const float term = mul_rn(sa[row], shared[i]);
    const float out = add_rn(sum, term);
    bad |= !pf_finite(term) || !pf_finite(out);
    y[i] = out;
    if (bad) atomicOr(error, PF_HIP_ERR_NONFINITE);
}

void pf_launch_exact_elementwise(int op, const float *d_a, const float *d_b, float *d_out, size_t n, uint32_t *d_error,
                                 hipStream_t stream) {
    if (n) hipLaunchKernelGGL(pf_k_exact_elementwise, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, op, d_a, d_b,
                              d_out, n, d_error);
}

void pf_launch_exact_combine(const float *d_down, const uint64_t *d_pair_to_row, const float *d_weights, const float *d_sa,
                             const float *d_shared, float *d_routed, float *d_y, int tokens, int top_k, int hidden,
                             uint32_t *d_error, hipStream_t stream) {
    const size_t n = (size_t)tokens * hidden;
    if (n) hipLaunchKernelGGL(pf_k_exact_combine, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, d_down,
                              d_pair_to_row, d_weights, d_sa, d_shared, d_routed, d_y, tokens, top_k, hidden, d_error);
}
