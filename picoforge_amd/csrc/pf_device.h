// Device-side helpers shared by the MoE kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "pf_expf_libm.h"

#define PF_WAVE 64

#include "pf_decode_addr.h"   // GGUF type ids, device layout of the tensors, the decode kernels' offsets

__device__ __forceinline__ int pf_lane() { return threadIdx.x & (PF_WAVE - 1); }

// ---- wave64 reductions ------------------------------------------------------
// DPP controls: quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror =
// 0x141, row_mirror = 0x140.  After the four steps every lane of a 16-lane row
// holds the row total; two cross-row exchanges finish the sum in all lanes.
__device__ __forceinline__ float pf_dpp_add(float v, const int ctrl_id) {
    int moved;
    switch (ctrl_id) {
    case 0: moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true); break;
    case 1: moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true); break;
    case 2: moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true); break;
    default: moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true); break;
    }
    return v + __int_as_float(moved);
}

__device__ __forceinline__ float pf_row16_sum(float v) {
    v = pf_dpp_add(v, 0);
    v = pf_dpp_add(v, 1);
    v = pf_dpp_add(v, 2);
    v = pf_dpp_add(v, 3);
    return v;
}

__device__ __forceinline__ float pf_wave_sum(float v) {
    v = pf_row16_sum(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

__device__ __forceinline__ float pf_wave_max(float v) {
    for (int m = 1; m < PF_WAVE; m <<= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}

// ---- scalar pieces of the formats ------------------------------------------
__device__ __forceinline__ float pf_half_bits_to_float(uint32_t h) {
    // Exact binary16 -> binary32 by bit construction (src/qwen4_packed.c:54-66),
    // independent of the wave's denormal mode.
    uint32_t sign = (h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u, bits;
    if (e == 0) {
        if (m == 0) bits = sign;
        else {
            int shift = __clz(m) - 21;          // m < 1024: leading one to bit 10
            m = (m << shift) & 1023u;
            bits = sign | ((uint32_t)(113 - shift) << 23) | (m << 13);
        }
    } else {
        bits = sign | ((e == 31 ? 255u : e + 112u) << 23) | (m << 13);
    }
    return __uint_as_float(bits);
}

__device__ __forceinline__ uint32_t pf_byte(const uint32_t *words, int i) {
    return (words[i >> 2] >> (8 * (i & 3))) & 255u;
}

// 6-bit scale and minimum of group g from the 12 packed bytes of a Q4_K block
// (src/qwen4_packed.c:89-90).
__device__ __forceinline__ void pf_q4k_scale_min(const uint32_t sc[3], int g, uint32_t &scale,
                                                 uint32_t &minimum) {
    if (g < 4) {
        scale = pf_byte(sc, g) & 63u;
        minimum = pf_byte(sc, g + 4) & 63u;
    } else {
        scale = (pf_byte(sc, g + 4) & 15u) | ((pf_byte(sc, g - 4) & 192u) >> 2);
        minimum = (pf_byte(sc, g + 4) >> 4) | ((pf_byte(sc, g) & 192u) >> 2);
    }
}

// E2M1 code of an MXFP4 block (src/qwen4_packed.c:97): magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6; bit 3 the
// sign (code 8 is -0).  Twice the magnitude is an integer: 0, 1, 2, 3, 4, 6, 8, 12.
__device__ __forceinline__ float pf_e2m1_value(uint32_t code) {
    const uint32_t m = code & 7u, twice = m < 4u ? m : (m == 4u ? 4u : m == 5u ? 6u : m == 6u ? 8u : 12u);
    const float v = 0.5f * (float)twice;
    return code & 8u ? -v : v;
}
// E8M0 scale byte: 2^(e - 127); e = 0 is 2^-127 (a subnormal float)
__device__ __forceinline__ float pf_e8m0_scale(uint32_t e) { return __uint_as_float(e ? e << 23 : 0x00400000u); }

__device__ __forceinline__ uint32_t pf_parity7(uint32_t s) {
    // eighth sign of an IQ2_XXS group: parity of the seven stored ones
    return __popc(s & 127u) & 1u;
}

__device__ __forceinline__ float pf_sigmoid(float x) {
    // the two branches of src/qwen4_cpu_internal.h:103-106 share their exponential, expf(-|x|):
    // 1 / (1 + e) for x >= 0, e / (1 + e) below; one evaluation whatever the lanes' signs
    const float e = expf(-fabsf(x));
    return (x >= 0.0f ? 1.0f : e) / (1.0f + e);
}
__device__ __forceinline__ float pf_silu(float x) { return x * pf_sigmoid(x); }

__device__ __forceinline__ bool pf_finite(float v) { return fabsf(v) <= 3.402823466e38f; }
