/* Seeded synthetic inputs for the MoE path: normal weights quantised to Q4_K,
 * uniformly drawn IQ2_XXS blocks, normal F32 tensors.
 *
 * The reference ships no quantiser (its tests draw raw block bytes,
 * tests/test_qwen4_packed.py:46-68); this one only has to produce valid blocks,
 * because every implementation under comparison decodes the same bytes.
 * All generators are counter based: element i of stream `seed` depends on
 * (seed, i) only, so results do not depend on the thread count. */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static uint64_t mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

/* two standard normals from one 64-bit draw (Box-Muller on two 32-bit uniforms) */
static void normal_pair(uint64_t seed, uint64_t index, float *a, float *b) {
    uint64_t r = mix64(seed * 0xd1342543de82ef95ull + index);
    r = mix64(r ^ seed);
    float u1 = ((float)(uint32_t)(r >> 40) + 0.5f) * (1.0f / 16777216.0f); /* (0,1) */
    float u2 = ((float)(uint32_t)((r >> 16) & 0xffffffu) + 0.5f) * (1.0f / 16777216.0f);
    float radius = sqrtf(-2.0f * logf(u1)), angle = 6.28318530717958647692f * u2;
    *a = radius * cosf(angle);
    *b = radius * sinf(angle);
}

void pf_synth_normal_f32(float *out, size_t n, uint64_t seed, float mean, float std) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < (n + 1) / 2; i++) {
        float a, b;
        normal_pair(seed, i, &a, &b);
        out[2 * i] = mean + std * a;
        if (2 * i + 1 < n) out[2 * i + 1] = mean + std * b;
    }
}

/* float -> binary16 bits, round to nearest even; finite inputs inside the half range */
static uint16_t half_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mant = x & 0x7fffffu;
    int e = (int)((x >> 23) & 255u) - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7bffu);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        mant |= 0x800000u;
        int shift = 14 - e;
        uint32_t h = mant >> shift, rem = mant & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (mant >> 13), rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

static float half_float(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u, bits;
    if (e == 0) {
        float v = (float)m * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    bits = sign | ((e + 112u) << 23) | (m << 13);
    float v;
    memcpy(&v, &bits, 4);
    return v;
}

static int clampi(int v, int lo, int hi) { return v < lo ? lo : v > hi ? hi : v; }

/* One Q4_K super-block from 256 floats.  Block layout (public ggml format):
 * half d, half dmin, 12 bytes of 6-bit scales/mins, 128 bytes of nibbles. */
static void q4k_block(const float *v, unsigned char *out) {
    float scale[8], lowest[8], max_scale = 0, max_min = 0;
    for (int g = 0; g < 8; g++) {
        float lo = 0, hi = 0;
        for (int i = 0; i < 32; i++) {
            float x = v[32 * g + i];
            if (x < lo) lo = x;
            if (x > hi) hi = x;
        }
        scale[g] = (hi - lo) / 15.0f;
        lowest[g] = -lo;
        if (scale[g] > max_scale) max_scale = scale[g];
        if (lowest[g] > max_min) max_min = lowest[g];
    }
    uint16_t dh = half_bits(max_scale / 63.0f), mh = half_bits(max_min / 63.0f);
    float d = half_float(dh), dmin = half_float(mh);
    unsigned sc[8], mn[8];
    for (int g = 0; g < 8; g++) {
        sc[g] = d > 0 ? (unsigned)clampi((int)lrintf(scale[g] / d), 0, 63) : 0;
        mn[g] = dmin > 0 ? (unsigned)clampi((int)lrintf(lowest[g] / dmin), 0, 63) : 0;
    }
    memset(out, 0, 144);
    out[0] = (unsigned char)(dh & 255u); out[1] = (unsigned char)(dh >> 8);
    out[2] = (unsigned char)(mh & 255u); out[3] = (unsigned char)(mh >> 8);
    unsigned char *p = out + 4;
    for (int g = 0; g < 4; g++) {
        p[g] = (unsigned char)((sc[g] & 63u) | ((sc[g + 4] >> 4) << 6));
        p[g + 4] = (unsigned char)((mn[g] & 63u) | ((mn[g + 4] >> 4) << 6));
        p[g + 8] = (unsigned char)((sc[g + 4] & 15u) | ((mn[g + 4] & 15u) << 4));
    }
    for (int g = 0; g < 8; g++) {
        float step = d * (float)sc[g], offset = dmin * (float)mn[g];
        for (int i = 0; i < 32; i++) {
            int q = step > 0 ? clampi((int)lrintf((v[32 * g + i] + offset) / step), 0, 15) : 0;
            out[16 + (g / 2) * 32 + i] |= (unsigned char)(q << ((g % 2) * 4));
        }
    }
}

void pf_synth_q4k_quantize(const float *values, size_t blocks, unsigned char *out) {
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) q4k_block(values + 256 * b, out + 144 * b);
}

/* blocks of N(0, std) weights, quantised on the fly; block b of stream `seed` */
void pf_synth_q4k_normal(unsigned char *out, size_t blocks, uint64_t seed, float std) {
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) {
        float v[256];
        for (int i = 0; i < 128; i++) {
            normal_pair(seed, b * 128 + (size_t)i, &v[2 * i], &v[2 * i + 1]);
            v[2 * i] *= std;
            v[2 * i + 1] *= std;
        }
        q4k_block(v, out + 144 * b);
    }
}

/* IQ2_XXS blocks with uniformly drawn grid indices, sign words and 4-bit scales;
 * d = d_base * (1 + 3u), a finite positive half.  Layout: half d, then eight
 * groups of {4 grid bytes, u32 = 4x7 sign bits | scale << 28}. */
void pf_synth_iq2xxs_uniform(unsigned char *out, size_t blocks, uint64_t seed, float d_base) {
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) {
        unsigned char *p = out + 66 * b;
        uint64_t r = mix64(mix64(seed) ^ (b * 0x9e3779b97f4a7c15ull));
        float u = (float)(uint32_t)(r >> 40) * (1.0f / 16777216.0f);
        uint16_t dh = half_bits(d_base * (1.0f + 3.0f * u));
        p[0] = (unsigned char)(dh & 255u); p[1] = (unsigned char)(dh >> 8);
        for (int g = 0; g < 8; g++) {
            uint64_t w = mix64(r + (uint64_t)g + 1);
            memcpy(p + 2 + 8 * g, &w, 8);
        }
    }
}

/* ---- formats of the real checkpoints' other tensors ---------------------------------------- */
static void normals(float *v, int n, uint64_t seed, size_t first, float std) {
    for (int i = 0; i < n / 2; i++) {
        normal_pair(seed, first / 2 + (size_t)i, &v[2 * i], &v[2 * i + 1]);
        v[2 * i] *= std;
        v[2 * i + 1] *= std;
    }
}

/* Q8_0 blocks (half d, 32 signed bytes) of N(0, std) weights: d = largest magnitude / 127 */
void pf_synth_q8_0_normal(unsigned char *out, size_t blocks, uint64_t seed, float std) {
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) {
        float v[32], top = 0;
        normals(v, 32, seed, b * 32, std);
        for (int i = 0; i < 32; i++) top = fmaxf(top, fabsf(v[i]));
        uint16_t dh = half_bits(top / 127.0f);
        float d = half_float(dh);
        unsigned char *p = out + 34 * b;
        p[0] = (unsigned char)(dh & 255u); p[1] = (unsigned char)(dh >> 8);
        for (int i = 0; i < 32; i++) p[2 + i] = (unsigned char)(signed char)(d > 0 ? clampi((int)lrintf(v[i] / d), -127, 127) : 0);
    }
}

/* Q2_K super-blocks (16 scale | min << 4 bytes, 64 bytes of 2-bit codes, half d, half dmin) of
 * N(0, std) weights: per group of 16 a step (hi - lo) / 3 and an offset -lo, both in 4 bits. */
void pf_synth_q2k_normal(unsigned char *out, size_t blocks, uint64_t seed, float std) {
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) {
        float v[256], step[16], lowest[16], max_step = 0, max_low = 0;
        normals(v, 256, seed, b * 256, std);
        for (int g = 0; g < 16; g++) {
            float lo = 0, hi = 0;
            for (int i = 0; i < 16; i++) { lo = fminf(lo, v[16 * g + i]); hi = fmaxf(hi, v[16 * g + i]); }
            step[g] = (hi - lo) / 3.0f;
            lowest[g] = -lo;
            max_step = fmaxf(max_step, step[g]);
            max_low = fmaxf(max_low, lowest[g]);
        }
        uint16_t dh = half_bits(max_step / 15.0f), mh = half_bits(max_low / 15.0f);
        float d = half_float(dh), dmin = half_float(mh);
        unsigned char *p = out + 84 * b;
        memset(p, 0, 84);
        for (int g = 0; g < 16; g++) {
            unsigned sc = d > 0 ? (unsigned)clampi((int)lrintf(step[g] / d), 0, 15) : 0;
            unsigned mn = dmin > 0 ? (unsigned)clampi((int)lrintf(lowest[g] / dmin), 0, 15) : 0;
            p[g] = (unsigned char)(sc | (mn << 4));
            float s = d * (float)sc, offset = dmin * (float)mn;
            for (int i = 0; i < 16; i++) {
                int lane = 16 * g + i, q = s > 0 ? clampi((int)lrintf((v[lane] + offset) / s), 0, 3) : 0;
                p[16 + lane / 128 * 32 + lane % 32] |= (unsigned char)(q << (2 * (lane % 128 / 32)));
            }
        }
        p[80] = (unsigned char)(dh & 255u); p[81] = (unsigned char)(dh >> 8);
        p[82] = (unsigned char)(mh & 255u); p[83] = (unsigned char)(mh >> 8);
    }
}

/* MXFP4 blocks (one E8M0 scale byte, 32 E2M1 codes, values 0..15 in the low nibbles) of N(0, std)
 * weights: the scale is the power of two that brings the largest magnitude to at most 6. */
void pf_synth_mxfp4_normal(unsigned char *out, size_t blocks, uint64_t seed, float std) {
    static const float level[8] = {0, .5f, 1, 1.5f, 2, 3, 4, 6};
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < blocks; b++) {
        float v[32], top = 0;
        normals(v, 32, seed, b * 32, std);
        for (int i = 0; i < 32; i++) top = fmaxf(top, fabsf(v[i]));
        int e = top > 0 ? clampi((int)ceilf(log2f(top / 6.0f)) + 127, 1, 252) : 127;
        float scale = ldexpf(1.0f, e - 127);
        unsigned char *p = out + 17 * b;
        memset(p, 0, 17);
        p[0] = (unsigned char)e;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(v[i]) / scale;
            int best = 0;
            for (int c = 1; c < 8; c++) if (fabsf(a - level[c]) < fabsf(a - level[best])) best = c;
            unsigned code = (unsigned)best | (v[i] < 0 ? 8u : 0u);
            p[1 + i % 16] |= (unsigned char)(code << ((i / 16) * 4));
        }
    }
}
