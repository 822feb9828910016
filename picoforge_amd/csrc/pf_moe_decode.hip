// Decode path: 1..4 tokens through one MoE layer as three dependent kernels.
//
//   pf_k_dec_router   router logits (F32 rows) and the shared router's sigmoid
//   pf_k_dec_gate_up  routing (every workgroup repeats it from the logits: candidate
//                     lists by several waves, merged by one), the union of the tokens'
//                     experts, gate/up + SwiGLU once per unique routed expert and for
//                     the shared expert, activations written as FP32 and as digit images
//   pf_k_dec_down     down products of the routed slots and of the shared expert (one
//                     wave each), slot-ordered weighted sum, shared branch added last
//
// A dependent kernel boundary costs about 1.6 us on this GPU when replayed from a
// graph; an in-kernel barrier across its eight L2 domains costs more, so the three
// data dependencies of the block are kernel boundaries.
//
// Arithmetic.  A lane owns 64 consecutive weights of a row (two 32-weight groups:
// one Q4_K nibble pair, two IQ2_XXS groups, two Q8_0 or MXFP4 blocks, a quarter of a
// Q2_K block); the routed gate/up tensors, the routed down tensor and the shared
// expert may each be in a format of their own.  Activations are turned into block
// fixed point once per vector: per 32-group a power-of-two step and, per value, a
// 21-bit integer written as three balanced base-128 digits.  Weight codes are small
// integers in both formats, so the group dot product is three v_dot4_i32_i8 chains
// and exact; the group scales are applied in FP32 afterwards.  The activation error
// is at most 2^-21 of the largest magnitude of its group.
#include "pf_moe_internal.h"
#include "pf_route_device.h"
#include "pf_route_fast.h"
#include "pf_route_fix.h"
#include "pf_upload_addr.h"

#ifdef PF_TIMING
#define STAMP(i) do { if (blockIdx.x == PF_TIMING && threadIdx.x == 0) reinterpret_cast<unsigned long long *>(a.exact_rows + 2)[i] = wall_clock64(); } while (0)
// the fused launch: workgroup b's phase i (eight per workgroup) into the activation rows' buffer, which that launch leaves unused
#define FSTAMP(i) do { if (threadIdx.x == 0) reinterpret_cast<unsigned long long *>(a.act)[8 * blockIdx.x + (i)] = wall_clock64(); } while (0)
#define STAMP_FIRST(i) do { if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.y == 0) reinterpret_cast<unsigned long long *>(a.exact_rows + 2)[i] = wall_clock64(); } while (0)
#else
#define STAMP(i) do {} while (0)
#define FSTAMP(i) do {} while (0)
#define STAMP_FIRST(i) do {} while (0)
#endif
// The unit is compiled four times, once per format combination (PF_DECODE_PART 0..3, see the dispatch
// at the end), so that the combinations' kernels build in parallel; part 0 also holds everything that
// does not depend on the combination.
#ifndef PF_DECODE_PART
#define PF_DECODE_PART 0
#endif
#define SEG_STRIDE 20   // dwords per 64-value segment of a digit plane (16 used): spreads LDS banks

// ---- digit images --------------------------------------------------------------------
// Image of a K-vector: three digit planes of SEG_STRIDE * K/64 dwords, then K/32 group
// steps (float), then K/32 group sums of the integer values.
__host__ __device__ constexpr int image_words(int K) { return 3 * SEG_STRIDE * (K / 64) + 2 * (K / 32); }

struct XSeg {          // one lane's 64 activations
    int d0[16], d1[16], d2[16];
    float step[2];
    int sum[2];
};

__device__ __forceinline__ void xseg_load(XSeg &s, const int *img, int K, int seg) {
    const int plane = SEG_STRIDE * (K / 64);
    const int4 *p0 = reinterpret_cast<const int4 *>(img + SEG_STRIDE * seg);
    const int4 *p1 = reinterpret_cast<const int4 *>(img + plane + SEG_STRIDE * seg);
    const int4 *p2 = reinterpret_cast<const int4 *>(img + 2 * plane + SEG_STRIDE * seg);
#pragma unroll
    for (int m = 0; m < 4; m++) {
        int4 a = p0[m], b = p1[m], c = p2[m];
        s.d0[4 * m] = a.x; s.d0[4 * m + 1] = a.y; s.d0[4 * m + 2] = a.z; s.d0[4 * m + 3] = a.w;
        s.d1[4 * m] = b.x; s.d1[4 * m + 1] = b.y; s.d1[4 * m + 2] = b.z; s.d1[4 * m + 3] = b.w;
        s.d2[4 * m] = c.x; s.d2[4 * m + 1] = c.y; s.d2[4 * m + 2] = c.z; s.d2[4 * m + 3] = c.w;
    }
    const float *steps = reinterpret_cast<const float *>(img + 3 * plane);
    const int *sums = img + 3 * plane + K / 32;
    s.step[0] = steps[2 * seg]; s.step[1] = steps[2 * seg + 1];
    s.sum[0] = sums[2 * seg]; s.sum[1] = sums[2 * seg + 1];
}

__device__ __forceinline__ int dpp_quad_xor1(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true); }
__device__ __forceinline__ int dpp_quad_xor2(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true); }

// power-of-two step for a group whose largest magnitude is m: |v| / step < 2^20
__device__ __forceinline__ void group_step(float m, float &step, float &inv) {
    int e = (__float_as_int(m) >> 23) & 255;
    e = e < 21 ? 21 : e;
    step = __int_as_float((e - 19) << 23);
    inv = __int_as_float((273 - e) << 23);
}

__device__ __forceinline__ void split_digits(int q, int &d0, int &d1, int &d2) {
    d0 = ((q + 64) & 127) - 64;
    const int r = (q - d0) >> 7;
    d1 = ((r + 64) & 127) - 64;
    d2 = (r - d1) >> 7;
}

// The eight values 8j..8j+7 of a K-vector (a, b) into its image; four neighbouring threads form one
// 32-group, so the four threads of a group must all be here.  Returns whether a value is not finite.
__device__ __forceinline__ bool image_chunk(int *img, const float4 a, const float4 b, int j, int K) {
    const int plane = SEG_STRIDE * (K / 64);
    bool bad = false;
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; c++) { m = fmaxf(m, fabsf(v[c])); bad |= !pf_finite(v[c]); }
    m = fmaxf(m, __int_as_float(dpp_quad_xor1(__float_as_int(m))));
    m = fmaxf(m, __int_as_float(dpp_quad_xor2(__float_as_int(m))));
    float step, inv;
    group_step(m, step, inv);
    int w0[2] = {0, 0}, w1[2] = {0, 0}, w2[2] = {0, 0}, sum = 0;
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const int q = __float2int_rn(v[c] * inv);
        sum += q;
        int d0, d1, d2;
        split_digits(q, d0, d1, d2);
        w0[c >> 2] |= (d0 & 255) << (8 * (c & 3));
        w1[c >> 2] |= (d1 & 255) << (8 * (c & 3));
        w2[c >> 2] |= (d2 & 255) << (8 * (c & 3));
    }
    sum += dpp_quad_xor1(sum);
    sum += dpp_quad_xor2(sum);
    const int at = SEG_STRIDE * (j >> 3) + 2 * (j & 7);
    img[at] = w0[0]; img[at + 1] = w0[1];
    img[plane + at] = w1[0]; img[plane + at + 1] = w1[1];
    img[2 * plane + at] = w2[0]; img[2 * plane + at + 1] = w2[1];
    if ((j & 3) == 0) {
        reinterpret_cast<float *>(img + 3 * plane)[j >> 2] = step;
        img[3 * plane + K / 32 + (j >> 2)] = sum;
    }
    return bad;
}

// Threads [first_thread, first_thread + thread_count) of the workgroup: image of src[0..K) (K % 32 == 0).
// Thread j takes the eight values 8j..8j+7, then 8(j + count).. and so on.
__device__ __forceinline__ bool build_image(int *img, const float *src, int K, int first_thread = 0,
                                            int thread_count = 1 << 30) {
    bool bad = false;
    const int j0 = (int)threadIdx.x - first_thread, stride = min(thread_count, (int)blockDim.x - first_thread);
    if (j0 < 0 || j0 >= stride) return false;
    for (int j = j0; j < K / 8; j += stride)
        bad |= image_chunk(img, reinterpret_cast<const float4 *>(src)[2 * j], reinterpret_cast<const float4 *>(src)[2 * j + 1], j, K);
    return bad;
}

// ---- digit images in global memory (kernels whose lanes are weight rows) ------------------------
// Where every lane of a wave is a weight row, the activation digits are the same for the whole wave and
// travel through scalar registers: the image lives in global memory (pf_image2_words), written by the
// kernel before.  PF_IMG_PLANES balanced base-256 digits (signed bytes): the values as integers relative
// to a step per 32-group that puts the group's largest magnitude at 127 * 256^(planes - 1); the rounding
// error is at most 2^-24 of that magnitude with three planes.
#define PF_IMG_TOP (PF_IMG_PLANES == 3 ? 8323072.0f : 32512.0f)   // the integer the group's largest magnitude becomes: 127 * 256^(planes - 1)
__device__ __forceinline__ void group_step2(float m, float &step, float &inv) {
    const bool none = !(m > 1e-30f);   // an all-zero (or vanishing) group
    inv = none ? 0.0f : PF_IMG_TOP / m;
    step = none ? 0.0f : m * (1.0f / PF_IMG_TOP);
}
// balanced base-256 digits of q, lowest first (each in -128..127)
__device__ __forceinline__ void image_digits(int q, int (&d)[PF_IMG_PLANES]) {
#pragma unroll
    for (int p = 0; p + 1 < PF_IMG_PLANES; p++) {
        d[p] = ((q + 128) & 255) - 128;
        q = (q - d[p]) >> 8;
    }
    d[PF_IMG_PLANES - 1] = q;
}
// the integer dot product from its per-plane parts (float: three planes leave 32 bits)
__device__ __forceinline__ float image_value(const int (&part)[PF_IMG_PLANES]) {
    float v = (float)part[PF_IMG_PLANES - 1];
#pragma unroll
    for (int p = PF_IMG_PLANES - 2; p >= 0; p--) v = fmaf(256.0f, v, (float)part[p]);
    return v;
}

// Thread j of a group of four neighbouring lanes: the eight values 8j..8j+7 of a K-vector into its image.
__device__ __forceinline__ bool image2_chunk(uint32_t *img, const float4 a, const float4 b, int j, int K) {
    bool bad = false;
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; c++) { m = fmaxf(m, fabsf(v[c])); bad |= !pf_finite(v[c]); }
    m = fmaxf(m, __int_as_float(dpp_quad_xor1(__float_as_int(m))));
    m = fmaxf(m, __int_as_float(dpp_quad_xor2(__float_as_int(m))));
    float step, inv;
    group_step2(m, step, inv);
    uint32_t w[PF_IMG_PLANES][2] = {};
    int sum = 0;
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const int q = __float2int_rn(v[c] * inv);
        sum += q;
        int d[PF_IMG_PLANES];
        image_digits(q, d);
#pragma unroll
        for (int p = 0; p < PF_IMG_PLANES; p++) w[p][c >> 2] |= (uint32_t)(d[p] & 255) << (8 * (c & 3));
    }
    sum += dpp_quad_xor1(sum);
    sum += dpp_quad_xor2(sum);
    const int g = j >> 2, at = PF_IMG_GROUP * g + 2 * (j & 3);
#pragma unroll
    for (int p = 0; p < PF_IMG_PLANES; p++) { img[at + 8 * p] = w[p][0]; img[at + 8 * p + 1] = w[p][1]; }
    if ((j & 3) == 0) {
        img[PF_IMG_GROUP * (K / 32) + g] = __float_as_uint(step);
        img[(PF_IMG_GROUP + 1) * (K / 32) + g] = (uint32_t)sum;
    }
    return bad;
}

// Lanes 0..31 of a wave, one value each: group g of a K-vector's image.
__device__ __forceinline__ int dpp_row_step(int v, const int which) {
    switch (which) {
    case 0: return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
    case 1: return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    case 2: return __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);   // row_half_mirror
    default: return __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);  // row_mirror
    }
}

__device__ __forceinline__ void image2_group(uint32_t *img, float v, int g, int K, int lane) {   // lanes 32..63 idle along
    float m = fabsf(v);
#pragma unroll
    for (int k = 0; k < 4; k++) m = fmaxf(m, __int_as_float(dpp_row_step(__float_as_int(m), k)));
    m = fmaxf(m, __shfl_xor(m, 16));
    float step, inv;
    group_step2(m, step, inv);
    const int q = __float2int_rn(v * inv);
    int sum = q;
#pragma unroll
    for (int k = 0; k < 4; k++) sum += dpp_row_step(sum, k);
    sum += __shfl_xor(sum, 16);
    int d[PF_IMG_PLANES];
    image_digits(q, d);
    uint8_t *bytes = reinterpret_cast<uint8_t *>(img + PF_IMG_GROUP * g);
    if (lane < 32) {
#pragma unroll
        for (int p = 0; p < PF_IMG_PLANES; p++) bytes[32 * p + lane] = (uint8_t)d[p];
    }
    if (lane == 0) {
        img[PF_IMG_GROUP * (K / 32) + g] = __float_as_uint(step);
        img[(PF_IMG_GROUP + 1) * (K / 32) + g] = (uint32_t)sum;
    }
}

// ---- one lane's 64 weights of a row --------------------------------------------------
template <int FMT> struct WSeg;
template <> struct WSeg<PF_Q4_K> { uint4 hdr, q0, q1; };
template <> struct WSeg<PF_IQ2_XXS> { uint4 p; uint32_t dbits; };

template <int FMT>
__device__ __forceinline__ void wseg_load(WSeg<FMT> &w, const PfKernelArgs &a, int t, size_t e, size_t n, int seg);

// Every loader takes its offsets from pf_segment_spans (pf_decode_addr.h), the function the host-side bounds
// test walks.
__device__ __forceinline__ PfTensorPlace tensor_place(const PfKernelArgs &a, int t) {
    PfTensorPlace p;
    p.row_bytes = a.row_bytes[t]; p.expert_bytes = a.expert_bytes[t]; p.scale_offset = a.scale_offset[t];
    p.bytes = p.gguf_bytes = 0;
    p.n_out = a.n_out[t]; p.blocks_per_row = a.blocks_per_row[t];
    return p;
}

template <>
__device__ __forceinline__ void wseg_load<PF_Q4_K>(WSeg<PF_Q4_K> &w, const PfKernelArgs &a, int t, size_t e, size_t n,
                                                   int seg) {
    PfSpan sp[4];
    pf_segment_spans(PF_Q4_K, tensor_place(a, t), e, n, seg, sp);
    w.hdr = *reinterpret_cast<const uint4 *>(a.w[t] + sp[0].at);
    const uint4 *q = reinterpret_cast<const uint4 *>(a.w[t] + sp[1].at);
    w.q0 = q[0];
    w.q1 = q[1];
}

template <>
__device__ __forceinline__ void wseg_load<PF_IQ2_XXS>(WSeg<PF_IQ2_XXS> &w, const PfKernelArgs &a, int t, size_t e,
                                                      size_t n, int seg) {
    PfSpan sp[4];
    pf_segment_spans(PF_IQ2_XXS, tensor_place(a, t), e, n, seg, sp);
    w.p = *reinterpret_cast<const uint4 *>(a.w[t] + sp[0].at);
    w.dbits = *reinterpret_cast<const uint16_t *>(a.w[t] + sp[1].at);
}

// Q8_0, device layout (32 code bytes per block, half scales apart): a segment is two blocks
template <> struct WSeg<PF_Q8_0> { uint4 q[4]; uint32_t d2; };
template <>
__device__ __forceinline__ void wseg_load<PF_Q8_0>(WSeg<PF_Q8_0> &w, const PfKernelArgs &a, int t, size_t e, size_t n,
                                                   int seg) {
    PfSpan sp[4];
    pf_segment_spans(PF_Q8_0, tensor_place(a, t), e, n, seg, sp);
    const uint4 *row = reinterpret_cast<const uint4 *>(a.w[t] + sp[0].at);
#pragma unroll
    for (int i = 0; i < 4; i++) w.q[i] = row[i];
    w.d2 = *reinterpret_cast<const uint32_t *>(a.w[t] + sp[1].at);
}

// MXFP4, device layout (16 nibble bytes per block, scale bytes apart): a segment is two blocks
template <> struct WSeg<PF_MXFP4> { uint4 q[2]; uint32_t e2; };
template <>
__device__ __forceinline__ void wseg_load<PF_MXFP4>(WSeg<PF_MXFP4> &w, const PfKernelArgs &a, int t, size_t e, size_t n,
                                                    int seg) {
    PfSpan sp[4];
    pf_segment_spans(PF_MXFP4, tensor_place(a, t), e, n, seg, sp);
    const uint4 *row = reinterpret_cast<const uint4 *>(a.w[t] + sp[0].at);
    w.q[0] = row[0];
    w.q[1] = row[1];
    w.e2 = *reinterpret_cast<const uint16_t *>(a.w[t] + sp[1].at);
}

// Q2_K, GGUF bytes (84-byte blocks, 4-byte aligned): a segment is a quarter of a block: 32 code
// bytes read at two bit planes, four scale | min << 4 bytes, the block's d and dmin
template <> struct WSeg<PF_Q2_K> { uint32_t q[8], sm, dd; };
template <>
__device__ __forceinline__ void wseg_load<PF_Q2_K>(WSeg<PF_Q2_K> &w, const PfKernelArgs &a, int t, size_t e, size_t n,
                                                   int seg) {
    PfSpan sp[4];
    pf_segment_spans(PF_Q2_K, tensor_place(a, t), e, n, seg, sp);
    const uint32_t *codes = reinterpret_cast<const uint32_t *>(a.w[t] + sp[0].at);
#pragma unroll
    for (int i = 0; i < 8; i++) w.q[i] = codes[i];
    w.sm = *reinterpret_cast<const uint32_t *>(a.w[t] + sp[1].at);
    w.dd = *reinterpret_cast<const uint32_t *>(a.w[t] + sp[2].at);
}

__device__ __forceinline__ float half_bits(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}

template <int FMT>
__device__ __forceinline__ float wseg_dot(const WSeg<FMT> &w, const XSeg &x, int seg, const uint32_t *tables);

// Q4_K: low nibbles of the 32 bytes are group 2j, high nibbles group 2j+1
template <>
__device__ __forceinline__ float wseg_dot<PF_Q4_K>(const WSeg<PF_Q4_K> &w, const XSeg &x, int seg, const uint32_t *) {
    const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
    int l0 = 0, l1 = 0, l2 = 0, h0 = 0, h1 = 0, h2 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int lo = (int)(q[i] & 0x0F0F0F0Fu), hi = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
        l0 = __builtin_amdgcn_sdot4(lo, x.d0[i], l0, false);
        l1 = __builtin_amdgcn_sdot4(lo, x.d1[i], l1, false);
        l2 = __builtin_amdgcn_sdot4(lo, x.d2[i], l2, false);
        h0 = __builtin_amdgcn_sdot4(hi, x.d0[8 + i], h0, false);
        h1 = __builtin_amdgcn_sdot4(hi, x.d1[8 + i], h1, false);
        h2 = __builtin_amdgcn_sdot4(hi, x.d2[8 + i], h2, false);
    }
    const float tl = (float)(l0 + (l1 << 7) + (l2 << 14)), th = (float)(h0 + (h1 << 7) + (h2 << 14));
    // 6-bit scales and minima of groups 2j, 2j+1 (j = seg % 4) from the 12 packed bytes
    const int j = seg & 3, sh = 16 * (j & 1);
    const uint32_t wa = w.hdr.y >> sh, wb = w.hdr.z >> sh, wc = w.hdr.w >> sh;
    uint32_t s0, m0, s1, m1;
    if (j < 2) {
        s0 = wa & 63u; s1 = (wa >> 8) & 63u; m0 = wb & 63u; m1 = (wb >> 8) & 63u;
    } else {
        s0 = (wc & 15u) | ((wa >> 2) & 48u);
        m0 = ((wc >> 4) & 15u) | ((wb >> 2) & 48u);
        s1 = ((wc >> 8) & 15u) | ((wa >> 10) & 48u);
        m1 = ((wc >> 12) & 15u) | ((wb >> 10) & 48u);
    }
    const float d = half_bits(w.hdr.x & 0xffffu), dmin = half_bits(w.hdr.x >> 16);
    const float lo = x.step[0] * fmaf(d * (float)s0, tl, -(dmin * (float)m0) * (float)x.sum[0]);
    const float hi = x.step[1] * fmaf(d * (float)s1, th, -(dmin * (float)m1) * (float)x.sum[1]);
    return lo + hi;
}

// IQ2_XXS: tables[(g << 4) | s] holds the four signed magnitudes of positions 0..3 of grid
// entry g under sign nibble s; tables[4096 + ...] positions 4..7 (bit 3 = the parity sign).
template <>
__device__ __forceinline__ float wseg_dot<PF_IQ2_XXS>(const WSeg<PF_IQ2_XXS> &w, const XSeg &x, int,
                                                      const uint32_t *tables) {
    float acc[2];
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const uint32_t idx = gg ? w.p.z : w.p.x, word = gg ? w.p.w : w.p.y;
        int a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
        for (int slot = 0; slot < 4; slot++) {
            const uint32_t g = (idx >> (8 * slot)) & 255u, s7 = (word >> (7 * slot)) & 127u;
            const uint32_t par = __popc(s7) & 1u;
            const int ml = (int)tables[(g << 4) | (s7 & 15u)];
            const int mh = (int)tables[4096u + ((g << 4) | (s7 >> 4) | (par << 3))];
            const int m = 8 * gg + 2 * slot;
            a0 = __builtin_amdgcn_sdot4(ml, x.d0[m], a0, false);
            a1 = __builtin_amdgcn_sdot4(ml, x.d1[m], a1, false);
            a2 = __builtin_amdgcn_sdot4(ml, x.d2[m], a2, false);
            a0 = __builtin_amdgcn_sdot4(mh, x.d0[m + 1], a0, false);
            a1 = __builtin_amdgcn_sdot4(mh, x.d1[m + 1], a1, false);
            a2 = __builtin_amdgcn_sdot4(mh, x.d2[m + 1], a2, false);
        }
        acc[gg] = x.step[gg] * (float)(2u * (word >> 28) + 1u) * (float)(a0 + (a1 << 7) + (a2 << 14));
    }
    return half_bits(w.dbits) * 0.125f * (acc[0] + acc[1]);
}

// Q8_0: signed byte codes against the three digit planes.  A group's integer can reach 2^32, so the
// top digit's share is added in float (relative error 2^-24 of the group's partial sum).
template <>
__device__ __forceinline__ float wseg_dot<PF_Q8_0>(const WSeg<PF_Q8_0> &w, const XSeg &x, int, const uint32_t *) {
    float out = 0.0f;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const uint32_t q[8] = {w.q[2 * g].x, w.q[2 * g].y, w.q[2 * g].z, w.q[2 * g].w,
                               w.q[2 * g + 1].x, w.q[2 * g + 1].y, w.q[2 * g + 1].z, w.q[2 * g + 1].w};
        int a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            a0 = __builtin_amdgcn_sdot4((int)q[i], x.d0[8 * g + i], a0, false);
            a1 = __builtin_amdgcn_sdot4((int)q[i], x.d1[8 * g + i], a1, false);
            a2 = __builtin_amdgcn_sdot4((int)q[i], x.d2[8 * g + i], a2, false);
        }
        const float total = (float)(a0 + (a1 << 7)) + 16384.0f * (float)a2;
        out = fmaf(x.step[g] * half_bits((w.d2 >> (16 * g)) & 0xffffu), total, out);
    }
    return out;
}

// MXFP4: four E2M1 codes of a dword as signed bytes holding twice their value (0, 1, 2, 3, 4, 6, 8, 12):
// one byte permute per sign, merged under the sign bits' byte mask
__device__ __forceinline__ int e2m1_twice4(uint32_t nibbles) {
    const uint32_t sel = nibbles & 0x07070707u;
    const uint32_t pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
    const uint32_t neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
    const uint32_t mask = ((nibbles >> 3) & 0x01010101u) * 0xFFu;
    return (int)((neg & mask) | (pos & ~mask));
}

template <>
__device__ __forceinline__ float wseg_dot<PF_MXFP4>(const WSeg<PF_MXFP4> &w, const XSeg &x, int, const uint32_t *) {
    float out = 0.0f;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const uint32_t q[4] = {w.q[g].x, w.q[g].y, w.q[g].z, w.q[g].w};
        int a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int lo = e2m1_twice4(q[i] & 0x0F0F0F0Fu), hi = e2m1_twice4((q[i] >> 4) & 0x0F0F0F0Fu);
            a0 = __builtin_amdgcn_sdot4(lo, x.d0[8 * g + i], a0, false);
            a1 = __builtin_amdgcn_sdot4(lo, x.d1[8 * g + i], a1, false);
            a2 = __builtin_amdgcn_sdot4(lo, x.d2[8 * g + i], a2, false);
            a0 = __builtin_amdgcn_sdot4(hi, x.d0[8 * g + 4 + i], a0, false);
            a1 = __builtin_amdgcn_sdot4(hi, x.d1[8 * g + 4 + i], a1, false);
            a2 = __builtin_amdgcn_sdot4(hi, x.d2[8 * g + 4 + i], a2, false);
        }
        const float scale = 0.5f * pf_e8m0_scale((w.e2 >> (8 * g)) & 255u);   // the integers are twice the values
        out = fmaf(x.step[g] * scale, (float)(a0 + (a1 << 7) + (a2 << 14)), out);
    }
    return out;
}

// Q2_K: group gg of the segment reads bit plane 2 * (seg % 2) + gg of the 32 code bytes; bytes 0..15
// and 16..31 are two sub-groups of 16 with their own scale and minimum, so the sums of the activation
// integers are taken per sub-group here (dot products with ones).
template <>
__device__ __forceinline__ float wseg_dot<PF_Q2_K>(const WSeg<PF_Q2_K> &w, const XSeg &x, int seg, const uint32_t *) {
    const float d = half_bits(w.dd & 0xffffu), dmin = half_bits(w.dd >> 16);
    float out = 0.0f;
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const int shift = 2 * (2 * (seg & 1) + gg);
        float group = 0.0f;
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            int c0 = 0, c1 = 0, c2 = 0, s0 = 0, s1 = 0, s2 = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int codes = (int)((w.q[4 * sub + i] >> shift) & 0x03030303u), m = 8 * gg + 4 * sub + i;
                c0 = __builtin_amdgcn_sdot4(codes, x.d0[m], c0, false);
                c1 = __builtin_amdgcn_sdot4(codes, x.d1[m], c1, false);
                c2 = __builtin_amdgcn_sdot4(codes, x.d2[m], c2, false);
                s0 = __builtin_amdgcn_sdot4(0x01010101, x.d0[m], s0, false);
                s1 = __builtin_amdgcn_sdot4(0x01010101, x.d1[m], s1, false);
                s2 = __builtin_amdgcn_sdot4(0x01010101, x.d2[m], s2, false);
            }
            const uint32_t sm = (w.sm >> (8 * (2 * gg + sub))) & 255u;
            group += fmaf(d * (float)(sm & 15u), (float)(c0 + (c1 << 7) + (c2 << 14)),
                          -(dmin * (float)(sm >> 4)) * (float)(s0 + (s1 << 7) + (s2 << 14)));
        }
        out = fmaf(x.step[gg], group, out);
    }
    return out;
}

// sum over `width` neighbouring lanes (power of two, <= 32); result in the lowest lane of each span
// (width is uniform; the DPP steps leave the span total in every lane of the span)
__device__ __forceinline__ float span_sum(float v, int width) {
    if (width >= 2) v = pf_dpp_add(v, 0);    // quad_perm [1,0,3,2]
    if (width >= 4) v = pf_dpp_add(v, 1);    // quad_perm [2,3,0,1]
    if (width >= 8) v = pf_dpp_add(v, 2);    // row_half_mirror
    if (width >= 16) v = pf_dpp_add(v, 3);   // row_mirror
    if (width >= 32) v += __shfl_xor(v, 16);
    return v;
}

__device__ __forceinline__ void stage_tables(uint32_t *lds, const uint32_t *global) {
    const uint4 *src = reinterpret_cast<const uint4 *>(global);
    uint4 *dst = reinterpret_cast<uint4 *>(lds);
    for (int i = threadIdx.x; i < 2048; i += blockDim.x) dst[i] = src[i];
}

template <int FMT> __host__ __device__ constexpr int table_words() { return FMT == PF_IQ2_XXS ? 8192 : 0; }

// Requests fields of the kernel's argument block now, together.  Left to itself the compiler fetches a field where it
// is first used, behind the wait for the fields before it: several turns to the scalar cache, one after the other,
// before a kernel's first weight bytes are asked for.
// (The fields are inputs of the statement only: as in-out operands they would stay in their registers for certain, but a
// pointer that has passed through the statement is no longer known to point to global memory, and its accesses become
// flat ones.)
template <typename T>
__device__ __forceinline__ void pf_arg_now(const T &field) { asm volatile("" ::"s"(field)); }
__device__ __forceinline__ void pf_args_now() {}
template <typename T, typename... Rest>
__device__ __forceinline__ void pf_args_now(const T &field, const Rest &...rest) {
    pf_arg_now(field);
    pf_args_now(rest...);
}


// ---- kernel 1: router logits -----------------------------------------------------------------
// One F32 row per wave, all tokens: blocks [0, router_blocks) take the experts' rows, the
// last block's first wave the shared router row (its sigmoid scales the shared expert).
#define ROUTER_CHUNKS 10   // 16-byte pieces of a router row per lane: hidden <= 2560
template <int NT>
__global__ void __launch_bounds__(256) pf_k_dec_router(PfKernelArgs a, int router_blocks, int tokens) {
    pf_args_now(a.w[0], a.w[7], a.x, a.x_pitch, a.logits, a.logit_ssq, a.shared_scale, a.ximg, router_blocks, tokens);
    STAMP_FIRST(0);
    const int H = a.hidden, E = a.experts, lane = pf_lane(), wave = threadIdx.x >> 6;
    if ((int)blockIdx.x > router_blocks) {
        // workgroups beyond the router's (launched where the next kernel reads them): the tokens' digit images,
        // 2048 values per workgroup
        const int per_token = (H + 2047) / 2048, q = (int)blockIdx.x - router_blocks - 1;
        const int t = q / per_token, j = (q % per_token) * 256 + (int)threadIdx.x;
        if (blockIdx.y == 0 && t < tokens && j < H / 8) {
            const float4 *row = reinterpret_cast<const float4 *>(a.x + (size_t)t * a.x_pitch);
            image2_chunk(a.ximg + (size_t)t * pf_image2_words(H), row[2 * j], row[2 * j + 1], j, H);
        }
        return;
    }
    // blockIdx.y: the group of NT tokens (more than NT tokens only with the tile-ordered kernels behind this one)
    const int t0 = NT * (int)blockIdx.y, nt = tokens - t0 < NT ? tokens - t0 : NT;
    a.x += (size_t)t0 * a.x_pitch;
    a.logits += (size_t)t0 * E;
    a.logit_ssq += (size_t)t0 * E;
    a.shared_scale += t0;
    const bool gate_row = (int)blockIdx.x == router_blocks;
    // the tag of the forward's activation lines (the launch behind this one, where it takes the whole expert stage)
    if (gate_row && blockIdx.y == 0 && threadIdx.x == 64 && a.fuse_gen) a.fuse_gen[0] = a.fuse_gen[0] + 1u;
    const int e = blockIdx.x * 4 + wave;
    if (gate_row ? wave != 0 : e >= E) return;
    const float4 *w = reinterpret_cast<const float4 *>(gate_row ? a.w[7] : a.w[0] + (size_t)e * H * 4);
    float acc[NT], sq[NT];
    bool bad = false;
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = sq[t] = 0.0f;
    // the whole row (hidden <= 2560: ten 16-byte chunks per lane) is requested before any use
    float4 wv[ROUTER_CHUNKS];
#pragma unroll
    for (int c = 0; c < ROUTER_CHUNKS; c++) {
        const int i = lane + PF_WAVE * c;
        wv[c] = i < H / 4 ? w[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
        float4 xv[ROUTER_CHUNKS];
#pragma unroll
        for (int c = 0; c < ROUTER_CHUNKS; c++) {
            const int i = lane + PF_WAVE * c;
            xv[c] = i < H / 4 && t < nt ? reinterpret_cast<const float4 *>(a.x + (size_t)t * a.x_pitch)[i]
                                        : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int c = 0; c < ROUTER_CHUNKS; c++) {
            const float p0 = wv[c].x * xv[c].x, p1 = wv[c].y * xv[c].y, p2 = wv[c].z * xv[c].z, p3 = wv[c].w * xv[c].w;
            acc[t] += (p0 + p1) + (p2 + p3);
            sq[t] = fmaf(p0, p0, fmaf(p1, p1, fmaf(p2, p2, fmaf(p3, p3, sq[t]))));
        }
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const float z = pf_wave_sum(acc[t]), s2 = pf_wave_sum(sq[t]);
        if (lane == 0 && t < nt) {
            // a nonfinite activation makes every product with it nonfinite (0 * inf is NaN), and a sum with a nonfinite
            // term stays nonfinite: the rows are not looked through element by element
            if (!pf_finite(z)) bad = true;
            if (gate_row) {
                a.shared_scale[t] = pf_sigmoid(z);
            } else {
                a.logits[(size_t)t * E + e] = z;
                a.logit_ssq[(size_t)t * E + e] = s2;
            }
        }
    }
    if (__any(bad) && lane == 0) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
}

// Warms the L2 of this workgroup's XCD with the down-projection rows the next kernel will read
// there.  Workgroups go to the eight XCDs round robin by index, in this kernel and in the next;
// the next kernel's workgroup nb (rows [nb * rows_per_block, +rows_per_block) of every slot)
// therefore runs on XCD nb % 8.  Run by workgroups that have no other work (compute units the
// gate/up tiles leave idle): workgroup `order` of the `per_xcd` on its XCD takes every per_xcd-th
// (slot, row block) item of that XCD; slot `uniques` is the shared expert.  The loaded values
// are not used: a wrong guess about the placement costs time, not results.
__device__ __forceinline__ void prefetch_down(const PfKernelArgs &a, const uint32_t *uniq, int uniques, int order,
                                              int per_xcd, int rows_per_block, int row_blocks) {
    const int xcd = blockIdx.x % 8, per_slot = row_blocks / 8, items = (uniques + 1) * per_slot;
    const int mine = (items - order + per_xcd - 1) / per_xcd;
    const size_t widest = (size_t)rows_per_block * max(a.row_bytes[3], a.row_bytes[6]);
    const int lines = (int)((widest + 127) / 128) + 1;   // the last item: the rows' scales, where they are stored apart
    uint32_t sink = 0;
    for (int i = threadIdx.x; i < mine * lines; i += blockDim.x) {
        const int item = order + per_xcd * (i / lines), l = i % lines;
        const int slot = item / per_slot, nb = xcd + 8 * (item % per_slot);
        const int tensor = slot == uniques ? 6 : 3;
        const size_t e = slot == uniques ? 0 : uniq[slot], row0 = (size_t)nb * rows_per_block;
        if (e >= (size_t)a.experts) continue;
        PfSpan sp;
        if (!pf_warm_span(a.type[tensor], tensor_place(a, tensor), e, row0, rows_per_block, l, lines, &sp)) continue;
        sink |= *reinterpret_cast<const volatile uint32_t *>(a.w[tensor] + sp.at);
    }
    if (sink == 0x9e3779b9u && a.hidden < 0) atomicOr(a.error_word, 0u);   // keeps the loads; never true
}

// ---- kernel 2: routing, expert union, gate/up + SwiGLU of the routed and the shared expert ------
struct RouteLds {
    uint32_t ids[64];        // [token][slot]
    float weights[64];
    uint32_t uniq[64];       // unique experts in first-use order
    uint32_t pair_slot[64];  // pair -> index into uniq
    uint32_t mask[64];       // unique -> bit t set when token t uses it
    uint32_t count, close_mask, bad;
    uint32_t close[PF_DECODE_MAX_TOKENS], nonfinite[PF_DECODE_MAX_TOKENS];
    PfRouteCands cands[PF_DECODE_MAX_TOKENS];
};

__device__ __forceinline__ float *scratch_of(int *images, int words) { return reinterpret_cast<float *>(images + words); }

// Entered by the whole block after the fast routing: reference-order routing of the
// ambiguous tokens (rare), then the union of the tokens' experts.  Ends with a block barrier.
template <int NT>
__device__ __forceinline__ void route_finish(const PfKernelArgs &a, RouteLds *R, float *scratch) {
    const int lane = pf_lane(), wave = threadIdx.x >> 6, E = a.experts, K = a.top_k;
    uint32_t close = 0, bad = 0;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        close |= R->close[t] << t;
        bad |= R->nonfinite[t];
    }
    if (close) {
        const int H = a.hidden;
        float *xs = scratch, *z = xs + H, *p = z + E, *q = p + E;
        for (int t = 0; t < NT; t++) {
            if (!((close >> t) & 1u)) continue;
            for (int k = threadIdx.x; k < H; k += blockDim.x) xs[k] = a.x[(size_t)t * a.x_pitch + k];
            __syncthreads();
            for (int e = threadIdx.x; e < E; e += blockDim.x)
                z[e] = pf_serial_logit(reinterpret_cast<const float *>(a.w[0]) + (size_t)e * H, xs, H);
            __syncthreads();
            if (wave == 0) pf_route_exact_wave(z, p, q, E, K, a.norm_topk != 0, R->ids + t * K, R->weights + t * K, lane);
            __syncthreads();
        }
    }
    if (wave == 0) {
        const int P = NT * K;
        if (NT == 1) {
            if (lane < P) { R->uniq[lane] = R->ids[lane]; R->pair_slot[lane] = lane; R->mask[lane] = 1u; }
            if (lane == 0) R->count = P;
        } else {
            // first-use order: pair p is a first use when no earlier pair names its expert
            const uint32_t id = lane < P ? R->ids[lane] : 0xffffffffu;
            int first_at = lane;
            uint32_t mask = 0;
            for (int q = P - 1; q >= 0; q--) {
                if (R->ids[q] == id) { first_at = q; mask |= 1u << (q / K); }
            }
            const bool first = lane < P && first_at == lane;
            const unsigned long long firsts = __ballot(first);
            const uint32_t slot = __popcll(firsts & ((1ull << first_at) - 1ull));
            if (lane < P) R->pair_slot[lane] = slot;
            if (first) { R->uniq[slot] = id; R->mask[slot] = mask; }
            if (lane == 0) R->count = __popcll(firsts);
        }
        if (lane == 0) { R->close_mask = close; R->bad = bad; }
    }
    __syncthreads();
}

// 1024 threads.  Routed block b: unique slot b / tiles, units [tile * (b % tiles), +tile) of
// that expert (tile = 16 or 32); shared blocks follow.  A wave owns tile / 16 units (a unit =
// gate row + up row: lower half-wave the gate rows, upper half-wave the up rows) and writes its
// activations itself, so no wave waits for another after the routing.
// One tile's rows against the tokens' images, the part of kernel 2 that depends on the tensors'
// format, in three steps: the weights requested, the products, the activations stored.
struct TilePlace {       // where this lane's rows sit in the tile
    int LPR, RPH, half, seg, r, steps, unit0;
    bool second, idle;
};

__device__ __forceinline__ TilePlace tile_place(int H, int tile, int spl) {
    TilePlace p;
    const int lane = pf_lane(), wave = threadIdx.x >> 6;
    p.LPR = row_lanes(H);
    p.RPH = 32 / p.LPR;
    p.half = lane >> 5;
    p.seg = lane & (p.LPR - 1);
    p.r = (lane & 31) / p.LPR;
    p.second = spl > 1 && p.seg + p.LPR < H / 64;   // this lane also holds segment seg + LPR of its row
    // the tile's units over 16 waves: RPH per wave step, one or two steps
    const int per_wave = max(p.RPH, tile / 16);
    p.steps = per_wave / p.RPH;
    p.unit0 = wave * per_wave;
    p.idle = p.unit0 >= tile;
    return p;
}

template <int FMT, int SPL> struct TileRows { WSeg<FMT> w[2][SPL]; };

template <int FMT, int SPL>
__device__ __forceinline__ void tile_load(TileRows<FMT, SPL> &rows, const TilePlace &p, const PfKernelArgs &a, int gate_tensor,
                                          uint32_t e, int n0) {
    if (p.idle) return;
#pragma unroll
    for (int st = 0; st < 2; st++) {
        if (st >= p.steps) break;
        wseg_load<FMT>(rows.w[st][0], a, gate_tensor + p.half, e, n0 + p.unit0 + st * p.RPH + p.r, p.seg);
        if (SPL > 1 && p.second)
            wseg_load<FMT>(rows.w[st][SPL - 1], a, gate_tensor + p.half, e, n0 + p.unit0 + st * p.RPH + p.r, p.seg + p.LPR);
    }
}

// act[t][st]: SwiGLU of unit unit0 + st * RPH + r for token t, valid in the lanes with half == 0 and seg == 0
template <int FMT, int NT, int SPL>
__device__ __forceinline__ void tile_dot(const TileRows<FMT, SPL> &rows, const TilePlace &p, const int *images,
                                         const uint32_t *tables, int W, int H, uint32_t mask, float (&act)[NT][2]) {
    const int lane = pf_lane();
#pragma unroll
    for (int t = 0; t < NT; t++) {
        act[t][0] = act[t][1] = 0.0f;
        if (p.idle || !((mask >> t) & 1u)) continue;
        XSeg x;
        xseg_load(x, images + t * W, H, p.seg);
        float dot[2];
#pragma unroll
        for (int st = 0; st < 2; st++) dot[st] = st < p.steps ? wseg_dot<FMT>(rows.w[st][0], x, p.seg, tables) : 0.0f;
        if (SPL > 1) __builtin_amdgcn_sched_barrier(0);   // the second segment's digits reuse the first's registers
        if (SPL > 1 && p.second) {
            xseg_load(x, images + t * W, H, p.seg + p.LPR);
#pragma unroll
            for (int st = 0; st < 2; st++)
                if (st < p.steps) dot[st] += wseg_dot<FMT>(rows.w[st][SPL - 1], x, p.seg + p.LPR, tables);
        }
#pragma unroll
        for (int st = 0; st < 2; st++) {
            if (st >= p.steps) break;
            const float v = span_sum(dot[st], p.LPR);
            const float up = __shfl(v, (lane & 31) + 32);
            act[t][st] = pf_silu(v) * up;
        }
    }
}

template <int NT>
__device__ __forceinline__ void tile_store(const float (&act)[NT][2], const TilePlace &p, const PfKernelArgs &a, int I, uint32_t mask,
                                           int u, int n0, bool shared) {
    if (p.idle || p.half != 0 || p.seg != 0) return;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        if (!((mask >> t) & 1u)) continue;
#pragma unroll
        for (int st = 0; st < 2; st++) {
            if (st >= p.steps) break;
            const int unit = p.unit0 + st * p.RPH + p.r;
            if (!pf_finite(act[t][st])) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
            if (shared) a.shared_act[(size_t)t * I + n0 + unit] = act[t][st];
            else a.act[((size_t)u * NT + t) * I + n0 + unit] = act[t][st];
        }
    }
}

template <int FMT, int NT, int SPL>
__device__ __forceinline__ void gate_up_tile(const PfKernelArgs &a, const int *images, const uint32_t *tables, int W, int H,
                                             int I, int gate_tensor, uint32_t e, uint32_t mask, int u, int n0, int tile,
                                             bool shared) {
    const TilePlace p = tile_place(H, tile, SPL);
    if (p.idle) return;
    TileRows<FMT, SPL> rows;
    tile_load<FMT, SPL>(rows, p, a, gate_tensor, e, n0);
    float act[NT][2];
    tile_dot<FMT, NT, SPL>(rows, p, images, tables, W, H, mask, act);
    tile_store<NT>(act, p, a, I, mask, u, n0, shared);
}

// FMT: format of the routed gate and up tensors; FMTS: of the shared expert's.
template <int FMT, int FMTS, int NT, int NPL, int SPL>
__global__ void __launch_bounds__(1024) pf_k_dec_gate_up(PfKernelArgs a, int routed_blocks, int shared_blocks, int parts, int chunk, int tile,
                                                         int mode) {
    extern __shared__ int lds[];
    __shared__ RouteLds R;
    const int H = a.hidden, K = a.top_k, E = a.experts, lane = pf_lane(), wave = threadIdx.x >> 6;
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    constexpr bool TABLES = FMT == PF_IQ2_XXS || FMTS == PF_IQ2_XXS;
    int *images = lds + (TABLES ? 8192 : 0);
    const int W = image_words(H), P = NT * K;
    const bool prefetcher = (int)blockIdx.x >= routed_blocks + shared_blocks;   // no tile: warms the L2 for the next kernel
    const bool shared = (int)blockIdx.x >= routed_blocks && !prefetcher;
    STAMP(0);
    if (TABLES) stage_tables(tables, a.iq2_signed);
    const int rounds = K + 1;
    // mode 0: every workgroup routes; 1: this launch only routes and publishes (one workgroup);
    // 2: the routes were published by an earlier launch
    if (!shared && mode != 2 && wave < parts * NT) {
        const int t = wave / parts;
        pf_route_stage1<NPL>(a.logits + (size_t)t * E, a.logit_ssq + (size_t)t * E, E, wave % parts, chunk, rounds,
                             a.norm_topk != 0, &R.cands[t], lane);
    }
    STAMP(1);
    for (int t = 0; t < NT; t++) build_image(images + t * W, a.x + (size_t)t * a.x_pitch, H, 768, 256);
    __syncthreads();
    STAMP(2);
    int u, n0, I, gate_tensor;
    uint32_t e, mask;
    if (shared) {
        u = P; n0 = tile * (blockIdx.x - routed_blocks); I = a.shared_inter; gate_tensor = 4;
        e = 0; mask = (1u << NT) - 1u;
    } else if (mode == 2) {
        const int U = (int)a.uniq[0];
        I = a.inter; gate_tensor = 1;
        const int tiles = I / tile;
        u = blockIdx.x / tiles; n0 = tile * (blockIdx.x % tiles);
        if (u >= U) return;
        e = a.uniq[1 + u]; mask = a.uniq[1 + 2 * P + u];
        if (e >= (uint32_t)E) {   // only reachable with nonfinite logits
            if (threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
            return;
        }
    } else {
        if (wave < NT) {
            PfRouteResult r = pf_route_stage2(&R.cands[wave], parts, K, rounds, a.norm_topk != 0, H, lane);
            if (lane < K) { R.ids[wave * K + lane] = r.id; R.weights[wave * K + lane] = r.weight; }
            if (lane == 0) { R.close[wave] = r.close ? 1u : 0u; R.nonfinite[wave] = r.bad ? 1u : 0u; }
        }
        __syncthreads();
        STAMP(3);
        route_finish<NT>(a, &R, reinterpret_cast<float *>(images + NT * W));
        const int U = R.count;
        if (blockIdx.x == 0) {
            // publish the routes and the union for the next kernel and the caller
            for (int p = threadIdx.x; p < P; p += blockDim.x) {
                a.ids[p] = R.ids[p];
                a.route_weights[p] = R.weights[p];
                a.uniq[1 + p] = p < U ? R.uniq[p] : 0u;
                a.uniq[1 + P + p] = R.pair_slot[p];
                a.uniq[1 + 2 * P + p] = p < U ? R.mask[p] : 0u;
            }
            if (threadIdx.x == 0) {
                a.uniq[0] = U;
                if (R.bad) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
                if (R.close_mask) atomicAdd(a.exact_rows, __popc(R.close_mask));
            }
        }
        if (mode == 1) return;
        if (prefetcher) {
            const int rows_next = down_block_rows(H, a.inter), first = routed_blocks + shared_blocks;
            prefetch_down(a, R.uniq, U, ((int)blockIdx.x - first) / 8, ((int)gridDim.x - first) / 8, rows_next,
                               (H + rows_next - 1) / rows_next);
            return;
        }
        I = a.inter; gate_tensor = 1;
        const int tiles = I / tile;
        u = blockIdx.x / tiles; n0 = tile * (blockIdx.x % tiles);
        if (u >= U) return;
        e = R.uniq[u]; mask = R.mask[u];
        if (e >= (uint32_t)E) {   // only reachable with nonfinite logits
            if (threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
            return;
        }
    }
    STAMP(4);
    if (shared) gate_up_tile<FMTS, NT, SPL>(a, images, tables, W, H, I, gate_tensor, e, mask, u, n0, tile, true);
    else gate_up_tile<FMT, NT, SPL>(a, images, tables, W, H, I, gate_tensor, e, mask, u, n0, tile, false);
    STAMP(5);
}

// ---- kernel 2, one token, Q4_K tensors in tile order ---------------------------------------------
// The tile-ordered copy of a Q4_K tensor (pf_k_q4k_tile: per 32-row tile and 256-block the 32 headers,
// then per 64-weight run the 16-byte halves 0 of the 32 rows and the halves 1) puts the same piece of
// 32 consecutive rows into 512 consecutive bytes, so here a lane is a weight row: lanes 0..31 the
// tile's gate rows, 32..63 its up rows, and a wave takes half a 256-block (four 32-groups) of all of
// them.  Every lane of the wave then meets the same activations: their digits come from the token's
// digit image in global memory through scalar loads and enter the dot products as scalar
// operands -- no LDS image, no reduction across lanes.  The waves' partial sums meet in LDS and are
// added in a fixed order.  Routing as in pf_k_dec_gate_up1.
typedef const __attribute__((address_space(4))) uint32_t *PfScalarWords;   // read through the scalar cache

template <int FMT> struct TileItem;
template <> struct TileItem<PF_Q4_K> { uint4 hdr, piece[2]; };   // a row's header and the two halves of one 64-weight run
template <> struct TileItem<PF_IQ2_XXS> { uint4 piece; uint32_t dbits; };   // two 32-groups (indices, sign/scale word) and the block's half scale
template <> struct TileItem<PF_Q8_0> { uint4 q[4]; uint32_t d2; };   // two blocks: 64 code bytes and their two half scales
typedef TileItem<PF_Q4_K> Q4TileItem;

template <int FMT> struct TileGeometryHost { static const uint8_t *tensor(const PfKernelArgs &, int) { return nullptr; } };
template <> struct TileGeometryHost<PF_Q4_K> { static const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wt[t]; } };
template <> struct TileGeometryHost<PF_IQ2_XXS> { static const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wi[t]; } };
template <> struct TileGeometryHost<PF_Q8_0> { static const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wq[t]; } };
template <int FMT> struct TileGeometry;
template <> struct TileGeometry<PF_Q4_K> {
    static __device__ __forceinline__ size_t expert_bytes(const PfKernelArgs &a, int t) { return a.expert_bytes[t]; }
    static __device__ __forceinline__ size_t chunk_at(int row_tile, int kblocks, int kb) { return pf_q4t_chunk_at(0, 0, row_tile, kblocks, kb); }
    static __device__ __forceinline__ const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wt[t]; }
};
template <> struct TileGeometry<PF_IQ2_XXS> {
    static __device__ __forceinline__ size_t expert_bytes(const PfKernelArgs &a, int t) { return pf_i2t_expert_bytes(a.n_out[t], a.blocks_per_row[t]); }
    static __device__ __forceinline__ size_t chunk_at(int row_tile, int kblocks, int kb) { return pf_i2t_chunk_at(0, 0, row_tile, kblocks, kb); }
    static __device__ __forceinline__ const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wi[t]; }
};

template <> struct TileGeometry<PF_Q8_0> {   // one chunk per 64-weight run: a 256-block is four of them
    static __device__ __forceinline__ size_t expert_bytes(const PfKernelArgs &a, int t) { return pf_q8t_expert_bytes(a.n_out[t], a.blocks_per_row[t] / 2); }
    static __device__ __forceinline__ size_t chunk_at(int row_tile, int kblocks, int kb) { return pf_q8t_chunk_at(0, 0, row_tile, 4 * kblocks, 4 * kb); }
    static __device__ __forceinline__ const uint8_t *tensor(const PfKernelArgs &a, int t) { return a.wq[t]; }
};

__device__ __forceinline__ void q4t_load(TileItem<PF_Q8_0> &w, const uint8_t *chunk, int row, int run) {
    const uint8_t *mine = chunk + (size_t)run * PF_I2T_CHUNK;
#pragma unroll
    for (int p = 0; p < 4; p++) w.q[p] = *reinterpret_cast<const uint4 *>(mine + pf_q8t_piece_at(p, row));
    w.d2 = *reinterpret_cast<const uint32_t *>(mine + pf_q8t_scales_at(row));
}
__device__ __forceinline__ void q4t_load(TileItem<PF_Q4_K> &w, const uint8_t *chunk, int row, int run) {
    w.hdr = *reinterpret_cast<const uint4 *>(chunk + pf_q4t_header_at(row));
    w.piece[0] = *reinterpret_cast<const uint4 *>(chunk + pf_q4t_piece_at(run, 0, row));
    w.piece[1] = *reinterpret_cast<const uint4 *>(chunk + pf_q4t_piece_at(run, 1, row));
}
__device__ __forceinline__ void q4t_load(TileItem<PF_IQ2_XXS> &w, const uint8_t *chunk, int row, int run) {
    w.piece = *reinterpret_cast<const uint4 *>(chunk + pf_i2t_piece_at(run, row));
    w.dbits = *reinterpret_cast<const uint16_t *>(chunk + pf_i2t_scale_at(row));
}

// groups 2 * run, 2 * run + 1 of the row's block (low and high nibbles of the run's bytes) against the image's digits,
// steps and sums of the same two groups (uniform pointers)
__device__ __forceinline__ float q4t_dot(const Q4TileItem &w, PfScalarWords digits, PfScalarWords steps, PfScalarWords sums, int run,
                                         const uint32_t *) {
    // the two groups' 6-bit scales and minima (src/qwen4_packed.c:89-90): bytes 2 * run, 2 * run + 1 of the packed twelve
    uint32_t sc2, mn2;
    if (run < 2) {
        sc2 = (w.hdr.y >> (16 * run)) & 0x3F3Fu;
        mn2 = (w.hdr.z >> (16 * run)) & 0x3F3Fu;
    } else {
        const int sh = 16 * (run - 2);
        sc2 = ((w.hdr.w >> sh) & 0x0F0Fu) | (((w.hdr.y >> sh) >> 2) & 0x3030u);
        mn2 = (((w.hdr.w >> sh) >> 4) & 0x0F0Fu) | (((w.hdr.z >> sh) >> 2) & 0x3030u);
    }
    const float d = half_bits(w.hdr.x & 0xffffu), dmin = half_bits(w.hdr.x >> 16);
    int lo_part[PF_IMG_PLANES] = {}, hi_part[PF_IMG_PLANES] = {};
    PfScalarWords even = digits, odd = digits + PF_IMG_GROUP;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const uint32_t q[4] = {w.piece[h].x, w.piece[h].y, w.piece[h].z, w.piece[h].w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int lo = (int)(q[i] & 0x0F0F0F0Fu), hi = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) {
                lo_part[p] = __builtin_amdgcn_sdot4(lo, (int)even[8 * p + 4 * h + i], lo_part[p], false);
                hi_part[p] = __builtin_amdgcn_sdot4(hi, (int)odd[8 * p + 4 * h + i], hi_part[p], false);
            }
        }
    }
    const float s0 = (float)(sc2 & 255u), m0 = (float)(mn2 & 255u), s1 = (float)(sc2 >> 8), m1 = (float)(mn2 >> 8);
    const float t0 = fmaf(d * s0, image_value(lo_part), -(dmin * m0) * (float)(int)sums[0]);
    const float t1 = fmaf(d * s1, image_value(hi_part), -(dmin * m1) * (float)(int)sums[1]);
    return fmaf(__uint_as_float(steps[0]), t0, __uint_as_float(steps[1]) * t1);
}

// IQ2_XXS: the run's two 32-groups; tables as in wseg_dot<PF_IQ2_XXS> (LDS: four signed magnitudes per grid entry and
// sign nibble); the digits as scalar operands
__device__ __forceinline__ float q4t_dot(const TileItem<PF_IQ2_XXS> &w, PfScalarWords digits, PfScalarWords steps, PfScalarWords sums, int,
                                         const uint32_t *tables) {
    (void)sums;
    float acc[2];
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const uint32_t idx = gg ? w.piece.z : w.piece.x, word = gg ? w.piece.w : w.piece.y;
        PfScalarWords dg = digits + PF_IMG_GROUP * gg;
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int slot = 0; slot < 4; slot++) {
            const uint32_t g = (idx >> (8 * slot)) & 255u, s7 = (word >> (7 * slot)) & 127u;
            const uint32_t par = __popc(s7) & 1u;
            const int ml = (int)tables[(g << 4) | (s7 & 15u)];
            const int mh = (int)tables[4096u + ((g << 4) | (s7 >> 4) | (par << 3))];
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) {
                part[p] = __builtin_amdgcn_sdot4(ml, (int)dg[8 * p + 2 * slot], part[p], false);
                part[p] = __builtin_amdgcn_sdot4(mh, (int)dg[8 * p + 2 * slot + 1], part[p], false);
            }
        }
        acc[gg] = __uint_as_float(steps[gg]) * (float)(2u * (word >> 28) + 1u) * image_value(part);
    }
    return half_bits(w.dbits) * 0.125f * (acc[0] + acc[1]);
}

// Q8_0: the run's two blocks of 32 signed codes against the digit planes
__device__ __forceinline__ float q4t_dot(const TileItem<PF_Q8_0> &w, PfScalarWords digits, PfScalarWords steps, PfScalarWords sums, int,
                                         const uint32_t *) {
    (void)sums;
    float acc[2];
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const uint32_t q[8] = {w.q[2 * gg].x, w.q[2 * gg].y, w.q[2 * gg].z, w.q[2 * gg].w,
                               w.q[2 * gg + 1].x, w.q[2 * gg + 1].y, w.q[2 * gg + 1].z, w.q[2 * gg + 1].w};
        PfScalarWords dg = digits + PF_IMG_GROUP * gg;
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) part[p] = __builtin_amdgcn_sdot4((int)q[i], (int)dg[8 * p + i], part[p], false);
        }
        const float d = half_bits(gg ? w.d2 >> 16 : w.d2 & 0xffffu);
        acc[gg] = __uint_as_float(steps[gg]) * d * image_value(part);
    }
    return acc[0] + acc[1];
}

// The tile's rows against the token: the 64-weight runs of all the rows go round the waves 1..15 (wave 0
// routes); a wave adds up its runs and leaves one partial sum per lane in LDS: partial[wave - 1][64].
#define Q4T_ITEMS 3   // run items a wave can hold: hidden <= 2816
struct Q4TilePlan {   // what does not depend on the expert: set up before the expert is known
    const uint8_t *base;    // this lane's tensor (gate or up) at the tile's first 256-block, expert 0
    size_t expert_bytes;
    int row, kblocks, items, groups;
};

template <int FMT>
__device__ __forceinline__ Q4TilePlan q4t_plan(const PfKernelArgs &a, bool shared, int n0) {
    Q4TilePlan p;
    const int lane = pf_lane();
    p.row = lane & 31;
    p.kblocks = a.hidden / 256;
    p.items = 4 * p.kblocks;
    p.groups = a.hidden / 32;
    // the two tensors by scalar selects and one per-lane choice (an index computed per lane would fetch the pointer
    // from the argument block through the vector memory path, a round trip before the first weight request)
    typedef TileGeometry<FMT> G;
    const bool up = lane >= 32;
    const uint8_t *gate_w = shared ? G::tensor(a, 4) : G::tensor(a, 1), *up_w = shared ? G::tensor(a, 5) : G::tensor(a, 2);
    const size_t gate_bytes = shared ? G::expert_bytes(a, 4) : G::expert_bytes(a, 1);
    const size_t up_bytes = shared ? G::expert_bytes(a, 5) : G::expert_bytes(a, 2);
    p.base = (up ? up_w : gate_w) + G::chunk_at(n0 / 32, p.kblocks, 0);
    p.expert_bytes = up ? up_bytes : gate_bytes;
    return p;
}

template <int FMT>
__device__ __forceinline__ void q4t_tile(const PfKernelArgs &a, const Q4TilePlan &p, float *partial, const uint32_t *tables,
                                         uint32_t e, int wave) {
    if (wave == 0) return;
    const int lane = pf_lane();
    const uint8_t *tile = p.base + (size_t)e * p.expert_bytes;
    const PfScalarWords image = (PfScalarWords)(uintptr_t)a.ximg;
    TileItem<FMT> w[Q4T_ITEMS];
#pragma unroll
    for (int k = 0; k < Q4T_ITEMS; k++) {
        const int it = wave - 1 + 15 * k;
        if (it < p.items) q4t_load(w[k], tile + TileGeometry<FMT>::chunk_at(0, p.kblocks, it >> 2), p.row, it & 3);
    }
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < Q4T_ITEMS; k++) {
        const int it = wave - 1 + 15 * k;
        if (it < p.items) {
            const int g = 2 * it;   // the run's first group within the row
            total += q4t_dot(w[k], image + PF_IMG_GROUP * g, image + PF_IMG_GROUP * p.groups + g, image + (PF_IMG_GROUP + 1) * p.groups + g,
                             it & 3, tables);
        }
    }
    partial[(wave - 1) * 64 + lane] = total;
}

// The kernels below take one token per value of blockIdx.y: the argument block's per-token pointers moved to token t
// (the output row stays indexed by the token: the output helpers take it as an argument).
__device__ __forceinline__ void q4t_at_token(PfKernelArgs &a, int t) {
    const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
    a.x += (size_t)t * a.x_pitch;
    a.logits += (size_t)t * a.experts;
    a.logit_ssq += (size_t)t * a.experts;
    a.ids += (size_t)t * a.top_k;
    a.route_weights += (size_t)t * a.top_k;
    if (a.slots) a.slots += (size_t)t * a.top_k;
    a.act += (size_t)t * a.top_k * a.inter;
    a.shared_act += (size_t)t * a.shared_inter;
    a.shared_scale += t;
    a.ximg += (size_t)t * pf_image2_words(a.hidden);
    a.aimg += (size_t)t * (a.top_k + 1) * pf_image2_words(widest);
}

// The workgroup sums the doubtful experts again in the reference's order, a wave each (pf_route_fix.h).  Not inlined:
// the rare path's registers (a router row's products) must not weigh on the kernel's; the LDS is named here again so
// that its accesses stay LDS instructions.
template <int NPL>
__device__ __forceinline__ void q4t_route_fix(const float *router, const float *x, const float *logits, const float *ssq, int E,
                                                        int K, bool norm, int H, int scratch_at, RouteLds *R) {
    extern __shared__ int lds[];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = pf_lane();
    const int how = pf_route_fix_block<NPL>(router, x, logits, ssq, E, K, norm, H, reinterpret_cast<float *>(lds) + scratch_at, R->ids,
                                            R->weights, wave, lane);
    if (threadIdx.x == 0) { R->close_mask = (uint32_t)how; R->bad = R->nonfinite[0]; }
    __syncthreads();
}

// FMT: format of the routed gate and up tensors, FMTS: of the shared expert's (the same, or the profiles' Q8_0);
// POOL: the routed tensors sit in pool slots (expert streaming)
template <int NPL, int FMT, int FMTS, bool POOL>
__device__ __forceinline__ void q4t_gate_up(PfKernelArgs &a, int routed_blocks) {
    extern __shared__ int lds[];
    __shared__ RouteLds R;
    __shared__ uint32_t early_expert;
    q4t_at_token(a, (int)blockIdx.y);
    const int H = a.hidden, K = a.top_k, E = a.experts, lane = pf_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    // IQ2_XXS: the signed-magnitude tables first (32 KB, staged by every wave but the routing one)
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    if (FMT == PF_IQ2_XXS && wave != 0) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.iq2_signed);
        for (int i = (int)threadIdx.x - 64; i < 2048; i += 960) reinterpret_cast<uint4 *>(tables)[i] = src[i];
    }
    float *partial = reinterpret_cast<float *>(lds + table_words<FMT>());   // [15 waves][64 lanes]
    float *scratch = partial + 15 * 64;   // the serial-order routing's arrays
    const bool shared = (int)blockIdx.x >= routed_blocks;
    const int tiles = a.inter / 32;
    const int u = shared ? K : (int)blockIdx.x / tiles;
    const int n0 = 32 * (shared ? (int)blockIdx.x - routed_blocks : (int)blockIdx.x % tiles);
    const bool norm = a.norm_topk != 0;
    const int rounds = K + 1;   // top_k < experts on this path
    float v[NPL], s2[NPL], total = 0.0f, top_all = 0.0f;
    PfTopk<NPL> top;
    uint32_t my_key = 0;
    bool bad = false;
    if (wave == 0 && !shared) {
        pf_load_row<NPL>(a.logits, E, lane, -INFINITY, v);
        pf_load_row<NPL>(a.logit_ssq, E, lane, 0.0f, s2);
#pragma unroll
        for (int j = 0; j < NPL; j++) bad |= lane * NPL + j < E && !pf_finite(v[j]);
        bad = __any(bad);
        if (!norm) {   // unnormalised weights need the full softmax denominator
            float m = v[0];
#pragma unroll
            for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
            top_all = pf_wave_max_fast(m);
#pragma unroll
            for (int j = 0; j < NPL; j++) total += expf(v[j] - top_all);   // exp(-inf) = 0 for padding
            total = pf_wave_sum(total);
        }
        top.setup(v, E, lane);
        for (int r = 0; r <= u; r++) {
            const uint32_t best = top.pop();
            if (lane == r) my_key = best;
        }
        const uint32_t mine = (uint32_t)__builtin_amdgcn_readlane((int)my_key, u);
        if (lane == 0) early_expert = mine ? pf_key_id(mine) : 0xffffffffu;
    }
    const Q4TilePlan plan = shared ? q4t_plan<FMTS>(a, true, n0) : q4t_plan<FMT>(a, false, n0);
    const int I = shared ? a.shared_inter : a.inter;
    if (!shared || FMT == PF_IQ2_XXS) __syncthreads();   // the early expert; the tables
    const uint32_t early = shared ? 0u : early_expert;
    const bool early_ok = early < (uint32_t)E;   // a nonfinite logit can leave no maximum: the error word says so below
    // Expert streaming: the slot's expert was routed by an earlier launch and sits in pool slot slots[u]; the tile is
    // read there, whatever the early guess says, and the routing below only has to agree with the ids it was fetched by.
    constexpr bool pooled = POOL;
    uint32_t pooled_at = 0u;
    if (pooled && !shared) {
        pooled_at = a.slots[u];
        if (pooled_at >= a.pool_slots) {
            if (threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS);
            pooled_at = 0u;
        }
    }
    if (shared) q4t_tile<FMTS>(a, plan, partial, tables, 0u, wave);
    else q4t_tile<FMT>(a, plan, partial, tables, pooled ? pooled_at : early_ok ? early : 0u, wave);
    if (wave == 0 && !shared) {
        // the remaining slots, the candidate beyond them and one more key, while the other waves' weight bytes travel
        for (int r = u + 1; r <= rounds; r++) {
            const uint32_t best = top.pop();
            if (lane == r) my_key = best;
        }
        uint32_t my_id;
        float my_z, my_s2, weight;
        bool close;
        const bool ambiguous = pf_topk_exact_order<NPL>(my_key, rounds + 1, v, s2, lane, my_id, my_z, my_s2);
        pf_route_finish_wave(my_z, my_s2, K, rounds, norm, H, total, top_all, lane, weight, close);
        close |= ambiguous;
        if (lane < K) { R.ids[lane] = my_id; R.weights[lane] = weight; }
        if (lane == 0) { R.close[0] = close ? 1u : 0u; R.nonfinite[0] = bad ? 1u : 0u; }
    }
    __syncthreads();
    uint32_t e = early;
    if (!shared) {
        if (R.close[0]) {   // the same for every thread of every workgroup: the inputs are the same
            q4t_route_fix<NPL>(reinterpret_cast<const float *>(a.w[0]), a.x, a.logits, a.logit_ssq, E, K, norm, H,
                               (int)(scratch - reinterpret_cast<float *>(lds)), &R);
        } else if (threadIdx.x == 0) {
            R.close_mask = 0;
            R.bad = R.nonfinite[0];
        }
        // the slot's expert in the final order (the early guess came from truncated keys; the serial-order routing
        // can name another expert)
        e = R.ids[u];
        if (!pooled && e != early && e < (uint32_t)E) {
            __syncthreads();
            q4t_tile<FMT>(a, plan, partial, tables, e, wave);
            __syncthreads();
        }
        if (blockIdx.x == 0) {
            // publish the routes for the next kernel and the caller (one token: slot = pair = unique expert)
            if (R.close[0] == 0) __syncthreads();   // R.bad above; route_finish ends with a barrier of its own
            for (int q = threadIdx.x; q < K; q += blockDim.x) {
                if (pooled && a.ids[q] != R.ids[q]) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS);   // not the experts that were fetched
                a.ids[q] = R.ids[q];
                a.route_weights[q] = R.weights[q];
                if (gridDim.y == 1) {   // the table of unique experts: read by the other down kernel, which runs after this one only for one token
                    a.uniq[1 + q] = R.ids[q];
                    a.uniq[1 + K + q] = q;
                    a.uniq[1 + 2 * K + q] = 1u;
                }
            }
            if (threadIdx.x == 0) {
                if (gridDim.y == 1) a.uniq[0] = K;
                if (R.bad) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
                if (R.close_mask) atomicAdd(a.exact_rows, 1u);
                if (R.close_mask == 2u) atomicAdd(a.exact_rows + 1, 1u);   // settled the long way
            }
        }
        if (e >= (uint32_t)E) {   // only reachable with nonfinite logits
            if (threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
            return;
        }
    }
    // the second wave: lane t < 32 adds up the gate row of unit n0 + t over the waves in wave order, lane 32 + t its
    // up row; then SwiGLU, the activation and its digits
    if (wave == 1) {
        float sum = 0.0f;
        for (int w = 0; w < 15; w++) sum += partial[w * 64 + lane];
        const float g = sum, up = __shfl(sum, (lane & 31) + 32);
        const float act = pf_silu(g) * up;
        // the 32 units are one 32-group of the activation row: its digit image for the down kernel
        // (vector u of the activation images; the shared expert's follows the top_k routed ones)
        const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
        if (lane < 32) {
            if (!pf_finite(act)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
            (shared ? a.shared_act : a.act + (size_t)u * I)[n0 + lane] = act;
        }
        image2_group(a.aimg + (size_t)u * pf_image2_words(widest), act, n0 / 32, I, lane);
    }
}

// With several tokens there are more workgroups than compute units; two workgroups per compute unit (64 registers a
// lane) measured slower than one after the other: the products are bound by the vector units, not by waiting.
template <int NPL, int FMT, int FMTS, bool POOL>
__global__ void __launch_bounds__(1024) pf_k_dec_gate_up_q4t(PfKernelArgs a, int routed_blocks) {
    q4t_gate_up<NPL, FMT, FMTS, POOL>(a, routed_blocks);
}

// ---- several tokens: routing in a launch of its own, then kernel 2 without it -----------------------------------
// With several tokens kernel 2 has more workgroups than the GPU has compute units, and a workgroup that routes before it
// can ask for its weights pays that wait in every round; it also keeps the re-route's 82 KB of LDS and the selection's
// registers, which leave room for one workgroup per compute unit only.  So the tokens are routed first, one workgroup
// each (a flagged token is routed again once, not by every workgroup of its grid row), and kernel 2 takes its expert
// from the ids: eight waves, at most 64 registers a lane and a few KB of LDS, four workgroups per compute unit, some
// computing while the others wait for their weights.
template <int NPL>
__global__ void __launch_bounds__(1024) pf_k_dec_route(PfKernelArgs a) {
    extern __shared__ int lds[];
    __shared__ RouteLds R;
    q4t_at_token(a, (int)blockIdx.x);
    const int H = a.hidden, K = a.top_k, E = a.experts, lane = pf_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool norm = a.norm_topk != 0;
    // up to eight waves rank a chunk of the experts each and leave its k + 1 best in LDS, wave 0 merges them
    constexpr int NPL1 = NPL > 8 ? NPL / 8 : 1;
    const int parts = min(8, (E + 63) / 64), chunk = (E + parts - 1) / parts, rounds = K + 1;
    if (wave < parts) pf_route_stage1<NPL1>(a.logits, a.logit_ssq, E, wave, chunk, rounds, norm, &R.cands[0], lane);
    __syncthreads();
    if (wave == 0) {
        const PfRouteResult r = pf_route_stage2(&R.cands[0], parts, K, rounds, norm, H, lane);
        if (lane < K) { R.ids[lane] = r.id; R.weights[lane] = r.weight; }
        if (lane == 0) { R.close[0] = r.close ? 1u : 0u; R.nonfinite[0] = r.bad ? 1u : 0u; }
    }
    __syncthreads();
    if (R.close[0]) {
        q4t_route_fix<NPL>(reinterpret_cast<const float *>(a.w[0]), a.x, a.logits, a.logit_ssq, E, K, norm, H, 0, &R);
    } else {
        if (threadIdx.x == 0) { R.close_mask = 0; R.bad = R.nonfinite[0]; }
        __syncthreads();
    }
    for (int q = threadIdx.x; q < K; q += blockDim.x) {
        a.ids[q] = R.ids[q];
        a.route_weights[q] = R.weights[q];
    }
    if (threadIdx.x == 0) {
        if (R.bad) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
        if (R.close_mask) atomicAdd(a.exact_rows, 1u);
        if (R.close_mask == 2u) atomicAdd(a.exact_rows + 1, 1u);   // settled the long way
    }
}

#define Q4G_WAVES 8    // all of them share the row's 64-weight runs,
#define Q4G_ITEMS 4    // this many a wave: hidden <= 64 * Q4G_ITEMS * Q4G_WAVES
template <int FMT>
__device__ __forceinline__ void q4g_tile(const PfKernelArgs &a, const Q4TilePlan &p, float *partial, const uint32_t *tables, uint32_t e, int wave) {
    const int lane = pf_lane();
    const uint8_t *tile = p.base + (size_t)e * p.expert_bytes;
    const PfScalarWords image = (PfScalarWords)(uintptr_t)a.ximg;
    TileItem<FMT> w[Q4G_ITEMS];
#pragma unroll
    for (int k = 0; k < Q4G_ITEMS; k++) {
        const int it = wave + Q4G_WAVES * k;
        if (it < p.items) q4t_load(w[k], tile + TileGeometry<FMT>::chunk_at(0, p.kblocks, it >> 2), p.row, it & 3);
    }
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < Q4G_ITEMS; k++) {
        const int it = wave + Q4G_WAVES * k;
        if (it < p.items) {
            const int g = 2 * it;
            total += q4t_dot(w[k], image + PF_IMG_GROUP * g, image + PF_IMG_GROUP * p.groups + g, image + (PF_IMG_GROUP + 1) * p.groups + g,
                             it & 3, tables);
        }
    }
    partial[wave * 64 + lane] = total;
}

template <int FMT, int FMTS>
__global__ void __launch_bounds__(64 * Q4G_WAVES) __attribute__((amdgpu_waves_per_eu(8))) pf_k_dec_gate_up_given(PfKernelArgs a, int routed_blocks) {
    extern __shared__ int lds[];
    q4t_at_token(a, (int)blockIdx.y);
    const int K = a.top_k, lane = pf_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    if (FMT == PF_IQ2_XXS) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.iq2_signed);
        for (int i = (int)threadIdx.x; i < 2048; i += 64 * Q4G_WAVES) reinterpret_cast<uint4 *>(tables)[i] = src[i];
    }
    float *partial = reinterpret_cast<float *>(lds + table_words<FMT>());   // [Q4G_WAVES][64 lanes]
    const bool shared = (int)blockIdx.x >= routed_blocks;
    const int tiles = a.inter / 32;
    const int u = shared ? K : (int)blockIdx.x / tiles;
    const int n0 = 32 * (shared ? (int)blockIdx.x - routed_blocks : (int)blockIdx.x % tiles);
    const int I = shared ? a.shared_inter : a.inter;
    // the slot's expert through the scalar cache
    uint32_t e = shared ? 0u : ((PfScalarWords)(uintptr_t)a.ids)[u];
    if (e >= (uint32_t)a.experts) {   // only reachable with nonfinite logits
        if (threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
        e = 0u;
    }
    const Q4TilePlan plan = shared ? q4t_plan<FMTS>(a, true, n0) : q4t_plan<FMT>(a, false, n0);
    if (FMT == PF_IQ2_XXS) __syncthreads();   // the tables
    if (shared) q4g_tile<FMTS>(a, plan, partial, tables, 0u, wave);
    else q4g_tile<FMT>(a, plan, partial, tables, e, wave);
    __syncthreads();
    if (wave == 0) {
        float sum = 0.0f;
        for (int w = 0; w < Q4G_WAVES; w++) sum += partial[w * 64 + lane];
        const float up = __shfl(sum, (lane & 31) + 32);
        const float act = pf_silu(sum) * up;
        const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
        if (lane < 32) {
            if (!pf_finite(act)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
            (shared ? a.shared_act : a.act + (size_t)u * I)[n0 + lane] = act;
        }
        image2_group(a.aimg + (size_t)u * pf_image2_words(widest), act, n0 / 32, I, lane);
    }
}

template <int NPL>
static void launch_dec_route_lists(const PfKernelArgs &a, int tokens, size_t lds, hipStream_t stream) {
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_route<NPL>), hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
        configured = true;
    }
    hipLaunchKernelGGL((pf_k_dec_route<NPL>), dim3(tokens), dim3(1024), lds, stream, a);
}

static void launch_dec_route(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    const size_t lds = pf_route_fix_lds_floats(a.hidden, a.experts) * 4;
    const int all = (a.experts + 63) / 64;
    if (all <= 1) launch_dec_route_lists<1>(a, tokens, lds, stream);
    else if (all <= 2) launch_dec_route_lists<2>(a, tokens, lds, stream);
    else if (all <= 4) launch_dec_route_lists<4>(a, tokens, lds, stream);
    else if (all <= 8) launch_dec_route_lists<8>(a, tokens, lds, stream);
    else launch_dec_route_lists<16>(a, tokens, lds, stream);
}

template <int FMT, int FMTS>
static void launch_gate_up_given(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    const int routed_blocks = a.top_k * (a.inter / 32);
    const size_t lds = (size_t)table_words<FMT>() * 4 + (size_t)Q4G_WAVES * 64 * 4;
    hipLaunchKernelGGL((pf_k_dec_gate_up_given<FMT, FMTS>), dim3(routed_blocks + a.shared_inter / 32, tokens), dim3(64 * Q4G_WAVES), lds, stream, a,
                       routed_blocks);
}

// Kernel 2 alone on the tile order (one token; the down kernel stays the segment one): layers whose routed gate and up
// tensors are Q4_K or IQ2_XXS with the copy kept and whose shared expert is in the same format or, as in the checkpoint
// profiles, Q8_0 with its copy kept.
template <int FMT, int FMTS>
static bool q4t_gate_up_applies(const PfKernelArgs &a) {
    if (!((FMT == PF_Q4_K || FMT == PF_IQ2_XXS) && (FMTS == FMT || FMTS == PF_Q8_0))) return false;
    for (int t : {1, 2}) if (!TileGeometryHost<FMT>::tensor(a, t)) return false;
    for (int t : {4, 5}) if (!TileGeometryHost<FMTS>::tensor(a, t)) return false;
    return a.hidden % 256 == 0 && 4 * (a.hidden / 256) <= 15 * Q4T_ITEMS && a.inter % 32 == 0 && a.shared_inter % 32 == 0 &&
           a.top_k < a.experts && a.top_k <= 15 && a.experts <= 1024;
}

template <int NPL, int FMT, int FMTS, bool POOL>
static void launch_gate_up_q4t_lists(const PfKernelArgs &a, dim3 grid, size_t lds, hipStream_t stream, int routed_blocks) {
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS (the re-route's chunk buffers)
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_gate_up_q4t<NPL, FMT, FMTS, POOL>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);   // the kernel has static LDS too
        configured = true;
    }
    hipLaunchKernelGGL((pf_k_dec_gate_up_q4t<NPL, FMT, FMTS, POOL>), grid, dim3(1024), lds, stream, a, routed_blocks);
}

template <int FMT, int FMTS, bool POOL = false>
static void launch_gate_up_q4t(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    const int H = a.hidden, I = a.inter, Is = a.shared_inter, E = a.experts, K = a.top_k;
    const int routed_blocks = K * (I / 32);
    const dim3 g1(routed_blocks + Is / 32, tokens);
    const int all = (E + 63) / 64;
    const size_t lds = (size_t)table_words<FMT>() * 4 + (size_t)15 * 64 * 4 + pf_route_fix_lds_floats(H, E) * 4;
    if (all <= 1) launch_gate_up_q4t_lists<1, FMT, FMTS, POOL>(a, g1, lds, stream, routed_blocks);
    else if (all <= 2) launch_gate_up_q4t_lists<2, FMT, FMTS, POOL>(a, g1, lds, stream, routed_blocks);
    else if (all <= 4) launch_gate_up_q4t_lists<4, FMT, FMTS, POOL>(a, g1, lds, stream, routed_blocks);
    else if (all <= 8) launch_gate_up_q4t_lists<8, FMT, FMTS, POOL>(a, g1, lds, stream, routed_blocks);
    else launch_gate_up_q4t_lists<16, FMT, FMTS, POOL>(a, g1, lds, stream, routed_blocks);
}

// ---- kernel 3: down products and the combine ---------------------------------------------------
// blockIdx.x = t * row_blocks + nb; one wave per slot plus one for the shared expert; a routed
// wave covers the block's rows in one step.  Every wave turns its slot's activation row into a
// digit image in LDS while its weight bytes are on their way.
// One wave's products of kernel 3: its slot's rows of the block against its activation image.
template <int FMT, int SPL>
__device__ __forceinline__ void down_rows(const PfKernelArgs &a, float *partial_row, int *image, const uint32_t *tables,
                                          const float *act_row, bool block_sync, int tensor, uint32_t e, int I, int H,
                                          int n_base, int rows_per_block, int s) {
    const int lane = pf_lane();
    const int LPR = row_lanes(I), rows = 64 / LPR, steps = rows >= rows_per_block ? 1 : rows_per_block / rows;
    const int seg = lane & (LPR - 1), r = lane / LPR;
    const bool second = SPL > 1 && seg + LPR < I / 64;   // this lane also holds segment seg + LPR of its row
    // the wave's first activations are requested before its weights: loads of a wave return in order, and the
    // image can then be built while the weight bytes are still on their way
    const bool first_chunk = lane < I / 8;
    float4 a0 = make_float4(0.0f, 0.0f, 0.0f, 0.0f), a1 = a0;
    if (first_chunk) {
        a0 = reinterpret_cast<const float4 *>(act_row)[2 * lane];
        a1 = reinterpret_cast<const float4 *>(act_row)[2 * lane + 1];
    }
    WSeg<FMT> w[SPL];   // further steps (a shared expert wider than the routed ones) load as they go
    wseg_load<FMT>(w[0], a, tensor, e, min(n_base + r, H - 1), seg);
    if (SPL > 1 && second) wseg_load<FMT>(w[SPL - 1], a, tensor, e, min(n_base + r, H - 1), seg + LPR);
    if (first_chunk) image_chunk(image, a0, a1, lane, I);
    for (int j = lane + 64; j < I / 8; j += 64)
        image_chunk(image, reinterpret_cast<const float4 *>(act_row)[2 * j], reinterpret_cast<const float4 *>(act_row)[2 * j + 1], j, I);
    if (block_sync) __syncthreads();   // the tables staged by the whole workgroup
    else pf_wave_lds_fence();
    XSeg x;   // one segment's digits at a time: with two segments they are read from LDS again at every step
    xseg_load(x, image, I, seg);
    if (SPL == 1) {
        for (int st = 0; st < steps; st++) {
            const float v = span_sum(wseg_dot<FMT>(w[0], x, seg, tables), LPR);
            const int row = st * rows + r;
            if (seg == 0 && row < rows_per_block) partial_row[row] = v;
            if (st + 1 < steps) wseg_load<FMT>(w[0], a, tensor, e, min(n_base + (st + 1) * rows + r, H - 1), seg);
        }
        return;
    }
    for (int st = 0; st < steps; st++) {
        WSeg<FMT> next[SPL];   // the following step's weights, on their way during this step's products
        if (st + 1 < steps) {
            wseg_load<FMT>(next[0], a, tensor, e, min(n_base + (st + 1) * rows + r, H - 1), seg);
            if (second) wseg_load<FMT>(next[SPL - 1], a, tensor, e, min(n_base + (st + 1) * rows + r, H - 1), seg + LPR);
        }
        if (st > 0) xseg_load(x, image, I, seg);
        float dot = wseg_dot<FMT>(w[0], x, seg, tables);
        __builtin_amdgcn_sched_barrier(0);   // the second segment's digits reuse the first's registers: no hoisting above
        if (second) {
            xseg_load(x, image, I, seg + LPR);
            dot += wseg_dot<FMT>(w[SPL - 1], x, seg + LPR, tables);
        }
        __builtin_amdgcn_sched_barrier(0);
        const float v = span_sum(dot, LPR);
        const int row = st * rows + r;
        if (seg == 0 && row < rows_per_block) partial_row[row] = v;
        if (st + 1 < steps) {
            w[0] = next[0];
            if (second) w[SPL - 1] = next[SPL - 1];
        }
    }
}

// FMT: format of the routed down tensor; FMTS: of the shared expert's.
// MAXT: the largest workgroup the instantiation is launched with (64 threads per slot and the shared
// expert): 768 leaves room for the second segment's registers when top_k <= 11.
template <int FMT, int FMTS, int NT, int SPL, int MAXT>
__global__ void __launch_bounds__(MAXT) pf_k_dec_down(PfKernelArgs a, int row_blocks, int rows_per_block, int image_pitch) {
    __shared__ float partial[17][64];
    extern __shared__ int lds[];
    constexpr bool TABLES = FMT == PF_IQ2_XXS || FMTS == PF_IQ2_XXS;
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    if (TABLES) stage_tables(tables, a.iq2_signed);
    const int H = a.hidden, K = a.top_k, lane = pf_lane(), s = threadIdx.x >> 6;
    const int t = blockIdx.x / row_blocks, nb = blockIdx.x % row_blocks, P = NT * K;
    const bool shared = s == K;
    const int I = shared ? a.shared_inter : a.inter;
    uint32_t e = 0, u = 0;
    if (!shared) {
        e = a.ids[t * K + s];
        u = a.uniq[1 + P + t * K + s];
        if (e >= (uint32_t)a.experts || u >= (uint32_t)P) {   // only reachable with nonfinite logits
            if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
            e = 0;
            u = 0;
        }
    }
    const int n_base = nb * rows_per_block;
    int *image = lds + (TABLES ? 8192 : 0) + s * image_pitch;
    // operands of the final combine, requested now so that they arrive with the weights
    float rw[16];
#pragma unroll
    for (int slot = 0; slot < 16; slot++) rw[slot] = slot < K ? a.route_weights[t * K + slot] : 0.0f;
    const float shared_scale = a.shared_scale[t];
    PfOutputRegs out_regs;
    if ((int)threadIdx.x < rows_per_block && n_base + (int)threadIdx.x < H)
        pf_output_prefetch(a, t, n_base + threadIdx.x, out_regs);
    if (shared)
        down_rows<FMTS, SPL>(a, partial[s], image, tables, a.shared_act + (size_t)t * I, TABLES, 6, 0, I, H, n_base,
                        rows_per_block, s);
    else
        down_rows<FMT, SPL>(a, partial[s], image, tables, a.act + ((size_t)u * NT + t) * I, TABLES, 3, e, I, H, n_base,
                       rows_per_block, s);
    __syncthreads();
    const int n = n_base + threadIdx.x;
    if ((int)threadIdx.x < rows_per_block && n < H) {
        float sum = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 16; slot++)   // slot order, as src/qwen4_moe.c:362-372
            if (slot < K) sum += rw[slot] * partial[slot][threadIdx.x];
        const float y = sum + shared_scale * partial[K][threadIdx.x];
        if (!pf_output_commit(a, t, n, y, out_regs)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
}

// ---- kernel 3, one token, Q4_K tensors in tile order ------------------------------------------------
// Eight output rows per workgroup, one wave per slot and one for the shared expert, as above; a lane is
// (row, 64-weight run): lanes 0..7 the rows' run 0, 8..15 run 1 and so on (further runs in turn), so the
// eight rows' pieces of a run are one 128-byte line of the tile-ordered copy.  The activation digits come
// from the digit images kernel 2 left in global memory (nothing is built here); the lanes of a row add
// up across the wave, the slots meet in LDS and are combined in slot order.
// One run of one row (its item loaded by q4t_load) against the slot's digits in LDS (mine: the slot's image).  Q4_K: header
// and two halves; IQ2_XXS: one 16-byte piece and the block's half scale, magnitudes from the tables.
__device__ __forceinline__ float down_dot(const TileItem<PF_Q4_K> &w, int rr, const uint32_t *mine, int run, int groups, const uint32_t *) {
    const uint4 hdr = w.hdr, p0 = w.piece[0], p1 = w.piece[1];
    const uint2 st = *reinterpret_cast<const uint2 *>(mine + PF_IMG_GROUP * groups + 2 * run);
    const uint2 sm = *reinterpret_cast<const uint2 *>(mine + (PF_IMG_GROUP + 1) * groups + 2 * run);
    uint32_t sc2, mn2;
    if (rr < 2) {
        sc2 = (hdr.y >> (16 * rr)) & 0x3F3Fu;
        mn2 = (hdr.z >> (16 * rr)) & 0x3F3Fu;
    } else {
        const int sh = 16 * (rr - 2);
        sc2 = ((hdr.w >> sh) & 0x0F0Fu) | (((hdr.y >> sh) >> 2) & 0x3030u);
        mn2 = (((hdr.w >> sh) >> 4) & 0x0F0Fu) | (((hdr.z >> sh) >> 2) & 0x3030u);
    }
    const float d = half_bits(hdr.x & 0xffffu), dmin = half_bits(hdr.x >> 16);
    const uint32_t q[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
    float value[2];
    // the run's two groups, PF_IMG_GROUP dwords each, plane by plane: the low nibbles against the first, the high against the second
#pragma unroll
    for (int g = 0; g < 2; g++) {
        uint32_t dg[PF_IMG_GROUP];
#pragma unroll
        for (int i = 0; i < PF_IMG_GROUP / 4; i++) {
            const uint4 v = reinterpret_cast<const uint4 *>(mine + PF_IMG_GROUP * (2 * run + g))[i];
            dg[4 * i] = v.x; dg[4 * i + 1] = v.y; dg[4 * i + 2] = v.z; dg[4 * i + 3] = v.w;
        }
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int nib = (int)((q[i] >> (4 * g)) & 0x0F0F0F0Fu);
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) part[p] = __builtin_amdgcn_sdot4(nib, (int)dg[8 * p + i], part[p], false);
        }
        value[g] = image_value(part);
    }
    const float s0 = (float)(sc2 & 255u), m0 = (float)(mn2 & 255u), s1 = (float)(sc2 >> 8), m1 = (float)(mn2 >> 8);
    const float t0 = fmaf(d * s0, value[0], -(dmin * m0) * (float)(int)sm.x);
    const float t1 = fmaf(d * s1, value[1], -(dmin * m1) * (float)(int)sm.y);
    return fmaf(__uint_as_float(st.x), t0, __uint_as_float(st.y) * t1);
}

// (tables: here the 256-entry magnitude grid, 2 KB, not the signed tables: staging 32 KB per workgroup cost this
// kernel more than the sign arithmetic does)
__device__ __forceinline__ float down_dot(const TileItem<PF_IQ2_XXS> &w, int, const uint32_t *mine, int run, int groups,
                                          const uint32_t *tables) {
    const uint4 piece = w.piece;
    const uint32_t dbits = w.dbits;
    const uint2 st = *reinterpret_cast<const uint2 *>(mine + PF_IMG_GROUP * groups + 2 * run);
    float acc[2];
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        uint32_t d32[PF_IMG_GROUP];
#pragma unroll
        for (int i = 0; i < PF_IMG_GROUP / 4; i++) {
            const uint4 v = reinterpret_cast<const uint4 *>(mine + PF_IMG_GROUP * (2 * run + gg))[i];
            d32[4 * i] = v.x; d32[4 * i + 1] = v.y; d32[4 * i + 2] = v.z; d32[4 * i + 3] = v.w;
        }
        const uint32_t idx = gg ? piece.z : piece.x, word = gg ? piece.w : piece.y;
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int slot = 0; slot < 4; slot++) {
            const uint32_t g = (idx >> (8 * slot)) & 255u, s7 = (word >> (7 * slot)) & 127u;
            const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);   // the eighth sign is the parity of the seven
            // the grid entry's eight magnitudes (8, 25 or 43: never zero) with the signs applied byte by byte: sign bit i
            // of a nibble moved to bit 8i, widened to a byte mask, then ~m + 1 in every flagged byte (no byte overflows)
            const uint2 mag = reinterpret_cast<const uint2 *>(tables)[g];
            const uint32_t tl = ((s8 & 15u) * 0x00204081u) & 0x01010101u, th = ((s8 >> 4) * 0x00204081u) & 0x01010101u;
            const int ml = (int)((mag.x ^ (tl * 0xFFu)) + tl), mh = (int)((mag.y ^ (th * 0xFFu)) + th);
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) {
                part[p] = __builtin_amdgcn_sdot4(ml, (int)d32[8 * p + 2 * slot], part[p], false);
                part[p] = __builtin_amdgcn_sdot4(mh, (int)d32[8 * p + 2 * slot + 1], part[p], false);
            }
        }
        acc[gg] = __uint_as_float(gg ? st.y : st.x) * (float)(2u * (word >> 28) + 1u) * image_value(part);
    }
    return half_bits(dbits) * 0.125f * (acc[0] + acc[1]);
}

// The formats kept row by row (the profiles' down tensors): a lane's run is the segment the loaders above fetch; lanes
// r * 8 + part, so that the eight runs of a row are neighbouring lanes and neighbouring bytes.
struct GroupDigits {   // one 32-group from the slot's image in LDS
    uint32_t dg[PF_IMG_GROUP];
    float step;
};
__device__ __forceinline__ void group_digits(GroupDigits &x, const uint32_t *mine, int group, int groups) {
#pragma unroll
    for (int i = 0; i < PF_IMG_GROUP / 4; i++) {
        const uint4 v = reinterpret_cast<const uint4 *>(mine + PF_IMG_GROUP * group)[i];
        x.dg[4 * i] = v.x; x.dg[4 * i + 1] = v.y; x.dg[4 * i + 2] = v.z; x.dg[4 * i + 3] = v.w;
    }
    x.step = __uint_as_float(mine[PF_IMG_GROUP * groups + group]);
}

__device__ __forceinline__ float down_dot(const WSeg<PF_Q8_0> &w, const uint32_t *mine, int run, int groups) {
    float out = 0.0f;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        GroupDigits x;
        group_digits(x, mine, 2 * run + g, groups);
        const uint32_t q[8] = {w.q[2 * g].x, w.q[2 * g].y, w.q[2 * g].z, w.q[2 * g].w,
                               w.q[2 * g + 1].x, w.q[2 * g + 1].y, w.q[2 * g + 1].z, w.q[2 * g + 1].w};
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) part[p] = __builtin_amdgcn_sdot4((int)q[i], (int)x.dg[8 * p + i], part[p], false);
        out = fmaf(x.step * half_bits((w.d2 >> (16 * g)) & 0xffffu), image_value(part), out);
    }
    return out;
}

__device__ __forceinline__ float down_dot(const WSeg<PF_MXFP4> &w, const uint32_t *mine, int run, int groups) {
    float out = 0.0f;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        GroupDigits x;
        group_digits(x, mine, 2 * run + g, groups);
        const uint32_t q[4] = {w.q[g].x, w.q[g].y, w.q[g].z, w.q[g].w};
        int part[PF_IMG_PLANES] = {};
#pragma unroll
        for (int i = 0; i < 4; i++) {   // a byte's low nibble is weight j of the block, its high nibble weight j + 16
            const int lo = e2m1_twice4(q[i] & 0x0F0F0F0Fu), hi = e2m1_twice4((q[i] >> 4) & 0x0F0F0F0Fu);
#pragma unroll
            for (int p = 0; p < PF_IMG_PLANES; p++) {
                part[p] = __builtin_amdgcn_sdot4(lo, (int)x.dg[8 * p + i], part[p], false);
                part[p] = __builtin_amdgcn_sdot4(hi, (int)x.dg[8 * p + 4 + i], part[p], false);
            }
        }
        const float scale = 0.5f * pf_e8m0_scale((w.e2 >> (8 * g)) & 255u);   // the integers are twice the values
        out = fmaf(x.step * scale, image_value(part), out);
    }
    return out;
}

// Q2_K: the sums of the activation integers per sub-group of 16 come from dot products with ones, as in wseg_dot.
__device__ __forceinline__ float down_dot(const WSeg<PF_Q2_K> &w, const uint32_t *mine, int run, int groups) {
    const float d = half_bits(w.dd & 0xffffu), dmin = half_bits(w.dd >> 16);
    float out = 0.0f;
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        GroupDigits x;
        group_digits(x, mine, 2 * run + gg, groups);
        const int shift = 2 * (2 * (run & 1) + gg);
        float group = 0.0f;
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            int c[PF_IMG_PLANES] = {}, ones[PF_IMG_PLANES] = {};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int codes = (int)((w.q[4 * sub + i] >> shift) & 0x03030303u);
#pragma unroll
                for (int p = 0; p < PF_IMG_PLANES; p++) {
                    const int digits = (int)x.dg[8 * p + 4 * sub + i];
                    c[p] = __builtin_amdgcn_sdot4(codes, digits, c[p], false);
                    ones[p] = __builtin_amdgcn_sdot4(0x01010101, digits, ones[p], false);
                }
            }
            const uint32_t sm = (w.sm >> (8 * (2 * gg + sub))) & 255u;
            group += fmaf(d * (float)(sm & 15u), image_value(c), -(dmin * (float)(sm >> 4)) * image_value(ones));
        }
        out = fmaf(x.step, group, out);
    }
    return out;
}

constexpr size_t Q4T_DOWN_LDS = 150 * 1024;   // dynamic LDS kernel 3 on the tile order may ask for
template <int F> __host__ __device__ constexpr bool tile_ordered() { return F == PF_Q4_K || F == PF_IQ2_XXS; }

// One wave's rows of its slot (eight in the tile order): partial_row[0..rows).  tensor: 3 (the slot's expert e) or 6 (the
// shared expert); I: the logical width, k_stored: the stored one; dots: rows * I / 64 floats of LDS of the wave's own.
template <int F>
__device__ __forceinline__ void down_wave(const PfKernelArgs &a, int tensor, uint32_t e, int I, int k_stored, int n_base, int rows,
                                          const uint32_t *image, uint32_t *mine, uint32_t *tables, float *dots, float *partial_row) {
    const int lane = pf_lane(), runs = I / 64, groups = I / 32;
    // IQ2_XXS: every wave keeps its own copy of the 2 KB magnitude grid, so that no wave waits for another before the
    // final sums (a shared copy needs a workgroup barrier between its staging and its first use)
    if (F == PF_IQ2_XXS) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.iq2_grid);
        reinterpret_cast<uint4 *>(tables)[lane] = src[lane];
        reinterpret_cast<uint4 *>(tables)[64 + lane] = src[64 + lane];
    }
    // the slot's image into this wave's part of LDS (each lane needs the digits of its own run; fetched per lane they
    // would cost eight requests a lane).  Sending the first weights' loads ahead of the image's, or two steps' weights
    // at once, measured the same or slower.
    const int words = (int)pf_image2_words(I);
    for (int i = 4 * lane; i < words; i += 256) *reinterpret_cast<uint4 *>(mine + i) = *reinterpret_cast<const uint4 *>(image + i);
    float total = 0.0f;
    bool fenced = false;
    if constexpr (tile_ordered<F>()) {
        typedef TileGeometry<F> G;
        const int r = lane & 7, part = lane >> 3, kblocks = k_stored / 256;
        const uint8_t *tile = G::tensor(a, tensor) + (size_t)e * G::expert_bytes(a, tensor) + G::chunk_at(n_base / 32, kblocks, 0);
        const int row_in_tile = (n_base & 31) + r;
        for (int run = part; run < runs; run += 8) {
            TileItem<F> item;
            q4t_load(item, tile + G::chunk_at(0, kblocks, run >> 2), row_in_tile, run & 3);
            if (!fenced) { pf_wave_lds_fence(); fenced = true; }   // the image's (and grid's) stores of this wave before its reads
            total += down_dot(item, run & 3, mine, run, groups, tables);
        }
        // the row's runs: lanes r, r + 8, ..., r + 56
        total += __shfl_xor(total, 8);
        total += __shfl_xor(total, 16);
        total += __shfl_xor(total, 32);
        if (lane < 8) partial_row[lane] = total;
    } else {
        // the (row, run) pairs of the wave's rows in turn over the lanes: neighbouring lanes are neighbouring runs of a
        // row, neighbouring bytes, and a row count that does not divide 64 (ten for a hidden width of 2560) leaves no
        // lane idle but in the last step.  The products meet in LDS; a lane per row adds its runs in order.
        const int items = rows * runs;
        for (int item = lane; item < items; item += 64) {
            const int r = item / runs, run = item - r * runs;
            WSeg<F> w;
            wseg_load<F>(w, a, tensor, e, (size_t)(n_base + r), run);
            if (!fenced) { pf_wave_lds_fence(); fenced = true; }
            dots[item] = down_dot(w, mine, run, groups);
        }
        pf_wave_lds_fence();
        if (lane < rows) {
            for (int run = 0; run < runs; run++) total += dots[lane * runs + run];
            partial_row[lane] = total;
        }
    }
}

// (at most 80 registers a lane: two workgroups of eleven waves then share a compute unit, which a hidden width of 2560,
// 320 workgroups on 256 compute units, needs to finish in one round)
template <int FMT, int FMTS, bool POOL>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(FMT == PF_IQ2_XXS ? 4 : 6))) pf_k_dec_down_q4t(PfKernelArgs a, int rows) {
    __shared__ float partial[17][16];
    extern __shared__ int lds[];   // IQ2_XXS: the waves' magnitude grids; [slot][image words of the widest activation row]; [slot][rows * runs] products
    constexpr bool GRID = FMT == PF_IQ2_XXS || FMTS == PF_IQ2_XXS;
    pf_args_now(a.ids, a.route_weights, a.shared_scale, a.aimg, a.hc_residual, a.wt[3], a.wt[6], a.w[3], a.w[6], a.expert_bytes[3],
                a.shared_inter, a.down_physical, a.hc_streams, a.error_word, rows);
    const int token = (int)blockIdx.y;
    q4t_at_token(a, token);
    const int H = a.hidden, K = a.top_k, lane = pf_lane();
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds) + (GRID ? 512 * s : 0);
    int *images = lds + (GRID ? 512 * (K + 1) : 0);
    const bool shared = s == K;
    const int n_base = rows * (int)blockIdx.x;
    const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
    float *dots = reinterpret_cast<float *>(images + (size_t)(K + 1) * pf_image2_words(widest)) + (size_t)s * rows * (widest / 64);
    // the slot's expert and the combine's operands through the scalar cache
    const PfScalarWords ids = (PfScalarWords)(uintptr_t)a.ids, rws = (PfScalarWords)(uintptr_t)a.route_weights;
    uint32_t e = shared ? 0u : ids[s];
    float rw[16];
#pragma unroll
    for (int slot = 0; slot < 16; slot++) rw[slot] = slot < K ? __uint_as_float(rws[slot]) : 0.0f;
    const float shared_scale = __uint_as_float(((PfScalarWords)(uintptr_t)a.shared_scale)[0]);
    if (e >= (uint32_t)a.experts) {   // only reachable with nonfinite logits
        if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
        e = 0;
    }
    if (POOL && !shared) {   // expert streaming: the expert's rows sit in its pool slot
        e = ((PfScalarWords)(uintptr_t)a.slots)[s];
        if (e >= a.pool_slots) {
            if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS);
            e = 0;
        }
    }
    PfOutputRegs out_regs;
    if ((int)threadIdx.x < rows) pf_output_prefetch(a, token, n_base + threadIdx.x, out_regs);
    const uint32_t *image = a.aimg + (size_t)s * pf_image2_words(widest);   // slot = unique expert with one token; the shared expert's follows
    uint32_t *mine = reinterpret_cast<uint32_t *>(images) + (size_t)s * pf_image2_words(widest);
    if (shared) down_wave<FMTS>(a, 6, 0u, a.shared_inter, a.shared_inter, n_base, rows, image, mine, tables, dots, partial[s]);
    else down_wave<FMT>(a, 3, e, a.inter, a.down_physical, n_base, rows, image, mine, tables, dots, partial[s]);
    __syncthreads();
    const int n = n_base + threadIdx.x;
    if ((int)threadIdx.x < rows && n < H) {
        float sum = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 16; slot++)   // slot order, as src/qwen4_moe.c:362-372
            if (slot < K) sum += rw[slot] * partial[slot][threadIdx.x];
        const float y = sum + shared_scale * partial[K][threadIdx.x];
        if (!pf_output_commit(a, token, n, y, out_regs)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
}

// ---- kernel 3 for batches of six tokens and more, tensors in tile order -------------------------------
// A workgroup takes 64 output rows of one token, a wave per slot (the last wave the shared expert), a lane per row: the
// 64 lanes of a wave share the run they are at, so the activation digits are scalar operands read from the digit image
// in memory, as in kernel 2 -- no copy of the images in LDS, no sums across lanes -- and a lane keeps its row's sum over
// the runs in a register.  That is 32 workgroups a token for 256 compute units: nothing for one token, but a batch
// fills them, while pf_k_dec_down_q4t goes through a batch in rounds of two tokens (two workgroups a compute unit),
// each round as long as its chain of requests (the slot's expert, its rows, the image) and about 2.2 us a token.
// Measured on the benchmark layer: 16 tokens 35.5 -> 18.0 us, 8 tokens 20.3 -> 12.9 us, 4 tokens 11.2 -> 13.0 us.
#define DOWN64_ITEMS 4   // requests a lane has on their way
template <int F>
__device__ __forceinline__ float down64_wave(const PfKernelArgs &a, int tensor, uint32_t e, int I, int k_stored, int n0, PfScalarWords image,
                                             const uint32_t *tables) {
    typedef TileGeometry<F> G;
    const int lane = pf_lane(), runs = I / 64, groups = I / 32, kblocks = k_stored / 256, row = lane & 31;
    const uint8_t *tile = G::tensor(a, tensor) + (size_t)e * G::expert_bytes(a, tensor) + G::chunk_at(n0 / 32 + (lane >> 5), kblocks, 0);
    float total = 0.0f;
    for (int first = 0; first < runs; first += DOWN64_ITEMS) {
        TileItem<F> w[DOWN64_ITEMS];
#pragma unroll
        for (int k = 0; k < DOWN64_ITEMS; k++) {
            const int it = first + k;
            if (it < runs) q4t_load(w[k], tile + G::chunk_at(0, kblocks, it >> 2), row, it & 3);
        }
#pragma unroll
        for (int k = 0; k < DOWN64_ITEMS; k++) {
            const int it = first + k;
            if (it < runs) {
                const int g = 2 * it;
                total += q4t_dot(w[k], image + PF_IMG_GROUP * g, image + PF_IMG_GROUP * groups + g, image + (PF_IMG_GROUP + 1) * groups + g,
                                 it & 3, tables);
            }
        }
    }
    return total;
}

template <int FMT, int FMTS>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(6))) pf_k_dec_down_rows64(PfKernelArgs a) {
    __shared__ float partial[17][64];
    extern __shared__ int lds[];   // IQ2_XXS: the signed tables
    constexpr bool TABLES = FMT == PF_IQ2_XXS || FMTS == PF_IQ2_XXS;
    const int token = (int)blockIdx.y;
    q4t_at_token(a, token);
    const int K = a.top_k, lane = pf_lane();
    const int s = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    if (TABLES) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.iq2_signed);
        for (int i = (int)threadIdx.x; i < 2048; i += (int)blockDim.x) reinterpret_cast<uint4 *>(tables)[i] = src[i];
    }
    const bool shared = s == K;
    const int n0 = 64 * (int)blockIdx.x;
    const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
    // the slot's expert and the combine's operands through the scalar cache
    const PfScalarWords ids = (PfScalarWords)(uintptr_t)a.ids, rws = (PfScalarWords)(uintptr_t)a.route_weights;
    uint32_t e = shared ? 0u : ids[s];
    float rw[16];
#pragma unroll
    for (int slot = 0; slot < 16; slot++) rw[slot] = slot < K ? __uint_as_float(rws[slot]) : 0.0f;
    const float shared_scale = __uint_as_float(((PfScalarWords)(uintptr_t)a.shared_scale)[0]);
    if (e >= (uint32_t)a.experts) {   // only reachable with nonfinite logits
        if (lane == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);
        e = 0;
    }
    PfOutputRegs out_regs;
    if (threadIdx.x < 64) pf_output_prefetch(a, token, n0 + threadIdx.x, out_regs);
    const PfScalarWords image = (PfScalarWords)(uintptr_t)(a.aimg + (size_t)s * pf_image2_words(widest));
    if (TABLES) __syncthreads();
    const float mine = shared ? down64_wave<FMTS>(a, 6, 0u, a.shared_inter, a.shared_inter, n0, image, tables)
                              : down64_wave<FMT>(a, 3, e, a.inter, a.down_physical, n0, image, tables);
    partial[s][lane] = mine;
    __syncthreads();
    if (threadIdx.x < 64) {
        float sum = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 16; slot++)   // slot order, as src/qwen4_moe.c:362-372
            if (slot < K) sum += rw[slot] * partial[slot][threadIdx.x];
        const float y = sum + shared_scale * partial[K][threadIdx.x];
        if (!pf_output_commit(a, token, n0 + threadIdx.x, y, out_regs)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
}

#ifndef PF_DOWN_ROWS64_FROM
#define PF_DOWN_ROWS64_FROM 6
#endif
template <int FD, int FS>
static bool down_rows64_applies(const PfKernelArgs &a, int tokens) {
    if (!TileGeometryHost<FD>::tensor(a, 3) || !TileGeometryHost<FS>::tensor(a, 6)) return false;
    return tokens >= PF_DOWN_ROWS64_FROM && a.hidden % 64 == 0 && a.top_k <= 15 && a.inter % 64 == 0 && a.shared_inter % 64 == 0;
}

template <int FD, int FS>
static void launch_down_rows64(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    constexpr bool TABLES = FD == PF_IQ2_XXS || FS == PF_IQ2_XXS;
    hipLaunchKernelGGL((pf_k_dec_down_rows64<FD, FS>), dim3(a.hidden / 64, tokens), dim3(64 * (a.top_k + 1)), TABLES ? 32768 : 0, stream, a);
}

// ---- one token: the whole expert stage in ONE launch ----------------------------------------------
// Workgroup b computes the 32 activations of its (slot, tile) as kernel 2 does, publishes them -- one 128-byte line:
// the group's digit image, step and sum, and the forward's tag -- and then takes eight output rows of the block as
// kernel 3 does, a wave per slot.  Between the two halves every wave waits for the lines of its slot (they are written
// by the sixteen workgroups of that slot), so the launch replaces a kernel boundary by one hand-off through memory:
//   * the down rows of all slots are requested as soon as the routing is known, by the routing wave, into LDS
//     (16 bytes a lane and instruction, lane l at base + 16 l): they travel while the gate and up products run;
//   * a line is 26 pairs {word, tag}: every pair is written with one 64-bit agent-scope atomic store and read with one
//     64-bit agent-scope atomic load (the XCDs' L2s are not coherent with one another), so a pair is never seen half
//     written, a reader that finds the forward's tag in a pair has that word, and the read that polls is the read
//     that fetches;
//   * every line is written FUSE_REPLICAS times and a workgroup polls the replica of its index modulo that: a line that
//     all 256 workgroups poll is a hot spot of the memory channel that holds it;
//   * the tag is a counter in the workspace that the router kernel before this one increments, so nothing has to be
//     cleared and a forward that was cut short leaves nothing a later one could mistake for its own.
// Every workgroup waits for lines of other workgroups, so all of them must be resident at once: the launch is used
// only where the device has a compute unit per workgroup, and the wait is bounded -- a wave that gives up sets
// PF_HIP_ERR_TIMEOUT and goes on with what it has, so the launch ends whatever happens.
#define FUSE_REPLICAS 8
#define FUSE_SPIN_LIMIT (1 << 20)
#define FUSE_DOWN_ROWS 8
#define FUSE_PAIRS (PF_IMG_GROUP + 2)   // pairs of a line: the digit words, the step, the sum
#define FUSE_LINE 64          // dwords of a line: FUSE_PAIRS pairs {word, tag}, padded to 256 bytes
struct FuseGeometry {
    int routed_blocks, expert_blocks;   // workgroups with a routed tile; with any tile (the shared expert's follow)
    int down_blocks;                    // workgroups with output rows
    int grid, lines;
};
__host__ __device__ inline FuseGeometry fuse_geometry(int H, int K, int I, int Is) {
    FuseGeometry g;
    g.routed_blocks = K * (I / 32);
    g.expert_blocks = g.routed_blocks + Is / 32;
    g.down_blocks = (H + FUSE_DOWN_ROWS - 1) / FUSE_DOWN_ROWS;
    g.grid = g.expert_blocks > g.down_blocks ? g.expert_blocks : g.down_blocks;
    g.lines = g.expert_blocks;
    return g;
}

__device__ __forceinline__ unsigned long long ld_agent(const unsigned long long *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(unsigned long long *p, unsigned long long v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// everything this wave has requested from memory has arrived (rows on their way into LDS included)
__device__ __forceinline__ void memory_settled() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The workgroup's 32 activations (lanes 0..31 of the calling wave) as a digit image in LDS: PF_IMG_GROUP dwords of
// digits, the step, the sum of the integers (one group of image2_group's image).
__device__ __forceinline__ void image_group_lds(uint32_t *img, float v, int lane) {
    float m = fabsf(v);
#pragma unroll
    for (int k = 0; k < 4; k++) m = fmaxf(m, __int_as_float(dpp_row_step(__float_as_int(m), k)));
    m = fmaxf(m, __shfl_xor(m, 16));
    float step, inv;
    group_step2(m, step, inv);
    const int q = __float2int_rn(v * inv);
    int sum = q;
#pragma unroll
    for (int k = 0; k < 4; k++) sum += dpp_row_step(sum, k);
    sum += __shfl_xor(sum, 16);
    int d[PF_IMG_PLANES];
    image_digits(q, d);
    uint8_t *bytes = reinterpret_cast<uint8_t *>(img);
    if (lane < 32) {
#pragma unroll
        for (int p = 0; p < PF_IMG_PLANES; p++) bytes[32 * p + lane] = (uint8_t)d[p];
    }
    if (lane == 0) { img[PF_IMG_GROUP] = __float_as_uint(step); img[PF_IMG_GROUP + 1] = (uint32_t)sum; }
}

__device__ __forceinline__ void fuse_to_lds(const void *global, unsigned char *lds) {
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(global), reinterpret_cast<uint32_t *>(lds), 16, 0, 0);
}
__device__ __forceinline__ void fuse_to_lds_dword(const void *global, unsigned char *lds) {   // lane l at base + 4 l
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(global), reinterpret_cast<uint32_t *>(lds), 4, 0, 0);
}
template <int FMT> __host__ __device__ constexpr int fuse_stage_bytes() { return FMT == PF_Q4_K ? 3072 : 1280; }   // a wave's down items

// One (row, run) item a lane into the stage: Q4_K the row's header and the run's two halves; IQ2_XXS the run's piece and
// the dword around the block's scale.
__device__ __forceinline__ void item_request(const TileItem<PF_Q4_K> *, const uint8_t *chunk, int row, int run, unsigned char *stage) {
    fuse_to_lds(chunk + pf_q4t_header_at(row), stage);
    fuse_to_lds(chunk + pf_q4t_piece_at(run, 0, row), stage + 1024);
    fuse_to_lds(chunk + pf_q4t_piece_at(run, 1, row), stage + 2048);
}
__device__ __forceinline__ void item_request(const TileItem<PF_IQ2_XXS> *, const uint8_t *chunk, int row, int run, unsigned char *stage) {
    fuse_to_lds(chunk + pf_i2t_piece_at(run, row), stage);
    fuse_to_lds_dword(chunk + (pf_i2t_scale_at(row) & ~(size_t)3), stage + 1024);
}
__device__ __forceinline__ void item_take(TileItem<PF_Q4_K> &w, const unsigned char *stage, int lane, int) {
    w.hdr = *reinterpret_cast<const uint4 *>(stage + 16 * lane);
    w.piece[0] = *reinterpret_cast<const uint4 *>(stage + 1024 + 16 * lane);
    w.piece[1] = *reinterpret_cast<const uint4 *>(stage + 2048 + 16 * lane);
}
__device__ __forceinline__ void item_take(TileItem<PF_IQ2_XXS> &w, const unsigned char *stage, int lane, int row) {
    w.piece = *reinterpret_cast<const uint4 *>(stage + 16 * lane);
    const uint32_t both = *reinterpret_cast<const uint32_t *>(stage + 1024 + 4 * lane);
    w.dbits = row & 1 ? both >> 16 : both & 0xffffu;
}

// FMT: the format of every expert tensor (routed and shared)
template <int NPL, int FMT>
__global__ void __launch_bounds__(1024) pf_k_dec_fused(PfKernelArgs a, FuseGeometry geo) {
    extern __shared__ __align__(16) int fuse_lds[];   // (16-byte aligned: rows land here 16 bytes a lane)
    int *const lds = fuse_lds;
    __shared__ RouteLds R;
    __shared__ uint32_t early_expert;
    __shared__ __attribute__((aligned(16))) uint32_t act_image[PF_IMG_GROUP + 4];
    __shared__ float down_partial[17][FUSE_DOWN_ROWS];
    typedef TileGeometry<FMT> G;
    const int b = (int)blockIdx.x, H = a.hidden, K = a.top_k, E = a.experts, lane = pf_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool has_tile = b < geo.expert_blocks, has_rows = b < geo.down_blocks;
    const bool shared = has_tile && b >= geo.routed_blocks;
    const bool routed = has_tile && !shared;
    const int tiles = a.inter / 32, tiles_s = a.shared_inter / 32;
    const int u = routed ? b / tiles : K;
    const int tile = shared ? b - geo.routed_blocks : b % tiles, n0 = 32 * tile;
    const uint32_t tag = a.fuse_gen[0];
    const int n_base = FUSE_DOWN_ROWS * b;
    PfOutputRegs out_regs;
    if (has_rows && (int)threadIdx.x < FUSE_DOWN_ROWS && n_base + (int)threadIdx.x < H) pf_output_prefetch(a, 0, n_base + threadIdx.x, out_regs);
    const float shared_scale = a.shared_scale[0];
    FSTAMP(0);
    // LDS: IQ2_XXS: the signed-magnitude tables (32 KB) and the magnitude grid (2 KB); the waves' partial sums; then the
    // serial-order routing's arrays or, in their place, the slots' down items and the slots' activation images
    uint32_t *tables = reinterpret_cast<uint32_t *>(lds);
    uint32_t *grid = tables + table_words<FMT>();
    constexpr int GRID_WORDS = FMT == PF_IQ2_XXS ? 512 : 0;
    if (FMT == PF_IQ2_XXS && wave != 0) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.iq2_signed);
        for (int i = (int)threadIdx.x - 64; i < 2048; i += 960) reinterpret_cast<uint4 *>(tables)[i] = src[i];
        if (wave == 1) {
            const uint4 *g = reinterpret_cast<const uint4 *>(a.iq2_grid);
            reinterpret_cast<uint4 *>(grid)[lane] = g[lane];
            reinterpret_cast<uint4 *>(grid)[64 + lane] = g[64 + lane];
        }
    }
    float *partial = reinterpret_cast<float *>(grid + GRID_WORDS);   // [15 waves][64 lanes]
    float *scratch = partial + 15 * 64;
    unsigned char *stages = reinterpret_cast<unsigned char *>(scratch);                     // [K + 1][fuse_stage_bytes]
    const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
    const int image_words = (int)pf_image2_words(widest);
    uint32_t *images = reinterpret_cast<uint32_t *>(stages + (size_t)(K + 1) * fuse_stage_bytes<FMT>());   // [K + 1][image_words]
    const bool norm = a.norm_topk != 0;
    const int rounds = K + 1, first_rounds = routed ? u + 1 : 0;
    float v[NPL], s2[NPL], total = 0.0f, top_all = 0.0f;
    PfTopk<NPL> top;
    uint32_t my_key = 0;
    bool bad = false;
    if (wave == 0) {
        pf_load_row<NPL>(a.logits, E, lane, -INFINITY, v);
        pf_load_row<NPL>(a.logit_ssq, E, lane, 0.0f, s2);
#pragma unroll
        for (int j = 0; j < NPL; j++) bad |= lane * NPL + j < E && !pf_finite(v[j]);
        bad = __any(bad);
        if (!norm) {
            float m = v[0];
#pragma unroll
            for (int j = 1; j < NPL; j++) m = fmaxf(m, v[j]);
            top_all = pf_wave_max_fast(m);
#pragma unroll
            for (int j = 0; j < NPL; j++) total += expf(v[j] - top_all);
            total = pf_wave_sum(total);
        }
        top.setup(v, E, lane);
        for (int r = 0; r < first_rounds; r++) {
            const uint32_t best = top.pop();
            if (lane == r) my_key = best;
        }
        if (routed) {
            const uint32_t mine = (uint32_t)__builtin_amdgcn_readlane((int)my_key, u);
            if (lane == 0) early_expert = mine ? pf_key_id(mine) : 0xffffffffu;
        }
    }
    const Q4TilePlan plan = q4t_plan<FMT>(a, shared, has_tile ? n0 : 0);
    if (routed || FMT == PF_IQ2_XXS) __syncthreads();   // the early expert; the tables
    const uint32_t early = routed ? early_expert : 0u;
    const bool early_ok = early < (uint32_t)E;
    FSTAMP(1);
    TileItem<FMT> gu[Q4T_ITEMS];
    auto request_tile = [&](uint32_t e) {
        if (wave == 0 || !has_tile) return;
        const uint8_t *t = plan.base + (size_t)e * plan.expert_bytes;
#pragma unroll
        for (int k = 0; k < Q4T_ITEMS; k++) {
            const int it = wave - 1 + 15 * k;
            if (it < plan.items) q4t_load(gu[k], t + G::chunk_at(0, plan.kblocks, it >> 2), plan.row, it & 3);
        }
    };
    auto tile_products = [&]() {
        if (wave == 0 || !has_tile) return;
        const PfScalarWords image = (PfScalarWords)(uintptr_t)a.ximg;
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < Q4T_ITEMS; k++) {
            const int it = wave - 1 + 15 * k;
            if (it < plan.items) {
                const int g = 2 * it;
                sum += q4t_dot(gu[k], image + PF_IMG_GROUP * g, image + PF_IMG_GROUP * plan.groups + g, image + (PF_IMG_GROUP + 1) * plan.groups + g,
                               it & 3, tables);
            }
        }
        partial[(wave - 1) * 64 + lane] = sum;
    };
    // The routing wave requests this workgroup's down rows of every slot: lane (row r of eight, run) fetches what the same
    // lane of the slot's wave multiplies later.  id_of(s): the slot's expert.
    const int row_in_tile = (n_base & 31) + (lane & 7), my_run = lane >> 3;
    auto request_rows = [&](auto id_of) {
        const int kb_r = a.inter / 256, kb_s = a.shared_inter / 256;
#pragma unroll
        for (int s = 0; s < 16; s++) {
            if (s > K) break;
            const bool sh = s == K;
            uint32_t e = sh ? 0u : id_of(s);
            if (e >= (uint32_t)E) e = 0u;   // only reachable with nonfinite logits: the error word says so
            const int kblocks = sh ? kb_s : kb_r, runs = 4 * kblocks;
            const int run = my_run < runs ? my_run : 0;
            const int tensor = sh ? 6 : 3;
            const uint8_t *chunk = G::tensor(a, tensor) + (size_t)e * G::expert_bytes(a, tensor) + G::chunk_at(n_base / 32, kblocks, run >> 2);
            item_request(static_cast<const TileItem<FMT> *>(nullptr), chunk, row_in_tile, run & 3, stages + (size_t)s * fuse_stage_bytes<FMT>());
        }
    };
    request_tile(early_ok ? early : 0u);
    tile_products();
    if (wave == 0) {
        for (int r = first_rounds; r <= rounds; r++) {
            const uint32_t best = top.pop();
            if (lane == r) my_key = best;
        }
        uint32_t my_id;
        float my_z, my_s2, weight;
        bool close;
        const bool ambiguous = pf_topk_exact_order<NPL>(my_key, rounds + 1, v, s2, lane, my_id, my_z, my_s2);
        pf_route_finish_wave(my_z, my_s2, K, rounds, norm, H, total, top_all, lane, weight, close);
        close |= ambiguous;
        if (lane < K) { R.ids[lane] = my_id; R.weights[lane] = weight; }
        if (lane == 0) { R.close[0] = close ? 1u : 0u; R.nonfinite[0] = bad ? 1u : 0u; }
        if (has_rows && !close) request_rows([&](int s) { return (uint32_t)__builtin_amdgcn_readlane((int)my_id, s); });
    }
    __syncthreads();
    FSTAMP(2);
    const bool again = R.close[0] != 0;
    if (again) {
        // a close call: the token is routed again in the reference's order (in the LDS the down rows land in: none were requested)
        q4t_route_fix<NPL>(reinterpret_cast<const float *>(a.w[0]), a.x, a.logits, a.logit_ssq, E, K, norm, H,
                           (int)(scratch - reinterpret_cast<float *>(lds)), &R);
        if (wave == 0 && has_rows) request_rows([&](int s) { return R.ids[s]; });
    } else if (threadIdx.x == 0) {
        R.close_mask = 0;
        R.bad = R.nonfinite[0];
    }
    uint32_t e = routed ? R.ids[u] : 0u;
    if (routed && e != early && e < (uint32_t)E) {   // the early guess came from truncated keys, or the token was routed again
        __syncthreads();
        request_tile(e);
        tile_products();
        __syncthreads();
    }
    if (b == 0) {
        if (!again) __syncthreads();   // R.bad above; the re-route ends with a barrier of its own
        for (int q = threadIdx.x; q < K; q += blockDim.x) {
            a.ids[q] = R.ids[q];
            a.route_weights[q] = R.weights[q];
        }
        if (threadIdx.x == 0) {
            if (R.bad) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
            if (R.close_mask) atomicAdd(a.exact_rows, 1u);
            if (R.close_mask == 2u) atomicAdd(a.exact_rows + 1, 1u);
        }
    }
    if (routed && e >= (uint32_t)E && threadIdx.x == 0) atomicOr(a.error_word, PF_HIP_ERR_BOUNDS | PF_HIP_ERR_NONFINITE);   // nonfinite logits
    // wave 1: the gate and up rows' sums over the waves in wave order, SwiGLU, the 32 activations as one group's image,
    // and the image as this workgroup's line, once per replica
    if (wave == 1 && has_tile) {
        float sum = 0.0f;
        for (int w = 0; w < 15; w++) sum += partial[w * 64 + lane];
        const float up = __shfl(sum, (lane & 31) + 32);
        float act = pf_silu(sum) * up;
        if (lane < 32 && !pf_finite(act)) { atomicOr(a.error_word, PF_HIP_ERR_NONFINITE); act = 0.0f; }
        image_group_lds(act_image, act, lane);
        pf_wave_lds_fence();
        if (lane < FUSE_PAIRS) {
            const unsigned long long pair = ((unsigned long long)tag << 32) | act_image[lane];
            unsigned long long *line = reinterpret_cast<unsigned long long *>(a.fuse_lines + (size_t)b * FUSE_LINE) + lane;
#pragma unroll
            for (int r = 0; r < FUSE_REPLICAS; r++) st_agent(line + (size_t)r * geo.lines * (FUSE_LINE / 2), pair);
        }
    }
    if (wave == 0) memory_settled();   // the down rows this wave requested have landed
    __syncthreads();
    FSTAMP(3);
    if (!has_rows) return;
    if (wave <= K) {
        const int s = wave;
        const bool sh = s == K;
        const int groups = sh ? tiles_s : tiles, runs = groups / 2;
        uint32_t *mine = images + (size_t)s * image_words;
        // the slot's lines: its groups' pairs go round the lanes
        const unsigned long long *src = reinterpret_cast<const unsigned long long *>(
            a.fuse_lines + ((size_t)(b % FUSE_REPLICAS) * geo.lines + (size_t)s * tiles) * FUSE_LINE);
        constexpr int TURNS = (16 * FUSE_PAIRS + 63) / 64;   // at most 16 groups a slot
        const int wanted = groups * FUSE_PAIRS;
        unsigned long long got[TURNS];
        bool ok = false;
        for (int spin = 0; spin < FUSE_SPIN_LIMIT && !ok; spin++) {
            bool here = true;
#pragma unroll
            for (int j = 0; j < TURNS; j++) {
                const int i = lane + 64 * j;
                if (i < wanted) {
                    const int group = i / FUSE_PAIRS, p = i - group * FUSE_PAIRS;
                    got[j] = ld_agent(src + (size_t)group * (FUSE_LINE / 2) + p);
                    here &= (uint32_t)(got[j] >> 32) == tag;
                }
            }
            ok = __all(here);
            if (!ok) __builtin_amdgcn_s_sleep(1);
        }
        if (!ok && lane == 0) atomicOr(a.error_word, PF_HIP_ERR_TIMEOUT);   // a workgroup never came: the launch still ends
        FSTAMP(4);
#pragma unroll
        for (int j = 0; j < TURNS; j++) {
            const int i = lane + 64 * j;
            if (i < wanted) {
                const int group = i / FUSE_PAIRS, p = i - group * FUSE_PAIRS;
                const uint32_t word = (uint32_t)got[j];
                if (p < PF_IMG_GROUP) mine[PF_IMG_GROUP * group + p] = word;
                else if (p == PF_IMG_GROUP) mine[PF_IMG_GROUP * groups + group] = word;
                else mine[(PF_IMG_GROUP + 1) * groups + group] = word;
            }
        }
        pf_wave_lds_fence();
        float dot = 0.0f;
        if (my_run < runs) {
            TileItem<FMT> item;
            item_take(item, stages + (size_t)s * fuse_stage_bytes<FMT>(), lane, row_in_tile);
            dot = down_dot(item, my_run & 3, mine, my_run, groups, grid);
        }
        // the row's runs: lanes r, r + 8, ..., r + 56
        dot += __shfl_xor(dot, 8);
        dot += __shfl_xor(dot, 16);
        dot += __shfl_xor(dot, 32);
        if (lane < FUSE_DOWN_ROWS) down_partial[s][lane] = dot;
    }
    __syncthreads();
    const int n = n_base + threadIdx.x;
    if ((int)threadIdx.x < FUSE_DOWN_ROWS && n < H) {
        float sum = 0.0f;
#pragma unroll
        for (int slot = 0; slot < 16; slot++)   // slot order, as src/qwen4_moe.c:362-372
            if (slot < K) sum += R.weights[slot] * down_partial[slot][threadIdx.x];
        const float y = sum + shared_scale * down_partial[K][threadIdx.x];
        if (!pf_output_commit(a, 0, n, y, out_regs)) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
    }
    FSTAMP(5);
}

// Layers the fused launch takes: one token, every expert tensor Q4_K or every one IQ2_XXS with the tile-ordered copies
// kept, intermediate widths of at most 512 (a lane holds one run of a down row), whole groups of eight output rows,
// the workspace's lines, and a device with a compute unit for every workgroup.
static int device_compute_units() {
    static int units = -1;
    if (units < 0) {
        int device = 0, count = 0;
        if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) count = 0;
        units = count;
    }
    return units;
}

template <int FMT>
static bool fused_applies(const PfKernelArgs &a) {
    if (!a.fuse_lines || !a.fuse_gen || a.slots) return false;
    if (a.inter % 256 || a.shared_inter % 256 || a.inter > 512 || a.shared_inter > 512 || a.hidden % 32 || a.top_k > 15) return false;
    const FuseGeometry g = fuse_geometry(a.hidden, a.top_k, a.inter, a.shared_inter);
    return g.grid <= device_compute_units();
}

template <int NPL, int FMT>
static void launch_fused_lists(const PfKernelArgs &a, const FuseGeometry &g, size_t lds, hipStream_t stream) {
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_fused<NPL, FMT>), hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
        configured = true;
    }
    hipLaunchKernelGGL((pf_k_dec_fused<NPL, FMT>), dim3(g.grid), dim3(1024), lds, stream, a, g);
}

template <int FMT>
static void launch_fused(const PfKernelArgs &a, hipStream_t stream) {
    const FuseGeometry g = fuse_geometry(a.hidden, a.top_k, a.inter, a.shared_inter);
    const size_t widest = a.inter > a.shared_inter ? a.inter : a.shared_inter;
    const size_t fix = pf_route_fix_lds_floats(a.hidden, a.experts) * 4;
    const size_t rows = (size_t)(a.top_k + 1) * (fuse_stage_bytes<FMT>() + pf_image2_words(widest) * 4);
    const size_t lds = (size_t)table_words<FMT>() * 4 + (FMT == PF_IQ2_XXS ? 2048 : 0) + (size_t)15 * 64 * 4 + (fix > rows ? fix : rows);
    const int all = (a.experts + 63) / 64;
    if (all <= 1) launch_fused_lists<1, FMT>(a, g, lds, stream);
    else if (all <= 2) launch_fused_lists<2, FMT>(a, g, lds, stream);
    else if (all <= 4) launch_fused_lists<4, FMT>(a, g, lds, stream);
    else if (all <= 8) launch_fused_lists<8, FMT>(a, g, lds, stream);
    else launch_fused_lists<16, FMT>(a, g, lds, stream);
}

#if PF_DECODE_PART == 0
// ---- IQ2_XXS in tile order ---------------------------------------------------------------------------
// From the split device layout (64-byte payloads row by row, half scales apart) to the chunks of pf_decode_addr.h per
// (32-row tile, 256-block): per 64-weight run the rows' 16-byte pieces, then the 32 rows' scales.  One thread per 16-byte piece or
// per scale; rows is a multiple of 32.
__global__ void pf_k_iq2_tile(const uint8_t *payload, const uint16_t *scales, uint8_t *dst, size_t rows, int blocks_per_row) {
    const PfMove m = pf_iq2_tile_move((size_t)blockIdx.x * blockDim.x + threadIdx.x, rows, blocks_per_row);
    if (!m.active) return;
    if (m.from == 0) *reinterpret_cast<uint4 *>(dst + m.dst) = *reinterpret_cast<const uint4 *>(payload + m.src);
    else *reinterpret_cast<uint16_t *>(dst + m.dst) = *reinterpret_cast<const uint16_t *>(reinterpret_cast<const uint8_t *>(scales) + m.src);
}

void pf_launch_iq2_tile(const uint8_t *d_payload, const uint16_t *d_scales, uint8_t *d_dst, size_t rows, int blocks_per_row,
                        hipStream_t stream) {
    const size_t threads = pf_iq2_tile_threads(rows, blocks_per_row);
    hipLaunchKernelGGL(pf_k_iq2_tile, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, d_payload, d_scales, d_dst, rows,
                       blocks_per_row);
}

// ---- Q8_0 in tile order (the profiles' shared gate and up) ------------------------------------------------
// From the split device layout (32 code bytes per block row by row, half scales apart) to the chunks of
// pf_decode_addr.h per (32-row tile, 64-weight run).  One thread per 16-byte piece or per pair of scales.
__global__ void pf_k_q8_tile(const uint8_t *payload, const uint16_t *scales, uint8_t *dst, size_t rows, int blocks_per_row) {
    const PfMove m = pf_q8_tile_move((size_t)blockIdx.x * blockDim.x + threadIdx.x, rows, blocks_per_row);
    if (!m.active) return;
    if (m.from == 0) {
        *reinterpret_cast<uint4 *>(dst + m.dst) = *reinterpret_cast<const uint4 *>(payload + m.src);
    } else {
        const uint8_t *s = reinterpret_cast<const uint8_t *>(scales);
        *reinterpret_cast<uint32_t *>(dst + m.dst) =
            (uint32_t)*reinterpret_cast<const uint16_t *>(s + m.src) | ((uint32_t)*reinterpret_cast<const uint16_t *>(s + m.src2) << 16);
    }
}

void pf_launch_q8_tile(const uint8_t *d_payload, const uint16_t *d_scales, uint8_t *d_dst, size_t rows, int blocks_per_row,
                       hipStream_t stream) {
    const size_t threads = pf_q8_tile_threads(rows, blocks_per_row);
    hipLaunchKernelGGL(pf_k_q8_tile, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, d_payload, d_scales, d_dst, rows,
                       blocks_per_row);
}

// ---- IQ2_XXS upload split -------------------------------------------------------------------------
__global__ void pf_k_iq2_split(const uint8_t *gguf, uint8_t *payload, uint16_t *scales, size_t blocks) {
    const PfMove m = pf_iq2_split_move((size_t)blockIdx.x * blockDim.x + threadIdx.x, blocks);   // one 16-bit word of a block per thread
    if (!m.active) return;
    const uint16_t v = *reinterpret_cast<const uint16_t *>(gguf + m.src);
    *reinterpret_cast<uint16_t *>((m.to ? reinterpret_cast<uint8_t *>(scales) : payload) + m.dst) = v;
}

void pf_launch_iq2_split(const uint8_t *d_gguf, uint8_t *d_payload, uint16_t *d_scales, size_t blocks,
                         hipStream_t stream) {
    const size_t threads = pf_iq2_split_threads(blocks);
    if (!threads) return;
    hipLaunchKernelGGL(pf_k_iq2_split, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, d_gguf,
                       d_payload, d_scales, blocks);
}

// The same for any format whose block leads with its scale (Q8_0: 2 + 32 bytes, MXFP4: 1 + 16): one
// byte per thread.
__global__ void pf_k_block_split(const uint8_t *gguf, uint8_t *payload, uint8_t *scales, size_t blocks, int block_bytes,
                                 int header_bytes) {
    const PfMove m = pf_block_split_move((size_t)blockIdx.x * blockDim.x + threadIdx.x, blocks, block_bytes, header_bytes);
    if (!m.active) return;
    (m.to ? scales : payload)[m.dst] = gguf[m.src];
}

void pf_launch_block_split(const uint8_t *d_gguf, uint8_t *d_payload, uint8_t *d_scales, size_t blocks,
                           int block_bytes, int header_bytes, hipStream_t stream) {
    const size_t threads = pf_block_split_threads(blocks, block_bytes);
    if (!threads) return;
    hipLaunchKernelGGL(pf_k_block_split, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, d_gguf,
                       d_payload, d_scales, blocks, block_bytes, header_bytes);
}

#endif

// ---- dispatch ----------------------------------------------------------------------------------------
// The format combinations with decode kernels: one format throughout (Q4_K or IQ2_XXS), and the two
// profiles of real checkpoints (src/qwen4_config.c:197-216, src/qwen4_weights.c:91-99): IQ2_XXS gate/up
// with Q2_K down, Q4_K gate/up with MXFP4 down, the shared expert in Q8_0.
static int decode_combination(const uint32_t type[8]) {
    const uint32_t g = type[1], d = type[3], s = type[4];
    if (type[2] != g || type[5] != s || type[6] != s) return 0;
    if (g == PF_Q4_K && d == PF_Q4_K && s == PF_Q4_K) return 1;
    if (g == PF_IQ2_XXS && d == PF_IQ2_XXS && s == PF_IQ2_XXS) return 2;
    if (g == PF_IQ2_XXS && d == PF_Q2_K && s == PF_Q8_0) return 3;
    if (g == PF_Q4_K && d == PF_MXFP4 && s == PF_Q8_0) return 4;
    return 0;
}

// A row of k values in a format: whole blocks, and whole 64-value segments for the lanes.
static bool row_width_ok(uint32_t type, uint32_t k) {
    const bool big = type == PF_Q4_K || type == PF_IQ2_XXS || type == PF_Q2_K;
    return k && k % (big ? 256 : 64) == 0;
}

#if PF_DECODE_PART == 0
// Widths: hidden 512..2560 in whole 256-blocks (2560 is the checkpoints' width), intermediate widths
// 256..2048 in whole 64-value segments (640 in the checkpoints); the routed down projection may be
// stored wider than its logical width only as Q2_K (640 padded to 768): the padding is never read.
bool pf_decode_supported(const PfHipMoeDesc &d) {
    if (!decode_combination(d.type)) return false;
    if (d.hidden < 512 || d.hidden > 64 * 4 * ROUTER_CHUNKS || d.hidden % 256) return false;
    if (d.inter < 256 || d.inter > 2048 || d.shared_inter < 256 || d.shared_inter > 2048 || d.inter % 64 || d.shared_inter % 64)
        return false;
    if (d.shared_inter > 4 * d.inter) return false;
    if (!row_width_ok(d.type[1], d.hidden) || !row_width_ok(d.type[4], d.hidden) || !row_width_ok(d.type[6], d.shared_inter) ||
        !row_width_ok(d.type[3], d.down_physical))
        return false;
    if (d.down_physical < d.inter || (d.down_physical != d.inter && d.type[3] != PF_Q2_K)) return false;
    if (d.experts > 1024 || d.top_k > 15 || d.top_k * PF_DECODE_MAX_TOKENS > 64 || d.top_k >= d.experts) return false;
    // the down kernel keeps one digit image per slot (and the IQ2_XXS tables) in LDS
    const uint32_t widest = d.inter > d.shared_inter ? d.inter : d.shared_inter;
    if ((size_t)(d.top_k + 1) * image_words((int)widest) * 4 + 32 * 1024 > 140 * 1024) return false;
    return true;
}

#endif

template <int FG, int FS, int NT, int NPL, int SPL>
static void launch_gate_up(const PfKernelArgs &a, dim3 grid, size_t lds, hipStream_t stream, int routed_blocks,
                           int shared_blocks, int parts, int chunk, int tile) {
    // more workgroups than compute units: routing once, in a launch of its own, beats every workgroup repeating it
    const bool split = grid.x > 256;
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_gate_up<FG, FS, NT, NPL, SPL>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        configured = true;
    }
    if (split)
        hipLaunchKernelGGL((pf_k_dec_gate_up<FG, FS, NT, NPL, SPL>), dim3(1), dim3(1024), lds, stream, a, routed_blocks,
                           shared_blocks, parts, chunk, tile, 1);
    hipLaunchKernelGGL((pf_k_dec_gate_up<FG, FS, NT, NPL, SPL>), grid, dim3(1024), lds, stream, a, routed_blocks, shared_blocks,
                       parts, chunk, tile, split ? 2 : 0);
}

void pf_launch_dec_router(const PfKernelArgs &a, int tokens, int router_blocks, hipStream_t stream);
#if PF_DECODE_PART == 0
void pf_launch_dec_router(const PfKernelArgs &a, int tokens, int router_blocks, hipStream_t stream) {
    // the router's rows, the shared router's row, then the tokens' digit images (2048 values per workgroup);
    // beyond four tokens: groups of four along the grid's second dimension
    const dim3 grid(router_blocks + 1 + tokens * ((a.hidden + 2047) / 2048), (tokens + 3) / 4), block(256);
    switch (tokens) {
    case 1: hipLaunchKernelGGL((pf_k_dec_router<1>), grid, block, 0, stream, a, router_blocks, tokens); break;
    case 2: hipLaunchKernelGGL((pf_k_dec_router<2>), grid, block, 0, stream, a, router_blocks, tokens); break;
    case 3: hipLaunchKernelGGL((pf_k_dec_router<3>), grid, block, 0, stream, a, router_blocks, tokens); break;
    default: hipLaunchKernelGGL((pf_k_dec_router<4>), grid, block, 0, stream, a, router_blocks, tokens); break;
    }
}
#endif

template <int FD, int FS, int NT, int SPL, int MAXT>
static void launch_down_bounded(const PfKernelArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t stream, int row_blocks,
                                int rows_per_block, int image_pitch) {
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_down<FD, FS, NT, SPL, MAXT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
        configured = true;
    }
    hipLaunchKernelGGL((pf_k_dec_down<FD, FS, NT, SPL, MAXT>), grid, block, lds, stream, a, row_blocks, rows_per_block,
                       image_pitch);
}

template <int FD, int FS, int NT, int SPL>
static void launch_down(const PfKernelArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t stream, int row_blocks,
                        int rows_per_block, int image_pitch) {
    constexpr int TIGHT = (SPL > 1) ? 768 : 1024;
    if (SPL > 1 && block.x <= 768)
        launch_down_bounded<FD, FS, NT, SPL, TIGHT>(a, grid, block, lds, stream, row_blocks, rows_per_block, image_pitch);
    else
        launch_down_bounded<FD, FS, NT, SPL, 1024>(a, grid, block, lds, stream, row_blocks, rows_per_block, image_pitch);
}

// Layers the kernels whose lanes are weight rows take, one token per grid row, for up to PF_TILE_DECODE_MAX_TOKENS
// tokens: every expert tensor Q4_K, or every one IQ2_XXS, with its tile-ordered copy kept; the two checkpoint profiles
// with the tile-ordered copies of their routed gate and up tensors and of the shared expert's Q8_0 gate and up (their
// down tensors are read row by row).  Returns the combination as decode_combination numbers it, 0 for other layers.
#if PF_DECODE_PART == 0
int pf_decode_tile_layer(const PfHipMoeDesc &d, const uint8_t *const q4k_tiled[8], const uint8_t *const iq2_tiled[8],
                         const uint8_t *const q8_tiled[8]) {
    const int combination = decode_combination(d.type);
    if (!combination) return 0;
    const uint32_t format = d.type[1];
    const uint8_t *const *tiled = format == PF_Q4_K ? q4k_tiled : iq2_tiled;
    bool fits = d.hidden % 256 == 0 && 4 * (d.hidden / 256) <= 15 * Q4T_ITEMS && d.top_k < d.experts && d.top_k <= 15 &&
                d.experts <= 1024;
    if (combination <= 2) {
        for (int t = 1; t <= 6; t++) fits &= tiled[t] != nullptr;
        fits &= d.inter % 256 == 0 && d.shared_inter % 256 == 0 && d.down_physical == d.inter;
    } else {
        fits &= tiled[1] && tiled[2] && q8_tiled[4] && q8_tiled[5];
        fits &= d.inter % 64 == 0 && d.shared_inter % 64 == 0 && row_width_ok(d.type[3], d.down_physical) &&
                row_width_ok(d.type[6], d.shared_inter) && d.down_physical >= d.inter;
    }
    // kernel 3's LDS: per slot the activation row's image and the products of up to 16 rows, and the IQ2_XXS grids
    const size_t widest = d.inter > d.shared_inter ? d.inter : d.shared_inter;
    fits &= (size_t)(d.top_k + 1) * ((pf_image2_words(widest) + 16 * (widest / 64)) * 4 + 2048) <= Q4T_DOWN_LDS;
    return fits ? combination : 0;
}
#endif

#if PF_DECODE_PART == 0
void pf_decode_fused_scratch(const PfHipMoeDesc &d, size_t *line_bytes) {
    *line_bytes = 0;
    const int combination = decode_combination(d.type);
    if (combination != 1 && combination != 2) return;
    if (d.inter % 256 || d.shared_inter % 256 || d.inter > 512 || d.shared_inter > 512 || d.hidden % 32 || d.down_physical != d.inter || d.top_k > 15) return;
    const FuseGeometry g = fuse_geometry((int)d.hidden, (int)d.top_k, (int)d.inter, (int)d.shared_inter);
    *line_bytes = (size_t)FUSE_REPLICAS * g.lines * FUSE_LINE * 4;
}
#endif

static PfHipMoeDesc desc_of(const PfKernelArgs &a) {
    PfHipMoeDesc d = {};
    d.hidden = a.hidden; d.experts = a.experts; d.top_k = a.top_k; d.inter = a.inter; d.shared_inter = a.shared_inter;
    d.down_physical = a.down_physical;
    for (int t = 0; t < 8; t++) d.type[t] = a.type[t];
    return d;
}

// the routing in a launch of its own, ahead of a gate/up kernel that is given the experts
// (from three tokens on: with two the routing launch costs more than the workgroups' own routing, 24.8 against 22.9 us,
// with one 18.4 against 16.5)
#ifndef PF_ROUTE_FIRST_FROM
#define PF_ROUTE_FIRST_FROM 3
#endif
template <bool POOL>
static bool routes_first(const PfKernelArgs &a, int tokens) {
    return !POOL && tokens >= PF_ROUTE_FIRST_FROM && a.hidden <= 64 * Q4G_ITEMS * Q4G_WAVES && a.top_k <= 15;
}

template <int FG, int FD, int FS, bool POOL = false>
static void launch_q4t_experts(const PfKernelArgs &a, int tokens, hipStream_t stream, int last) {
    const int H = a.hidden, I = a.inter, Is = a.shared_inter, K = a.top_k;
    // kernel 2: every workgroup extracts the maxima up to its own slot from all of its token's logits; with several
    // tokens the routing runs first, in a launch of its own
    if (routes_first<POOL>(a, tokens)) {   // four launches: `last` counts them
        launch_dec_route(a, tokens, stream);
        if (last < 3) return;
        launch_gate_up_given<FG, FS>(a, tokens, stream);
        if (last < 4) return;
    } else {
        launch_gate_up_q4t<FG, FS, POOL>(a, tokens, stream);
        if (last < 3) return;
    }
    if constexpr (!POOL && (FD == PF_Q4_K || FD == PF_IQ2_XXS) && (FS == PF_Q4_K || FS == PF_IQ2_XXS)) {
        if (down_rows64_applies<FD, FS>(a, tokens)) {
            launch_down_rows64<FD, FS>(a, tokens, stream);
            return;
        }
    }
    const size_t widest = I > Is ? I : Is;
    constexpr bool GRID = FD == PF_IQ2_XXS || FS == PF_IQ2_XXS;
    // rows per workgroup: eight in the tile order; for down tensors kept row by row the fewest that leave no more
    // workgroups than compute units (256 on this GPU), so that a hidden width of 2560 runs ten rows in one round
    int rows = 8;
    if (!tile_ordered<FD>() && !tile_ordered<FS>()) {
        rows = (H + 255) / 256;
        while (rows < 16 && H % rows) rows++;
        if (H % rows || rows > 16) rows = 8;
    }
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_dec_down_q4t<FD, FS, POOL>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)Q4T_DOWN_LDS);
        configured = true;
    }
    hipLaunchKernelGGL((pf_k_dec_down_q4t<FD, FS, POOL>), dim3(H / rows, tokens), dim3(64 * (K + 1)),
                       (GRID ? 2048 * (size_t)(K + 1) : 0) + (size_t)(K + 1) * (pf_image2_words(widest) + rows * (widest / 64)) * 4, stream, a, rows);
}

template <int FG, int FD, int FS>
static void launch_decode_q4t(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    const int last = stage_limit ? stage_limit : 4;
    pf_launch_dec_router(a, tokens, (a.experts + 3) / 4, stream);
    if (last < 2) return;
    if constexpr (FG == FD && FG == FS && (FG == PF_Q4_K || FG == PF_IQ2_XXS)) {
        if (tokens == 1 && fused_applies<FG>(a)) {
            launch_fused<FG>(a, stream);
            return;
        }
    }
    launch_q4t_experts<FG, FD, FS>(a, tokens, stream, last);
}

// FG: format of the routed gate and up tensors, FD: of the routed down tensor, FS: of the shared expert
template <int FG, int FD, int FS, int NT, int SPL2>
static void launch_decode_passes(const PfKernelArgs &a, hipStream_t stream, int stage_limit) {
    const int H = a.hidden, I = a.inter, Is = a.shared_inter, E = a.experts, K = a.top_k;
    const size_t tab2 = (FG == PF_IQ2_XXS || FS == PF_IQ2_XXS) ? 8192 * 4 : 0;
    const size_t tab3 = (FD == PF_IQ2_XXS || FS == PF_IQ2_XXS) ? 8192 * 4 : 0;
    // kernel 1 (stage_limit, profiling: launch only the first so many kernels; 0 = all)
    const int router_blocks = (E + 3) / 4, last = stage_limit ? stage_limit : 3;
    pf_launch_dec_router(a, NT, router_blocks, stream);
    if (last < 2) return;
    // kernel 2: the candidate stage uses up to 8 of waves 0..11 per token
    // 32 units per workgroup: every workgroup repeats the routing, and one workgroup per compute
    // unit measured faster than two half as long
    const int tile = 32;
    const int routed_blocks = NT * K * (I / tile), shared_blocks = Is / tile;
    const size_t lds2 = tab2 + (size_t)NT * image_words(H) * 4 + ((size_t)H + 3 * (size_t)E) * 4;
    int parts = NT == 1 ? 8 : NT == 2 ? 6 : NT == 3 ? 4 : 3;
    while (parts > 1 && (E + parts - 1) / parts < 64) parts--;
    const int chunk = (E + parts - 1) / parts, npl = (chunk + 63) / 64;
    // compute units left over by the tiles (256 on this GPU) warm the L2 for the down kernel, whose
    // row blocks must then spread evenly over the eight XCDs
    const int rows_next = down_block_rows(H, I), row_blocks_next = (H + rows_next - 1) / rows_next;
    int prefetch_blocks = (256 - routed_blocks - shared_blocks) / 8 * 8;
    if (prefetch_blocks < 8 || row_blocks_next % 8) prefetch_blocks = 0;
    dim3 g2(routed_blocks + shared_blocks + prefetch_blocks);
    bool tile_order = false;
    if constexpr (NT == 1 && (FG == PF_Q4_K || FG == PF_IQ2_XXS) && (FS == FG || FS == PF_Q8_0)) tile_order = q4t_gate_up_applies<FG, FS>(a);
    if constexpr (NT == 1 && (FG == PF_Q4_K || FG == PF_IQ2_XXS) && (FS == FG || FS == PF_Q8_0)) {
        if (tile_order) launch_gate_up_q4t<FG, FS>(a, 1, stream);   // it publishes the unique-expert table kernel 3 below reads
    }
    if (tile_order) {}
    else if (npl <= 1) launch_gate_up<FG, FS, NT, 1, SPL2>(a, g2, lds2, stream, routed_blocks, shared_blocks, parts, chunk, tile);
    else if (npl <= 2) launch_gate_up<FG, FS, NT, 2, SPL2>(a, g2, lds2, stream, routed_blocks, shared_blocks, parts, chunk, tile);
    else if (npl <= 4) launch_gate_up<FG, FS, NT, 4, SPL2>(a, g2, lds2, stream, routed_blocks, shared_blocks, parts, chunk, tile);
    else launch_gate_up<FG, FS, NT, 8, SPL2>(a, g2, lds2, stream, routed_blocks, shared_blocks, parts, chunk, tile);   // experts <= 1024
    if (last < 3) return;
    // kernel 3
    const int rows_per_block = down_block_rows(H, I), row_blocks = (H + rows_per_block - 1) / rows_per_block;
    const int image_pitch = image_words(I > Is ? I : Is);
    const size_t lds3 = tab3 + (size_t)(K + 1) * image_pitch * 4;
    if (row_passes(I) > 1 || row_passes(Is) > 1)
        launch_down<FD, FS, NT, 2>(a, dim3(NT * row_blocks), dim3(64 * (K + 1)), lds3, stream, row_blocks, rows_per_block, image_pitch);
    else
        launch_down<FD, FS, NT, 1>(a, dim3(NT * row_blocks), dim3(64 * (K + 1)), lds3, stream, row_blocks, rows_per_block, image_pitch);
}

// SPL2: passes over a row of `hidden` values in kernel 2 (2 only for widths such as 2560)
template <int FG, int FD, int FS, int NT>
static void launch_decode(const PfKernelArgs &a, hipStream_t stream, int stage_limit) {
    if (row_passes(a.hidden) > 1) launch_decode_passes<FG, FD, FS, NT, 2>(a, stream, stage_limit);
    else launch_decode_passes<FG, FD, FS, NT, 1>(a, stream, stage_limit);
}

template <int FG, int FD, int FS>
static void launch_decode_tokens(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    switch (tokens) {
    case 1: launch_decode<FG, FD, FS, 1>(a, stream, stage_limit); break;
    case 2: launch_decode<FG, FD, FS, 2>(a, stream, stage_limit); break;
    case 3: launch_decode<FG, FD, FS, 3>(a, stream, stage_limit); break;
    default: launch_decode<FG, FD, FS, 4>(a, stream, stage_limit); break;
    }
}

void pf_launch_decode_q4k(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_decode_iq2(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_decode_q2profile(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_decode_q4profile(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit);
void pf_launch_decode_q4profile_experts(const PfKernelArgs &a, int tokens, hipStream_t stream);
void pf_launch_decode_iq2_experts(const PfKernelArgs &a, int tokens, hipStream_t stream);
void pf_launch_decode_q2profile_experts(const PfKernelArgs &a, int tokens, hipStream_t stream);

#if PF_DECODE_PART == 0
void pf_launch_decode_q4k(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    if (pf_decode_tile_layer(desc_of(a), a.wt, a.wi, a.wq) == 1) launch_decode_q4t<PF_Q4_K, PF_Q4_K, PF_Q4_K>(a, tokens, stream, stage_limit);
    else launch_decode_tokens<PF_Q4_K, PF_Q4_K, PF_Q4_K>(a, tokens, stream, stage_limit);
}

void pf_launch_decode_stream_experts(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    switch (decode_combination(a.type)) {
    case 2: pf_launch_decode_iq2_experts(a, tokens, stream); break;
    case 3: pf_launch_decode_q2profile_experts(a, tokens, stream); break;
    case 4: pf_launch_decode_q4profile_experts(a, tokens, stream); break;
    default: launch_q4t_experts<PF_Q4_K, PF_Q4_K, PF_Q4_K, true>(a, tokens, stream, 3);
    }
}

int pf_decode_launches(const PfKernelArgs &a, int tokens) {
    const int combination = pf_decode_tile_layer(desc_of(a), a.wt, a.wi, a.wq);
    if (tokens != 1) return combination != 0 && routes_first<false>(a, tokens) ? 4 : 3;
    if (combination == 1) return fused_applies<PF_Q4_K>(a) ? 2 : 3;
    if (combination == 2) return fused_applies<PF_IQ2_XXS>(a) ? 2 : 3;
    return 3;
}

void pf_launch_decode(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    switch (decode_combination(a.type)) {
    case 1: pf_launch_decode_q4k(a, tokens, stream, stage_limit); break;
    case 2: pf_launch_decode_iq2(a, tokens, stream, stage_limit); break;
    case 3: pf_launch_decode_q2profile(a, tokens, stream, stage_limit); break;
    case 4: pf_launch_decode_q4profile(a, tokens, stream, stage_limit); break;
    default: break;   // pf_decode_supported keeps other combinations away
    }
}
#elif PF_DECODE_PART == 1
void pf_launch_decode_iq2(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    if (pf_decode_tile_layer(desc_of(a), a.wt, a.wi, a.wq) == 2)
        launch_decode_q4t<PF_IQ2_XXS, PF_IQ2_XXS, PF_IQ2_XXS>(a, tokens, stream, stage_limit);
    else launch_decode_tokens<PF_IQ2_XXS, PF_IQ2_XXS, PF_IQ2_XXS>(a, tokens, stream, stage_limit);
}

void pf_launch_decode_iq2_experts(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    launch_q4t_experts<PF_IQ2_XXS, PF_IQ2_XXS, PF_IQ2_XXS, true>(a, tokens, stream, 3);
}
#elif PF_DECODE_PART == 2
void pf_launch_decode_q2profile(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    if (pf_decode_tile_layer(desc_of(a), a.wt, a.wi, a.wq) == 3)
        launch_decode_q4t<PF_IQ2_XXS, PF_Q2_K, PF_Q8_0>(a, tokens, stream, stage_limit);
    else launch_decode_tokens<PF_IQ2_XXS, PF_Q2_K, PF_Q8_0>(a, tokens, stream, stage_limit);
}

void pf_launch_decode_q2profile_experts(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    launch_q4t_experts<PF_IQ2_XXS, PF_Q2_K, PF_Q8_0, true>(a, tokens, stream, 3);
}
#else
void pf_launch_decode_q4profile(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    if (pf_decode_tile_layer(desc_of(a), a.wt, a.wi, a.wq) == 4)
        launch_decode_q4t<PF_Q4_K, PF_MXFP4, PF_Q8_0>(a, tokens, stream, stage_limit);
    else launch_decode_tokens<PF_Q4_K, PF_MXFP4, PF_Q8_0>(a, tokens, stream, stage_limit);
}

void pf_launch_decode_q4profile_experts(const PfKernelArgs &a, int tokens, hipStream_t stream) {
    launch_q4t_experts<PF_Q4_K, PF_MXFP4, PF_Q8_0, true>(a, tokens, stream, 3);
}
#endif
