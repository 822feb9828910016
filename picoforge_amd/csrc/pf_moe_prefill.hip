// Prefill path: a chunk of tokens through one MoE layer as grouped matrix products on the
// matrix cores.
//
//   pf_k_rows_to_half   f32 rows -> power-of-two scaled fp16 pairs (high + low part) and the
//                       per-32-group sums, the scale, max^2, finite check
//   pf_k_pf_router      router logits [T, E] by FP32 MFMA
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
#include "pf_upload_addr.h"

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

// halfs per row of a converted matrix: high parts, low parts, per 256-block the 16 group-sum halfs
// [even groups: 4 high, 4 low][odd groups: 4 high, 4 low]
// halfs per row of the fp16 form: high parts, low parts, 16 group-sum parts per (started) 256 columns
__host__ __device__ constexpr size_t pf_half_row(int cols) { return 2 * (size_t)cols + 16 * (((size_t)cols + 255) / 256); }

// ---- Q4_K tensors in tile order (once, at upload) ---------------------------------------------
// The grouped product's loader moves one 32-row tile's share of a 256-block per instruction group.
// In GGUF row order that is 32 pieces a row pitch apart; here the same bytes are regrouped so that
// it is 4608 consecutive bytes: [32 headers of 16 bytes][run 0..3: 16-byte halves 0 of the 32 rows,
// then halves 1].  One thread per 16-byte piece; rows is a multiple of 32.
__global__ void pf_k_q4k_tile(const uint8_t *src, uint8_t *dst, size_t rows, int blocks_per_row) {
    const PfMove m = pf_q4k_tile_move((size_t)blockIdx.x * blockDim.x + threadIdx.x, rows, blocks_per_row);
    if (!m.active) return;
    *reinterpret_cast<uint4 *>(dst + m.dst) = *reinterpret_cast<const uint4 *>(src + m.src);
}

void pf_launch_q4k_tile(const uint8_t *d_src, uint8_t *d_dst, size_t rows, int blocks_per_row, hipStream_t stream) {
    const size_t pieces = pf_q4k_tile_threads(rows, blocks_per_row);
    hipLaunchKernelGGL(pf_k_q4k_tile, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream, d_src, d_dst, rows, blocks_per_row);
}

// ---- rows to scaled fp16 pairs ------------------------------------------------------------------
// One workgroup per row (cols a multiple of 32).  scale = 2^e with max|row| / scale in
// [0.5, 1) (1 for a zero row).  Thread j converts the eight values 8j..8j+7; four neighbouring
// threads form one 32-group.
// gate (may be null): a row of `cols` weights; gate_out[row] = sigmoid(row . gate), the shared router's scale (four
// partial sums a lane, lanes and waves added in a fixed order).
__global__ void __launch_bounds__(256) pf_k_rows_to_half(const float *src, size_t src_pitch, int cols, half_t *dst,
                                                         float *scale_out, float *max2_out, uint32_t *error_word,
                                                         const float *gate, float *gate_out) {
    __shared__ float part[4];
    __shared__ float dots[4];
    float dot = 0.0f;
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
        if (gate) {
            const float4 ga = reinterpret_cast<const float4 *>(gate)[2 * j], gb = reinterpret_cast<const float4 *>(gate)[2 * j + 1];
            dot += ((a.x * ga.x + a.y * ga.y) + (a.z * ga.z + a.w * ga.w)) + ((b.x * gb.x + b.y * gb.y) + (b.z * gb.z + b.w * gb.w));
        }
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
            half_t *sums = out + 2 * cols + 16 * (g >> 3) + 8 * (g & 1) + ((g & 7) >> 1);
            sums[0] = sh;
            sums[4] = sl;
        }
    }
    if (gate) {   // uniform
        dot = pf_wave_sum(dot);
        if (pf_lane() == 0) dots[threadIdx.x >> 6] = dot;
        __syncthreads();
        if (threadIdx.x == 0) {
            const float z = (dots[0] + dots[1]) + (dots[2] + dots[3]);
            gate_out[row] = pf_sigmoid(z);
            if (!pf_finite(z)) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
        }
    }
    if (threadIdx.x == 0) {
        scale_out[row] = scale;
        if (max2_out) max2_out[row] = m * m;
    }
}

// The same for rows of at most 512 values (the activation rows): one wave per row, four rows per workgroup, the row
// read once -- a lane keeps its eight values between the maximum and the conversion.  With a workgroup per row three
// of its four waves only took part in the maximum.
__device__ __forceinline__ void rows_to_half_short(size_t block, const float *src, size_t src_pitch, int cols, size_t rows, half_t *dst,
                                                   float *scale_out, float *max2_out, uint32_t *error_word) {
    const size_t row = block * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int j = pf_lane();
    const bool mine = j < cols / 8;
    const float *s = src + row * src_pitch;
    float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f), b = a;
    if (mine) { a = reinterpret_cast<const float4 *>(s)[2 * j]; b = reinterpret_cast<const float4 *>(s)[2 * j + 1]; }
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float m = 0.0f;
    bool bad = false;
#pragma unroll
    for (int c = 0; c < 8; c++) { bad |= !pf_finite(v[c]); m = fmaxf(m, fabsf(v[c])); }
    m = pf_wave_max(m);
    if (__any(bad) && j == 0) atomicOr(error_word, PF_HIP_ERR_NONFINITE);
    int e = (__float_as_int(m) >> 23) & 255;                  // m in [2^(e-127), 2^(e-126))
    e = (e == 0 || e == 255) ? 126 : min(e, 252);             // zero, subnormal or nonfinite row: scale 1
    const float scale = __int_as_float((e + 1) << 23);        // 2^(e-126)
    const float inv = __int_as_float((253 - e) << 23);        // 2^(126-e)
    half_t *out = dst + row * pf_half_row(cols);
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
    if (mine) {
        *reinterpret_cast<half8v *>(out + 8 * j) = hi;
        *reinterpret_cast<half8v *>(out + cols + 8 * j) = lo;
    }
    sum += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sum), 0xB1, 0xF, 0xF, true));   // quad xor 1
    sum += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sum), 0x4E, 0xF, 0xF, true));   // quad xor 2
    if (mine && (j & 3) == 0) {
        const int g = j >> 2;
        const half_t sh = (half_t)sum, sl = (half_t)(sum - (float)sh);
        half_t *sums = out + 2 * cols + 16 * (g >> 3) + 8 * (g & 1) + ((g & 7) >> 1);
        sums[0] = sh;
        sums[4] = sl;
    }
    if (j == 0) {
        scale_out[row] = scale;
        if (max2_out) max2_out[row] = m * m;
    }
}

__global__ void __launch_bounds__(256) pf_k_rows_to_half_short(const float *src, size_t src_pitch, int cols, size_t rows, half_t *dst,
                                                               float *scale_out, float *max2_out, uint32_t *error_word) {
    rows_to_half_short(blockIdx.x, src, src_pitch, cols, rows, dst, scale_out, max2_out, error_word);
}

// Two matrices of short rows in one launch (the routed and the shared activation rows): workgroups [0, blocks_a) take
// the first, the others the second.
__global__ void __launch_bounds__(256) pf_k_rows_to_half_short2(const float *src_a, int cols_a, size_t rows_a, half_t *dst_a, float *scale_a,
                                                                unsigned blocks_a, const float *src_b, int cols_b, size_t rows_b,
                                                                half_t *dst_b, float *scale_b, uint32_t *error_word) {
    if (blockIdx.x < blocks_a) rows_to_half_short(blockIdx.x, src_a, (size_t)cols_a, cols_a, rows_a, dst_a, scale_a, nullptr, error_word);
    else rows_to_half_short(blockIdx.x - blocks_a, src_b, (size_t)cols_b, cols_b, rows_b, dst_b, scale_b, nullptr, error_word);
}

static void launch_rows_to_half(const float *src, size_t src_pitch, int cols, size_t rows, half_t *dst, float *scale_out,
                                float *max2_out, uint32_t *error_word, hipStream_t stream) {
    if (rows == 0) return;
    if (cols <= 512)
        hipLaunchKernelGGL(pf_k_rows_to_half_short, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, src, src_pitch, cols, rows,
                           dst, scale_out, max2_out, error_word);
    else
        hipLaunchKernelGGL(pf_k_rows_to_half, dim3((unsigned)rows), dim3(256), 0, stream, src, src_pitch, cols, dst, scale_out,
                           max2_out, error_word, (const float *)nullptr, (float *)nullptr);
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
// partial tiles are added in wave order).  Also writes the routing tolerance's bound on the sum of
// squared products, max(x)^2 * |w_e|^2.  (The shared router's logit comes from pf_k_rows_to_half.)
//
// Operands.  A product step wants, from lane (i, kk), element k = kk of row i: fetched like that
// from global memory, every load instruction touches 32 rows, and the address unit, which takes a
// cache line at a time, sets the pace (the kernel took 3.3 times the matrix cores' time at the
// benchmark shape).
// Instead a wave fetches a 32-column piece of its 32 + 32 rows as eight instructions of eight whole
// 128-byte lines each (lane = 8 * row + 16-byte piece), stores it into LDS of its own at a row
// pitch of 144 bytes, and reads its operands from there, 16 bytes a lane: columns
// 4 (2 c + kk) .. + 3 for steps 4 c .. 4 c + 3, the same pairing for both operands.  The next
// piece's global loads are on their way while the current one is multiplied; the LDS is the
// wave's alone, so no barrier is needed before the partial tiles meet.
typedef float float4v __attribute__((ext_vector_type(4)));
#define PF_ROUTER_PITCH 36   // floats between rows of a staged piece: eight neighbouring lanes' 16-byte reads cover all banks
__global__ void __launch_bounds__(256) pf_k_pf_router(PfKernelArgs a, int tokens) {
    __shared__ float partial[3][16][64];
    __shared__ __align__(16) float staged[4][2][32 * PF_ROUTER_PITCH];   // [wave][x | w][row][column]
    const int H = a.hidden, E = a.experts, lane = pf_lane(), wave = threadIdx.x >> 6;
    const int t0 = blockIdx.x * 32, e0 = blockIdx.y * 32;
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) a.route_flags[0] = 0;   // the routing's list starts empty
    const int i = lane & 31, kk = lane >> 5;
    // the four waves split the rows' 128-byte lines (hidden is a multiple of 32)
    const int lines = H / 32, l0 = lines * wave / 4, l1 = lines * (wave + 1) / 4;
    const int lr = lane >> 3, piece = lane & 7;   // fetch: row within a group of eight, 16-byte piece of the line
    const float4v *xsrc[4], *wsrc[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const int t = min(t0 + 8 * g + lr, tokens - 1), e = min(e0 + 8 * g + lr, E - 1);
        xsrc[g] = reinterpret_cast<const float4v *>(a.x + (size_t)t * a.x_pitch) + piece;
        wsrc[g] = reinterpret_cast<const float4v *>(a.w[0] + (size_t)e * H * 4) + piece;
    }
    float *xs = staged[wave][0], *ws = staged[wave][1];
    float16v acc = {0};
    if (l0 < l1) {
        float4v xg[4], wg[4];
#pragma unroll
        for (int g = 0; g < 4; g++) { xg[g] = xsrc[g][8 * l0]; wg[g] = wsrc[g][8 * l0]; }
        for (int l = l0; l < l1; l++) {
            // the piece fetched last into LDS (after the reads of the piece before it, in the wave's program order),
            // then the next one's loads on their way (the last step fetches its own piece again; two pieces ahead
            // measured no faster)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                *reinterpret_cast<float4v *>(xs + (8 * g + lr) * PF_ROUTER_PITCH + 4 * piece) = xg[g];
                *reinterpret_cast<float4v *>(ws + (8 * g + lr) * PF_ROUTER_PITCH + 4 * piece) = wg[g];
            }
            const int next = l + 1 < l1 ? l + 1 : l;
#pragma unroll
            for (int g = 0; g < 4; g++) { xg[g] = xsrc[g][8 * next]; wg[g] = wsrc[g][8 * next]; }
            float4v xv[4], wv[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                xv[c] = *reinterpret_cast<const float4v *>(xs + i * PF_ROUTER_PITCH + 4 * (2 * c + kk));
                wv[c] = *reinterpret_cast<const float4v *>(ws + i * PF_ROUTER_PITCH + 4 * (2 * c + kk));
            }
#pragma unroll
            for (int c = 0; c < 4; c++) {
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[c].x, wv[c].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[c].y, wv[c].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[c].z, wv[c].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[c].w, wv[c].w, acc, 0, 0, 0);
            }
        }
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
        if (row >= tokens || col >= E) continue;
        a.logits[(size_t)row * E + col] = acc[r];
        a.logit_ssq[(size_t)row * E + col] = a.x_max2[row] * wn;
    }
}

// ---- grouped product ------------------------------------------------------------------------------
enum { PF_GEMM_GATE_UP = 0, PF_GEMM_DOWN = 1 };

// Workgroup = one 32-row tile of an expert against 64 NW weight rows: NW compute waves, each
// with two 32-row weight tiles (gate + up of 32 units, or 2 x 32 down rows), and 1 + NW / 4 loader
// waves.
//
// Only the loader waves issue global loads.  They move the operands of one stage (64 of the K
// columns) straight into LDS, 16 bytes per lane, up to four stages ahead of the products, through
// a ring of five slots: with one workgroup per compute unit that keeps about 100 KB on their way;
// a wave counts at most 63 loads, so the stream is split over three loaders (activations; the
// weight runs of compute waves 0-3; of 4-7).  A stalled memory pipeline holds up the loaders, never the waves that feed the matrix
// cores.  One workgroup barrier per stage hands the landed slot to the compute waves and the slot
// they have just left back to the loaders.
//
//   slot   [0, A_PART)            high parts of the 32 activation rows, 128 bytes each: four images
//                                 of eight rows, chunk-major (16-byte chunk c of row r at 128 c + 16 r)
//          [A_PART, 2 A_PART)     low parts likewise
//          [SLOT_W, +2 NW KB)     the stage's 32-byte nibble run of every weight row: per tile the
//                                 first halves of the 32 rows, then the second halves
//   once per 256-block: the 16-byte block headers of the 2 NW tiles, the activation rows' group sums
//
// IQ2_XXS differs in the weight bytes only: a row's stage is 16 bytes (two 32-groups of four grid
// indices and one word of signs and scale), so a wave's two tiles are one 1 KB image
// [tile][row][16 bytes]; per 256-block a row brings its fp16 scale (the dword around it); the
// 256 x 8 magnitude grid and the 128 sign masks sit in LDS behind the ring.
//
// Matrix-core operands.  Lane (n = lane % 32, h = lane / 32) holds column n (a weight row) and
// supplies K slots 8h..8h+7.  In stage j, step t, these are the codes 8t..8t+7 of group 2j + h
// (h = 0: the low nibbles of the run, h = 1: the high nibbles), so a lane needs the scale and the
// minimum of one group per stage, and activation columns 64 j + 32 h + 8 t + 0..7.
#define NW 8                               // compute waves per workgroup
#define NL (1 + NW / 4)                    // loader waves
#define RING_SLOTS 5
#define A_GROUP 1152                       // bytes between eight-row images: 1 KB + 128, neighbours start on opposite bank halves
#define A_PART (4 * A_GROUP)
#define SLOT_W (2 * A_PART)
#define SLOT_BYTES (SLOT_W + 2 * NW * 1024)
#define HDR_OFF (RING_SLOTS * SLOT_BYTES)
#define BLOCK_BYTES (2 * NW * 512 + 1024)   // per 256-block: headers, then sums; two copies (blocks alternate)
#define SUMS_OFF (HDR_OFF + 2 * NW * 512)
#define GEMM_LDS (HDR_OFF + 2 * BLOCK_BYTES)   // 146 432 bytes with 8 compute waves: one workgroup per compute unit
#define IQ2_GRID_OFF GEMM_LDS                  // IQ2_XXS: 256 grid entries of 8 magnitudes, then 128 masks of 8 fp16 sign bits
#define IQ2_SIGN_OFF (IQ2_GRID_OFF + 2048)
#define GEMM_LDS_IQ2 (IQ2_SIGN_OFF + 2048)
static_assert(RING_SLOTS == 5 && NW % 4 == 0, "the loaders' wait counts below assume three younger stages on their way");

__device__ __forceinline__ void to_lds(const void *global, unsigned char *lds) {
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(global), reinterpret_cast<uint32_t *>(lds), 16, 0, 0);
}

__device__ __forceinline__ void to_lds_dword(const void *global, unsigned char *lds) {   // 4 bytes per lane, lane l at lds + 4 l
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(global), reinterpret_cast<uint32_t *>(lds), 4, 0, 0);
}

__device__ __forceinline__ void stage_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

struct GemmTarget {   // one work item of the grouped product: a 32-row tile of an expert against one slab of weight rows
    bool shared;
    int first, count, inter, kblocks, a_cols, slab;
    int m0, rows_here;    // first row of the tile within the expert's rows, rows in it
    int waves;            // compute waves whose weight rows exist (the last slab of a narrow matrix has fewer)
    uint32_t zero_row;    // index of the all-zero row that ends the fp16 form of the activation matrix
    uint32_t row_bytes;   // of the weight tensor(s)
    uint32_t wave_rows;   // weight rows between the tiles of consecutive compute waves
    bool tiled;           // weights in the tile order of pf_k_q4k_tile (else GGUF row order)
    const uint8_t *w0, *w1;   // first weight row of compute wave 0's two tiles
    const uint16_t *s0, *s1;  // IQ2_XXS: the tensors' fp16 block scales, and the index of the tiles' first row's first scale
    uint32_t sidx0, sidx1, bpr;
    const half_t *a16;
    const float *a_scale;
};

// Work item q -> (row tile, slab).  Workgroups go to the eight XCDs round robin by index and a
// workgroup's items are a multiple of eight apart.  The tile list is cut into groups of GEMM_XCD_TILES
// consecutive tiles and the groups dealt to the XCDs in turn; the items of a group (its tiles' slabs)
// get numbers eight apart: neighbouring workgroups of one XCD, one L2, at the same time.  The slabs of
// a row tile read the same activation rows, and the row tiles of one expert, neighbours in the list,
// the same weights: fetched once from memory where they fall into one group.  False: nothing to do
// for q.  Every wave of the workgroup evaluates this for itself, with the same result.
#define GEMM_XCD_TILES 8
template <int MODE, int FMT>
__device__ __forceinline__ bool gemm_item(const PfKernelArgs &a, int tokens, int slabs, uint32_t q, GemmTarget &g) {
    const int E = a.experts, K = a.top_k;
    const uint32_t xcd = q % 8, turn = q / 8, r = turn / slabs;
    const uint32_t tile = GEMM_XCD_TILES * ((r / GEMM_XCD_TILES) * 8 + xcd) + r % GEMM_XCD_TILES;
    if (tile >= a.tiles[0]) return false;
    const uint32_t entry = a.tiles[1 + tile];
    const int expert = entry & 0xffffu;
    g.m0 = 32 * (int)(entry >> 16);
    g.slab = turn % slabs;
    g.shared = expert == E;
    const int P = tokens * K;
    g.first = g.shared ? P : (int)a.offsets[expert];
    g.count = g.shared ? tokens : (int)a.offsets[expert + 1] - g.first;
    if (g.count <= g.m0) return false;
    g.rows_here = min(32, g.count - g.m0);
    g.inter = g.shared ? a.shared_inter : a.inter;
    const size_t ex = g.shared ? 0 : (size_t)expert;
    if (a.type[MODE == PF_GEMM_GATE_UP ? (g.shared ? 4 : 1) : (g.shared ? 6 : 3)] != (uint32_t)FMT)
        return false;   // another format: the plain grouped product takes the item
    if (MODE == PF_GEMM_GATE_UP) {
        const int tg = g.shared ? 4 : 1;
        if (32 * NW * g.slab >= g.inter) return false;
        g.row_bytes = (uint32_t)a.row_bytes[tg];
        g.tiled = a.wt[tg] != nullptr;
        g.w0 = (g.tiled ? a.wt[tg] : a.w[tg]) + ex * a.expert_bytes[tg] + (size_t)(32 * NW * g.slab) * g.row_bytes;
        g.w1 = (g.tiled ? a.wt[tg + 1] : a.w[tg + 1]) + ex * a.expert_bytes[tg + 1] + (size_t)(32 * NW * g.slab) * g.row_bytes;
        if (FMT == PF_IQ2_XXS) {
            g.bpr = (uint32_t)a.blocks_per_row[tg];
            g.s0 = reinterpret_cast<const uint16_t *>(a.w[tg] + a.scale_offset[tg]);
            g.s1 = reinterpret_cast<const uint16_t *>(a.w[tg + 1] + a.scale_offset[tg + 1]);
            g.sidx0 = g.sidx1 = (uint32_t)((ex * a.n_out[tg] + 32 * NW * g.slab) * g.bpr);
        }
        g.wave_rows = 32;
        g.waves = min(NW, (g.inter - 32 * NW * g.slab) / 32);
        g.kblocks = a.hidden / 256; g.a_cols = a.hidden;
        g.a16 = reinterpret_cast<const half_t *>(a.x16); g.a_scale = a.x_scale;
        g.zero_row = a.token_cap;
    } else {
        const int td = g.shared ? 6 : 3;
        if (64 * NW * g.slab >= a.hidden) return false;
        g.row_bytes = (uint32_t)a.row_bytes[td];
        g.tiled = a.wt[td] != nullptr;
        g.w0 = (g.tiled ? a.wt[td] : a.w[td]) + ex * a.expert_bytes[td] + (size_t)(64 * NW * g.slab) * g.row_bytes;
        g.w1 = g.w0 + (size_t)32 * g.row_bytes;
        if (FMT == PF_IQ2_XXS) {
            g.bpr = (uint32_t)a.blocks_per_row[td];
            g.s0 = g.s1 = reinterpret_cast<const uint16_t *>(a.w[td] + a.scale_offset[td]);
            g.sidx0 = (uint32_t)((ex * a.n_out[td] + 64 * NW * g.slab) * g.bpr);
            g.sidx1 = g.sidx0 + 32 * g.bpr;
        }
        g.wave_rows = 64;
        g.waves = min(NW, (a.hidden - 64 * NW * g.slab) / 64);
        g.kblocks = g.inter / 256; g.a_cols = g.inter;
        g.a16 = reinterpret_cast<const half_t *>(g.shared ? a.sact16 : a.act16);
        g.a_scale = g.shared ? a.sact_scale : a.act_scale;
        g.zero_row = g.shared ? a.token_cap : a.token_cap * (uint32_t)K;
    }
    return true;
}

// first item at or after q (stepping by the grid size) that has work; false when the list is exhausted
template <int MODE, int FMT>
__device__ __forceinline__ bool gemm_next_item(const PfKernelArgs &a, int tokens, int slabs, uint32_t items, uint32_t &q,
                                               GemmTarget &g) {
    for (; q < items; q += gridDim.x)
        if (gemm_item<MODE, FMT>(a, tokens, slabs, q, g)) return true;
    return false;
}

// Loads of the stages that may still be on their way when stage s is handed over: the younger
// stages issued so far, at most three.  Three consecutive stages hold one that opens a 256-block
// (and carries `block_loads` more) unless stage s opens one itself; fewer than three only happens
// at the end, inside the last block.
#define WAIT_YOUNGER(younger, opens, per_stage, block_loads)                             \
    do {                                                                                 \
        if ((younger) >= 3 && (opens)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (per_stage) + (block_loads)) : "memory"); \
        else if ((younger) >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (per_stage)) : "memory");        \
        else if ((younger) == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (per_stage)) : "memory");        \
        else if ((younger) == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(1 * (per_stage)) : "memory");        \
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                            \
    } while (0)

// A loader wave.  ROLE 0 moves the activation images and the group sums (and leaves the rows'
// scales for the epilogue); ROLE q >= 1 the weight runs and block headers of compute waves
// 4 (q - 1) .. 4 (q - 1) + 3.  It walks the workgroup's items as one stream of stages, up to
// RING_SLOTS - 1 stages ahead of the compute waves, also across item boundaries: the ring never
// drains between items.  Every workgroup barrier here pairs with one of gemm_compute.
template <int MODE, int FMT, int ROLE>
__device__ __forceinline__ void gemm_loader(const PfKernelArgs &a, int tokens, int slabs, uint32_t items, unsigned char *ring,
                                            float (*row_scale)[32]) {
    const int lane = pf_lane(), K = a.top_k;
    GemmTarget g;
    uint32_t q = blockIdx.x;
    bool more = gemm_next_item<MODE, FMT>(a, tokens, slabs, items, q, g);
    int kb = 0, j = 0, slot_index = 0, block_parity = 0, item_index = 0;
    uint32_t a_off[4] = {0, 0, 0, 0}, a_live[4] = {0, 0, 0, 0}, s_off = 0, s_live = 0, w_off = 0, h_off = 0, block_step = 0,
             run0 = 0, run_step = 0;
    size_t wave_bytes = 0;
    auto open_item = [&]() {   // per-lane source offsets of the item the issue cursor has reached
        if (ROLE == 0) {
            // activation images: instruction i carries rows 8i..8i+7, lane = 8 * chunk + row.  The
            // lanes of rows beyond the tile's last all read the first 16 bytes of the matrix's
            // all-zero row, whatever the stage: one cache line serves them (a_live masks the
            // stage's column offset away), so padding costs no memory traffic.
            const uint32_t a_pitch = (uint32_t)pf_half_row(g.a_cols);
            auto source_row = [&](int m) -> uint32_t {
                if (m >= g.rows_here) return g.zero_row;
                if (g.shared) return (uint32_t)(g.m0 + m);
                return MODE == PF_GEMM_GATE_UP ? a.row_to_pair[g.first + g.m0 + m] / (uint32_t)K : (uint32_t)(g.first + g.m0 + m);
            };
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int m = 8 * i + (lane & 7);
                a_live[i] = m < g.rows_here ? 0xffffffffu : 0u;
                a_off[i] = source_row(m) * a_pitch + (8u * (uint32_t)(lane >> 3) & a_live[i]);
            }
            const uint32_t mine = source_row(lane & 31);
            s_live = (lane & 31) < g.rows_here ? 0xffffffffu : 0u;
            s_off = mine * a_pitch + ((2u * (uint32_t)g.a_cols + 8u * (uint32_t)(lane >> 5)) & s_live);
            // the rows' scales for the epilogue of this item (read many barriers later; four copies
            // in turn, because this wave may open the item after next before the epilogue of the
            // current one is over)
            if (lane < 32) row_scale[item_index & 3][lane] = (lane < g.rows_here) ? g.a_scale[mine] : 0.0f;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        } else if (FMT == PF_IQ2_XXS) {
            // lane = 32 * (tile of the wave's pair) + row: the row's two groups of the stage, and per
            // block the dword that holds the row's fp16 scale
            w_off = (uint32_t)(lane & 31) * g.row_bytes;
            h_off = (uint32_t)(lane & 31) * g.bpr;
            wave_bytes = (size_t)g.wave_rows * g.row_bytes;
        } else {
            // weight runs: lane = 32 * half + row; headers: lane = 32 * (tile of the wave's pair) + row.
            // Tile order: a 32-row tile's 256-block is 4608 consecutive bytes, the 32 headers, then per
            // run the 1 KB image exactly as it lands in LDS; row order: 144-byte blocks at the row pitch.
            w_off = g.tiled ? 16u * (uint32_t)lane : (uint32_t)(lane & 31) * g.row_bytes + 16u * (uint32_t)(lane >> 5);
            h_off = g.tiled ? 16u * (uint32_t)(lane & 31) : (uint32_t)(lane & 31) * g.row_bytes;
            block_step = g.tiled ? 4608u : 144u; run0 = g.tiled ? 512u : 16u; run_step = g.tiled ? 1024u : 32u;
            wave_bytes = (size_t)g.wave_rows * g.row_bytes;
        }
        item_index++;
    };
    auto issue = [&]() {   // the stage under the issue cursor, then advance the cursor
        unsigned char *slot = ring + slot_index * SLOT_BYTES;
        unsigned char *block = ring + block_parity * BLOCK_BYTES;
        if (ROLE == 0) {
            const uint32_t high = 256u * (uint32_t)kb + 64u * (uint32_t)j, low = high + (uint32_t)g.a_cols;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                to_lds(g.a16 + a_off[i] + (high & a_live[i]), slot + i * A_GROUP);
                to_lds(g.a16 + a_off[i] + (low & a_live[i]), slot + A_PART + i * A_GROUP);
            }
            if (j == 0) to_lds(g.a16 + s_off + (16u * (uint32_t)kb & s_live), block + SUMS_OFF);
        } else if (FMT == PF_IQ2_XXS) {
            const uint8_t *tile = (lane >> 5) ? g.w1 : g.w0;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int v = 4 * (ROLE - 1) + c, vv = min(v, g.waves - 1);   // a wave without rows repeats the last one's
                to_lds(tile + (size_t)vv * wave_bytes + w_off + 64u * (uint32_t)kb + 16u * (uint32_t)j, slot + SLOT_W + v * 1024);
            }
            if (j == 0) {
                const uint16_t *scales = (lane >> 5) ? g.s1 : g.s0;
                const uint32_t first = (lane >> 5) ? g.sidx1 : g.sidx0;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int v = 4 * (ROLE - 1) + c, vv = min(v, g.waves - 1);
                    const uint32_t at = first + (uint32_t)vv * g.wave_rows * g.bpr + h_off + (uint32_t)kb;
                    to_lds_dword(scales + (at & ~1u), block + HDR_OFF + v * 256);
                }
            }
        } else {
            const uint32_t run = block_step * (uint32_t)kb + run0 + run_step * (uint32_t)j;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int v = 4 * (ROLE - 1) + c;
                const size_t at = (size_t)min(v, g.waves - 1) * wave_bytes;   // a wave without rows repeats the last one's
                to_lds(g.w0 + at + run + w_off, slot + SLOT_W + (2 * v) * 1024);
                to_lds(g.w1 + at + run + w_off, slot + SLOT_W + (2 * v + 1) * 1024);
            }
            if (j == 0) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int v = 4 * (ROLE - 1) + c;
                    const size_t at = (size_t)min(v, g.waves - 1) * wave_bytes;
                    to_lds(((lane >> 5) ? g.w1 : g.w0) + at + block_step * (uint32_t)kb + h_off, block + HDR_OFF + v * 1024);
                }
            }
        }
        slot_index = slot_index + 1 == RING_SLOTS ? 0 : slot_index + 1;
        if (++j == 4) {
            j = 0;
            block_parity ^= 1;
            if (++kb == g.kblocks) {
                kb = 0;
                q += gridDim.x;
                more = gemm_next_item<MODE, FMT>(a, tokens, slabs, items, q, g);
                if (more) open_item();
            }
        }
    };
    if (more) open_item();
    // Before the barrier of stage s its loads have landed (loads complete in order).  After it,
    // the slot of stage s - 1 is free for stage s + RING_SLOTS - 1.  A stage that opens a block also
    // brings its headers and sums, into the copy that the block before the previous one used.
    int issued = 0;
    while (issued < RING_SLOTS - 1 && more) { issue(); issued++; }
    for (int s = 0; s < issued; s++) {
        const int younger = issued - s - 1;   // at most RING_SLOTS - 2
        const bool opens = (s & 3) != 0;      // one of stages s + 1 .. s + 3 opens a block
        if (ROLE == 0) WAIT_YOUNGER(younger, opens, 8, 1);
        else if (FMT == PF_IQ2_XXS) WAIT_YOUNGER(younger, opens, 4, 4);
        else WAIT_YOUNGER(younger, opens, 8, 4);
        stage_barrier();
        if (more) { issue(); issued++; }
    }
}

// 6-bit scale and minimum of group 2 jj + h (h per lane) from the 12 packed bytes of a block
// header (src/qwen4_packed.c:88-91)
__device__ __forceinline__ void q4_scale_min(const uint4 &hdr, int jj, int h, uint32_t &sc, uint32_t &mn) {
    const int sh = 16 * (jj & 1) + 8 * h;
    if (jj < 2) {
        sc = (hdr.y >> sh) & 63u;
        mn = (hdr.z >> sh) & 63u;
    } else {
        const uint32_t hi = (hdr.w >> sh) & 255u, lo_s = (hdr.y >> sh) & 255u, lo_m = (hdr.z >> sh) & 255u;
        sc = (hi & 15u) | ((lo_s & 192u) >> 2);
        mn = (hi >> 4) | ((lo_m & 192u) >> 2);
    }
}

// eight codes (the nibbles under mask in two dwords) times the group's scale, exact in fp16: a
// nibble under the exponent byte 0x64 reads as 1024 + q (low nibble) or 1024 + 16 q (high nibble,
// left in place), and (1024 + q) * s - 1024 * s = q * s, (1024 + 16 q) * (s / 16) - 64 s = q * s;
// s2 and c are the pair of constants that belongs to the lane's nibble position
__device__ __forceinline__ half8v q4_scaled_codes(uint32_t w0, uint32_t w1, uint32_t mask, half2v s2, half2v c) {
    const uint32_t q0 = w0 & mask, q1 = w1 & mask;
    const uint32_t bias = 0x64646464u;
    const half2v p0 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q0, 0x04010400u));
    const half2v p1 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q0, 0x04030402u));
    const half2v p2 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q1, 0x04010400u));
    const half2v p3 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, q1, 0x04030402u));
    const half2v v0 = p0 * s2 - c, v1 = p1 * s2 - c, v2 = p2 * s2 - c, v3 = p3 * s2 - c;
    return half8v{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
}

// A compute wave: all K against its two weight tiles.  A 256-block's result is
// d * P - dmin * Q with P = sum (scale * code) x and Q = sum_g min_g * (sum of x over group g).
// slot_off and block_parity carry the ring position from one item to the next.
__device__ __forceinline__ void gemm_compute(const unsigned char *ring, int kblocks, float16v &acc0, float16v &acc1, int &slot_off,
                                             int &block_parity) {
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5;
    const uint32_t mask = h ? 0xF0F0F0F0u : 0x0F0F0F0Fu;
    const half_t unit = h ? (half_t)0.0625f : (half_t)1.0f;
    const int bias_shift = h ? 6 : 10;
    const unsigned char *a_lane = ring + (n >> 3) * A_GROUP + (4 * h) * 128 + (n & 7) * 16;
    const unsigned char *w_lane = ring + SLOT_W + (2 * wave) * 1024 + n * 16;
    const float16v zero = {0};
    for (int kb = 0; kb < kblocks; kb++) {
        float16v part0 = zero, part1 = zero, q0 = zero, q1 = zero;
        float d0 = 0.0f, m0 = 0.0f, d1 = 0.0f, m1 = 0.0f;
        half2v s2[2][4], c2[2][4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            stage_barrier();
            const unsigned char *slot_a = a_lane + slot_off, *slot_w = w_lane + slot_off;
            slot_off = slot_off + SLOT_BYTES == RING_SLOTS * SLOT_BYTES ? 0 : slot_off + SLOT_BYTES;
            // every LDS operand of the stage is requested up front (they return in order: the first
            // product waits for the weight runs and one fragment pair, the rest arrive under way)
            const uint4 wa0 = *reinterpret_cast<const uint4 *>(slot_w), wb0 = *reinterpret_cast<const uint4 *>(slot_w + 512);
            const uint4 wa1 = *reinterpret_cast<const uint4 *>(slot_w + 1024), wb1 = *reinterpret_cast<const uint4 *>(slot_w + 1536);
            half8v ah[4], al[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                ah[t] = *reinterpret_cast<const half8v *>(slot_a + 128 * t);
                al[t] = *reinterpret_cast<const half8v *>(slot_a + A_PART + 128 * t);
            }
            if (j == 0) {
                const unsigned char *block = ring + block_parity * BLOCK_BYTES;
                block_parity ^= 1;
                const uint4 hdr0 = *reinterpret_cast<const uint4 *>(block + HDR_OFF + (2 * wave) * 512 + n * 16);
                const uint4 hdr1 = *reinterpret_cast<const uint4 *>(block + HDR_OFF + (2 * wave + 1) * 512 + n * 16);
                const half8v as = *reinterpret_cast<const half8v *>(block + SUMS_OFF + lane * 16);
                asm volatile("" ::: "memory");   // the requests stay above the arithmetic
                // the hardware conversion is exact for every binary16 value, subnormals included
                const half2v dm0 = __builtin_bit_cast(half2v, hdr0.x), dm1 = __builtin_bit_cast(half2v, hdr1.x);
                d0 = (float)dm0.x; m0 = (float)dm0.y; d1 = (float)dm1.x; m1 = (float)dm1.y;
                half_t min0[4], min1[4];
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    uint32_t sc, mn;
                    q4_scale_min(hdr0, jj, h, sc, mn);
                    min0[jj] = (half_t)(int)mn;
                    const half_t s0 = (half_t)(int)sc * unit, k0 = (half_t)(int)(sc << bias_shift);
                    s2[0][jj] = half2v{s0, s0};
                    c2[0][jj] = half2v{k0, k0};
                    q4_scale_min(hdr1, jj, h, sc, mn);
                    min1[jj] = (half_t)(int)mn;
                    const half_t s1 = (half_t)(int)sc * unit, k1 = (half_t)(int)(sc << bias_shift);
                    s2[1][jj] = half2v{s1, s1};
                    c2[1][jj] = half2v{k1, k1};
                }
                // Q: K slots 8h..8h+3 hold the high parts of the sums of the lane's four groups,
                // 8h+4..8h+7 the low parts; the four minima appear once against each
                const half8v mv0 = {min0[0], min0[1], min0[2], min0[3], min0[0], min0[1], min0[2], min0[3]};
                const half8v mv1 = {min1[0], min1[1], min1[2], min1[3], min1[0], min1[1], min1[2], min1[3]};
                q0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(as, mv0, zero, 0, 0, 0);
                q1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(as, mv1, zero, 0, 0, 0);
            }
            asm volatile("" ::: "memory");
            const uint32_t w0[8] = {wa0.x, wa0.y, wa0.z, wa0.w, wb0.x, wb0.y, wb0.z, wb0.w};
            const uint32_t w1[8] = {wa1.x, wa1.y, wa1.z, wa1.w, wb1.x, wb1.y, wb1.z, wb1.w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const half8v b0 = q4_scaled_codes(w0[2 * t], w0[2 * t + 1], mask, s2[0][j], c2[0][j]);
                const half8v b1 = q4_scaled_codes(w1[2 * t], w1[2 * t + 1], mask, s2[1][j], c2[1][j]);
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[t], b0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[t], b1, part1, 0, 0, 0);
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[t], b0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[t], b1, part1, 0, 0, 0);
            }
            if (j == 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    acc0[r] = fmaf(-m0, q0[r], acc0[r]);
                    acc1[r] = fmaf(-m1, q1[r], acc1[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc0[r] = fmaf(d0, part0[r], acc0[r]);
            acc1[r] = fmaf(d1, part1[r], acc1[r]);
        }
    }
}

// The same for IQ2_XXS tiles (src/qwen4_packed.c:95-121): a weight is d / 8 * (2 s + 1) * magnitude * sign with a
// 4-bit s per 32-group, magnitudes 8, 25 or 43 from the grid and d per 256-block, so
// (2 s + 1) * magnitude <= 1333 is an exact fp16 operand: a magnitude byte under the exponent byte
// 0x64 reads as 1024 + m, (1024 + m) * (2 s + 1) - 1024 * (2 s + 1) = m * (2 s + 1) in one fused step,
// and the sign is a bit flip.  A 256-block's result is (d / 8) * P.  Lane (n, h) takes group 2 j + h in
// stage j: step t is its grid entry t (8 weights) with the 7 sign bits t of the group's second word.
// sidx0 / sidx1 / bpr locate the rows' fp16 block scales (which half of the loaded dword is theirs).
__device__ __forceinline__ void gemm_compute_iq2(const unsigned char *ring, int kblocks, float16v &acc0, float16v &acc1,
                                                 int &slot_off, int &block_parity, uint32_t sidx0, uint32_t sidx1, uint32_t bpr,
                                                 int wave_rows) {
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5;
    const unsigned char *a_lane = ring + (n >> 3) * A_GROUP + (4 * h) * 128 + (n & 7) * 16;
    const unsigned char *w_lane = ring + SLOT_W + wave * 1024 + n * 16 + 8 * h;
    const uint2 *grid = reinterpret_cast<const uint2 *>(ring + IQ2_GRID_OFF);
    const uint4 *signs = reinterpret_cast<const uint4 *>(ring + IQ2_SIGN_OFF);
    // index of this lane's rows' first scale; the loader fetched the dword around scale index + kb
    const uint32_t row0 = sidx0 + ((uint32_t)wave * wave_rows + n) * bpr, row1 = sidx1 + ((uint32_t)wave * wave_rows + n) * bpr;
    const float16v zero = {0};
    for (int kb = 0; kb < kblocks; kb++) {
        float16v part0 = zero, part1 = zero;
        float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            stage_barrier();
            const unsigned char *slot_a = a_lane + slot_off, *slot_w = w_lane + slot_off;
            slot_off = slot_off + SLOT_BYTES == RING_SLOTS * SLOT_BYTES ? 0 : slot_off + SLOT_BYTES;
            const uint2 g0 = *reinterpret_cast<const uint2 *>(slot_w), g1 = *reinterpret_cast<const uint2 *>(slot_w + 512);
            half8v ah[4], al[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                ah[t] = *reinterpret_cast<const half8v *>(slot_a + 128 * t);
                al[t] = *reinterpret_cast<const half8v *>(slot_a + A_PART + 128 * t);
            }
            if (j == 0) {
                const unsigned char *block = ring + block_parity * BLOCK_BYTES;
                block_parity ^= 1;
                const uint32_t pair0 = *reinterpret_cast<const uint32_t *>(block + HDR_OFF + wave * 256 + 4 * n);
                const uint32_t pair1 = *reinterpret_cast<const uint32_t *>(block + HDR_OFF + wave * 256 + 128 + 4 * n);
                const uint32_t bits0 = ((row0 + (uint32_t)kb) & 1u) ? pair0 >> 16 : pair0 & 0xffffu;
                const uint32_t bits1 = ((row1 + (uint32_t)kb) & 1u) ? pair1 >> 16 : pair1 & 0xffffu;
                d0 = (float)__builtin_bit_cast(half_t, (unsigned short)bits0) * 0.125f;
                d1 = (float)__builtin_bit_cast(half_t, (unsigned short)bits1) * 0.125f;
            }
            asm volatile("" ::: "memory");   // the requests stay above the arithmetic
            const half_t s0 = (half_t)(int)(2u * (g0.y >> 28) + 1u), s1 = (half_t)(int)(2u * (g1.y >> 28) + 1u);
            const half_t k0 = (half_t)(int)(1024u * (2u * (g0.y >> 28) + 1u)), k1 = (half_t)(int)(1024u * (2u * (g1.y >> 28) + 1u));
            const half2v s20 = {s0, s0}, s21 = {s1, s1}, c20 = {k0, k0}, c21 = {k1, k1};
            auto codes = [&](const uint2 &g, int t, half2v s2, half2v c) -> half8v {
                const uint2 m = grid[(g.x >> (8 * t)) & 255u];
                const uint4 flip = signs[(g.y >> (7 * t)) & 127u];
                const uint32_t bias = 0x64646464u;
                const half2v p0 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, m.x, 0x04010400u));
                const half2v p1 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, m.x, 0x04030402u));
                const half2v p2 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, m.y, 0x04010400u));
                const half2v p3 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, m.y, 0x04030402u));
                const half2v v0 = p0 * s2 - c, v1 = p1 * s2 - c, v2 = p2 * s2 - c, v3 = p3 * s2 - c;
                const uint4 bits = {__builtin_bit_cast(uint32_t, v0) ^ flip.x, __builtin_bit_cast(uint32_t, v1) ^ flip.y,
                                    __builtin_bit_cast(uint32_t, v2) ^ flip.z, __builtin_bit_cast(uint32_t, v3) ^ flip.w};
                return __builtin_bit_cast(half8v, bits);
            };
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const half8v b0 = codes(g0, t, s20, c20), b1 = codes(g1, t, s21, c21);
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[t], b0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[t], b1, part1, 0, 0, 0);
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[t], b0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[t], b1, part1, 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc0[r] = fmaf(d0, part0[r], acc0[r]);
            acc1[r] = fmaf(d1, part1[r], acc1[r]);
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
    // inclusive scan of the 256 partial sums in eight doubling steps, then made exclusive
    uint32_t run_rows = rows, run_tiles = ntiles;
    for (int d = 1; d < 256; d <<= 1) {
        const uint32_t add_rows = tid >= d ? rows_before[tid - d] : 0u, add_tiles = tid >= d ? tiles_before[tid - d] : 0u;
        __syncthreads();
        run_rows += add_rows;
        run_tiles += add_tiles;
        rows_before[tid] = run_rows;
        tiles_before[tid] = run_tiles;
        __syncthreads();
    }
    if (tid == 255) {
        offsets[E] = run_rows;
        tiles[0] = run_tiles;
    }
    __syncthreads();
    rows_before[tid] = run_rows - rows;
    tiles_before[tid] = run_tiles - ntiles;
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

// One workgroup per compute unit; workgroup b takes items b, b + grid, b + 2 grid, ...
template <int MODE, int FMT>
__global__ void __launch_bounds__(64 * (NW + NL), 3) pf_k_pf_gemm(PfKernelArgs a, int tokens, int slabs) {
    extern __shared__ __align__(16) unsigned char ring[];
    __shared__ float row_scale[4][32];
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5;
    const uint32_t items = (a.tiles[0] + 8u * GEMM_XCD_TILES - 1u) / (8u * GEMM_XCD_TILES) * (8u * GEMM_XCD_TILES) * (uint32_t)slabs;
    if (FMT == PF_IQ2_XXS) {
        // grid magnitudes, and for every 7-bit sign field the fp16 sign bits of its eight weights
        // (the eighth sign makes the number of negative weights even)
        if (threadIdx.x < 256) reinterpret_cast<uint64_t *>(ring + IQ2_GRID_OFF)[threadIdx.x] = a.iq2_grid[threadIdx.x];
        if (threadIdx.x >= 256 && threadIdx.x < 384) {
            const uint32_t s7 = threadIdx.x - 256, s8 = s7 | ((__popc(s7) & 1u) << 7);
            uint4 flip;
            flip.x = ((s8 >> 0) & 1u) << 15 | ((s8 >> 1) & 1u) << 31;
            flip.y = ((s8 >> 2) & 1u) << 15 | ((s8 >> 3) & 1u) << 31;
            flip.z = ((s8 >> 4) & 1u) << 15 | ((s8 >> 5) & 1u) << 31;
            flip.w = ((s8 >> 6) & 1u) << 15 | ((s8 >> 7) & 1u) << 31;
            reinterpret_cast<uint4 *>(ring + IQ2_SIGN_OFF)[s7] = flip;
        }
        __syncthreads();
    }
    if (wave >= NW) {
        __builtin_amdgcn_s_setprio(3);   // the loaders issue little and everything waits for it
        if (wave == NW) gemm_loader<MODE, FMT, 0>(a, tokens, slabs, items, ring, row_scale);
        else if (wave == NW + 1) gemm_loader<MODE, FMT, 1>(a, tokens, slabs, items, ring, row_scale);
        else gemm_loader<MODE, FMT, 2>(a, tokens, slabs, items, ring, row_scale);
        return;
    }
    GemmTarget g;
    int slot_off = 0, block_parity = 0, item_index = 0;
    uint32_t q = blockIdx.x;
    while (gemm_next_item<MODE, FMT>(a, tokens, slabs, items, q, g)) {
        float16v acc0 = {0}, acc1 = {0};
        if (FMT == PF_IQ2_XXS)
            gemm_compute_iq2(ring, g.kblocks, acc0, acc1, slot_off, block_parity, g.sidx0, g.sidx1, g.bpr, (int)g.wave_rows);
        else
            gemm_compute(ring, g.kblocks, acc0, acc1, slot_off, block_parity);
        // epilogue: the lane holds column n of its two tiles; register r is row 8 (r / 4) + 4 h + r % 4
        const float *scales = row_scale[item_index & 3];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = 8 * (r >> 2) + 4 * h + (r & 3);
            if (m >= g.rows_here || wave >= g.waves) continue;
            const float rs = scales[m];
            if (MODE == PF_GEMM_GATE_UP) {
                const int unit = 32 * NW * g.slab + 32 * wave + n;
                const float gate = acc0[r] * rs, up = acc1[r] * rs;
                const float v = pf_silu(gate) * up;
                if (g.shared) a.shared_act[(size_t)(g.m0 + m) * g.inter + unit] = v;
                else a.act[(size_t)(g.first + g.m0 + m) * g.inter + unit] = v;
            } else {
                const int r0 = 64 * NW * g.slab + 64 * wave + n;
                float *out = a.down + (size_t)(g.first + g.m0 + m) * a.hidden;
                out[r0] = acc0[r] * rs;
                out[r0 + 32] = acc1[r] * rs;
            }
        }
        item_index++;
        q += gridDim.x;
    }
}

// ---- the grouped product for the other formats of real checkpoints --------------------------------
// Q8_0 (shared expert), Q2_K and MXFP4 (routed down projections) have no operand path in the ring
// kernel above.  This kernel computes the same items with the same operands' arithmetic (exact
// integer weight operands in fp16, two-part fp16 activations, FP32 accumulation, scales applied to
// the partial sums in FP32) but without the LDS ring: a workgroup is one row tile against one slab
// of 4 x 32 (gate/up) or 4 x 64 (down) weight rows, a wave takes its operands straight from global
// memory (the activation fragments are shared through the caches by the four waves and the slabs).
// Group scales that are not integers (Q8_0: a half per 32 weights; MXFP4: a power of two per 32)
// multiply the group's partial sums; Q2_K folds its 4-bit scale into the operand (scale * code
// <= 45) and obtains sum(min * x) from a second product with the minimum as the operand, as
// d * P - dmin * Q per 256-block.

// eight bytes as eight halfs, exact: a byte under the exponent byte 0x64 reads as 1024 + byte
__device__ __forceinline__ half8v half8_of_bytes(uint32_t b0, uint32_t b1, half_t offset) {
    const uint32_t bias = 0x64646464u;
    const half2v c = {offset, offset};
    const half2v v0 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, b0, 0x04010400u)) - c;
    const half2v v1 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, b0, 0x04030402u)) - c;
    const half2v v2 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, b1, 0x04010400u)) - c;
    const half2v v3 = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(bias, b1, 0x04030402u)) - c;
    return half8v{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
}
// signed bytes: flip the sign bit, read as unsigned, take 128 more away
__device__ __forceinline__ half8v half8_of_signed_bytes(uint32_t b0, uint32_t b1) {
    return half8_of_bytes(b0 ^ 0x80808080u, b1 ^ 0x80808080u, (half_t)1152.0f);
}

// Eight E2M1 codes (one per byte of two dwords, in the low nibble) as halfs holding twice their value:
// 0, 1, 2, 3, 4, 6, 8, 12 are 0x0000, 0x3C00, 0x4000, 0x4200, 0x4400, 0x4600, 0x4800, 0x4A00, so a byte
// permute looks up the halfs' high bytes, bit 3 of the code becomes the sign bit, and two more permutes
// spread the four bytes over two pairs of halfs (selector 0x0C writes a zero byte).
__device__ __forceinline__ half8v half8_of_e2m1(uint32_t n0, uint32_t n1) {
    auto pairs = [](uint32_t n, uint32_t &lo, uint32_t &hi) {
        uint32_t top = __builtin_amdgcn_perm(0x4A484644u, 0x42403C00u, n & 0x07070707u);
        top |= (n << 4) & 0x80808080u;
        lo = __builtin_amdgcn_perm(0u, top, 0x010C000Cu);
        hi = __builtin_amdgcn_perm(0u, top, 0x030C020Cu);
    };
    uint4 bits;
    pairs(n0, bits.x, bits.y);
    pairs(n1, bits.z, bits.w);
    return __builtin_bit_cast(half8v, bits);
}

struct PlainRow {            // one weight row as the kernel reads it
    const uint8_t *payload;  // first byte of the row (device layout of its format)
    const uint8_t *scales;   // first scale of the row, for the formats stored split
};

__device__ __forceinline__ PlainRow plain_row(const PfKernelArgs &a, int t, size_t e, size_t row) {
    const size_t index = e * a.n_out[t] + row;
    PlainRow r;
    r.payload = a.w[t] + index * a.row_bytes[t];
    r.scales = a.w[t] + a.scale_offset[t] + index * a.blocks_per_row[t] * (a.type[t] == PF_MXFP4 ? 1 : 2);
    return r;
}

// acc0 / acc1 += staged activation columns [c0, c0 + cols) x the same columns of weight rows r0 / r1.
// ahi / alo: this lane's activation row in LDS (high and low parts of the staged columns); sums: the
// row's sums over every 16 staged columns (high parts, low parts sums_low further on; Q2_K only).
// The weight bytes of several groups are requested before the first product of the batch.
// A wave takes every `parts`-th batch (256-block for Q2_K) starting with batch `part`: with parts > 1 the
// waves of a workgroup share one pair of rows and their partial sums are added afterwards.
template <int FMT>
__device__ __forceinline__ void plain_product(const PlainRow &r0, const PlainRow &r1, const half_t *ahi, const half_t *alo,
                                              const half_t *sums, int sums_low, int c0, int cols, int h, int part, int parts,
                                              float16v &acc0, float16v &acc1) {
    const float16v zero = {0};
    if (FMT == PF_Q2_K) {
        // a row's last block may be half used (logical width 640 of 768 stored): its second half is skipped,
        // and the sums of the groups beyond the width are zero
        for (int b = part; b < (cols + 255) / 256; b += parts) {
            const uint8_t *blk0 = r0.payload + 84 * (size_t)(c0 / 256 + b), *blk1 = r1.payload + 84 * (size_t)(c0 / 256 + b);
            const uint32_t dd0 = *reinterpret_cast<const uint32_t *>(blk0 + 80), dd1 = *reinterpret_cast<const uint32_t *>(blk1 + 80);
            float16v part0 = zero, part1 = zero;
            const uint32_t *sw0 = reinterpret_cast<const uint32_t *>(blk0), *sw1 = reinterpret_cast<const uint32_t *>(blk1);   // 4-byte aligned
            // Q: the 16 groups' minima (scale bytes 8h..8h+7, high nibbles) against the rows' sums over the same groups
            const half8v sh = *reinterpret_cast<const half8v *>(sums + 16 * b + 8 * h), sl = *reinterpret_cast<const half8v *>(sums + sums_low + 16 * b + 8 * h);
            const half8v mv0 = half8_of_bytes((sw0[2 * h] >> 4) & 0x0F0F0F0Fu, (sw0[2 * h + 1] >> 4) & 0x0F0F0F0Fu, (half_t)1024.0f);
            const half8v mv1 = half8_of_bytes((sw1[2 * h] >> 4) & 0x0F0F0F0Fu, (sw1[2 * h + 1] >> 4) & 0x0F0F0F0Fu, (half_t)1024.0f);
            float16v low0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh, mv0, zero, 0, 0, 0);
            float16v low1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(sh, mv1, zero, 0, 0, 0);
            low0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(sl, mv0, low0, 0, 0, 0);
            low1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(sl, mv1, low1, 0, 0, 0);
#pragma unroll
            for (int half = 0; half < 2; half++) {   // eight groups of 16 weights per batch: one 32-byte half of the codes
                if (256 * b + 128 * half >= cols) break;
                const uint32_t *q0 = reinterpret_cast<const uint32_t *>(blk0 + 16 + 32 * half + 8 * h);
                const uint32_t *q1 = reinterpret_cast<const uint32_t *>(blk1 + 16 + 32 * half + 8 * h);
                // bytes 8h..8h+7 and 16 + 8h..: the groups at l % 32 = 0 and 16, each at four bit planes
                const uint32_t c0a[2] = {q0[0], q0[1]}, c0b[2] = {q0[4], q0[5]}, c1a[2] = {q1[0], q1[1]}, c1b[2] = {q1[4], q1[5]};
                const uint32_t scales0[4] = {sw0[0], sw0[1], sw0[2], sw0[3]}, scales1[4] = {sw1[0], sw1[1], sw1[2], sw1[3]};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int gi = 8 * half + j, shift = 2 * (j >> 1), k = 256 * b + 16 * gi + 8 * h;
                    const uint32_t s0 = (scales0[gi >> 2] >> (8 * (gi & 3))) & 255u, s1 = (scales1[gi >> 2] >> (8 * (gi & 3))) & 255u;
                    const uint32_t *w0c = (j & 1) ? c0b : c0a, *w1c = (j & 1) ? c1b : c1a;
                    const half8v xh = *reinterpret_cast<const half8v *>(ahi + k), xl = *reinterpret_cast<const half8v *>(alo + k);
                    // byte-wise scale * code: at most 15 * 3, no carry between bytes
                    const half8v w0 = half8_of_bytes(((w0c[0] >> shift) & 0x03030303u) * (s0 & 15u), ((w0c[1] >> shift) & 0x03030303u) * (s0 & 15u), (half_t)1024.0f);
                    const half8v w1 = half8_of_bytes(((w1c[0] >> shift) & 0x03030303u) * (s1 & 15u), ((w1c[1] >> shift) & 0x03030303u) * (s1 & 15u), (half_t)1024.0f);
                    part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh, w0, part0, 0, 0, 0);
                    part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh, w1, part1, 0, 0, 0);
                    part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl, w0, part0, 0, 0, 0);
                    part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl, w1, part1, 0, 0, 0);
                }
            }
            const half2v h0 = __builtin_bit_cast(half2v, dd0), h1 = __builtin_bit_cast(half2v, dd1);
            const float d0 = (float)h0.x, n0 = (float)h0.y, d1 = (float)h1.x, n1 = (float)h1.y;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc0[r] = fmaf(d0, part0[r], fmaf(-n0, low0[r], acc0[r]));
                acc1[r] = fmaf(d1, part1[r], fmaf(-n1, low1[r], acc1[r]));
            }
        }
        return;
    }
    for (int g0 = 4 * part; g0 < cols / 32; g0 += 4 * parts) {   // batches of four groups of 32 weights (cols is a multiple of 128)
        const int first = c0 / 32 + g0;            // of the row's groups
        uint2 q0[4][2], q1[4][2];
        float s0[4], s1[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (FMT == PF_Q8_0) {
                s0[j] = (float)__builtin_bit_cast(half_t, reinterpret_cast<const uint16_t *>(r0.scales)[first + j]);
                s1[j] = (float)__builtin_bit_cast(half_t, reinterpret_cast<const uint16_t *>(r1.scales)[first + j]);
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    q0[j][t] = *reinterpret_cast<const uint2 *>(r0.payload + 32 * (size_t)(first + j) + 16 * t + 8 * h);
                    q1[j][t] = *reinterpret_cast<const uint2 *>(r1.payload + 32 * (size_t)(first + j) + 16 * t + 8 * h);
                }
            } else {   // MXFP4: bytes 8h..8h+7 of the block: low nibbles values 8h.., high nibbles values 16 + 8h..
                s0[j] = 0.5f * pf_e8m0_scale(r0.scales[first + j]);   // the operands are twice the values
                s1[j] = 0.5f * pf_e8m0_scale(r1.scales[first + j]);
                q0[j][0] = *reinterpret_cast<const uint2 *>(r0.payload + 16 * (size_t)(first + j) + 8 * h);
                q1[j][0] = *reinterpret_cast<const uint2 *>(r1.payload + 16 * (size_t)(first + j) + 8 * h);
                q0[j][1] = uint2{q0[j][0].x >> 4, q0[j][0].y >> 4};
                q1[j][1] = uint2{q1[j][0].x >> 4, q1[j][0].y >> 4};
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float16v part0 = zero, part1 = zero;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int k = 32 * (g0 + j) + 16 * t + 8 * h;
                const half8v xh = *reinterpret_cast<const half8v *>(ahi + k), xl = *reinterpret_cast<const half8v *>(alo + k);
                half8v w0, w1;
                if (FMT == PF_Q8_0) {
                    w0 = half8_of_signed_bytes(q0[j][t].x, q0[j][t].y);
                    w1 = half8_of_signed_bytes(q1[j][t].x, q1[j][t].y);
                } else {
                    w0 = half8_of_e2m1(q0[j][t].x & 0x0F0F0F0Fu, q0[j][t].y & 0x0F0F0F0Fu);
                    w1 = half8_of_e2m1(q1[j][t].x & 0x0F0F0F0Fu, q1[j][t].y & 0x0F0F0F0Fu);
                }
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh, w0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xh, w1, part1, 0, 0, 0);
                part0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl, w0, part0, 0, 0, 0);
                part1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xl, w1, part1, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc0[r] = fmaf(s0[j], part0[r], acc0[r]);
                acc1[r] = fmaf(s1[j], part1[r], acc1[r]);
            }
        }
    }
}

#define PLAIN_CHUNK 512                     // activation columns staged per pass
#define PLAIN_PITCH (PLAIN_CHUNK + 8)       // halfs between staged rows: 16 bytes of padding spread the rows over the banks
#define PLAIN_SUMS (PLAIN_CHUNK / 16 + 8)   // halfs between the rows' sums over 16 columns
#define PLAIN_TILE_BYTES (2 * 32 * PLAIN_PITCH * 2)
#define PLAIN_LDS (PLAIN_TILE_BYTES + 2 * 32 * PLAIN_SUMS * 2)

// grid: (row tiles the list can hold) x slabs; 4 waves.  Items whose tensors are in a format of the ring
// kernel are skipped here, as the ring kernel skips these.  Per pass the workgroup stages 512 columns
// of the tile's 32 activation rows (high and low parts) in LDS, one 1 KB row part per load instruction.
// split != 0 (gate/up only): the four waves share 32 units and take a quarter of the columns each; their
// partial sums meet in LDS and wave 0 adds them in wave order.  For matrices with few row tiles (the
// shared expert) that gives four times as many workgroups.
template <int MODE>
__global__ void __launch_bounds__(256) pf_k_pf_gemm_plain(PfKernelArgs a, int tokens, int slabs, int split) {
    extern __shared__ __align__(16) unsigned char plain_lds[];
    __shared__ uint32_t src_row[32];
    __shared__ float src_scale[32];
    half_t *tile = reinterpret_cast<half_t *>(plain_lds), *sums = reinterpret_cast<half_t *>(plain_lds + PLAIN_TILE_BYTES);
    const int lane = pf_lane(), wave = threadIdx.x >> 6, n = lane & 31, h = lane >> 5;
    const int E = a.experts, K = a.top_k, P = tokens * K;
    const uint32_t item_tile = blockIdx.x / slabs, slab = blockIdx.x % slabs;
    if (item_tile >= a.tiles[0]) return;
    const uint32_t entry = a.tiles[1 + item_tile];
    const int expert = entry & 0xffffu, m0 = 32 * (int)(entry >> 16);
    const bool shared = expert == E;
    const int first = shared ? P : (int)a.offsets[expert];
    const int count = shared ? tokens : (int)a.offsets[expert + 1] - first;
    if (count <= m0) return;
    const int rows_here = min(32, count - m0), inter = shared ? a.shared_inter : a.inter;
    const size_t ex = shared ? 0 : (size_t)expert;
    const int t0 = MODE == PF_GEMM_GATE_UP ? (shared ? 4 : 1) : (shared ? 6 : 3);
    const uint32_t fmt = a.type[t0];
    if (fmt != PF_Q8_0 && fmt != PF_Q2_K && fmt != PF_MXFP4) return;
    int row_a, row_b, t1, limit;
    const int slab_rows = MODE != PF_GEMM_GATE_UP ? 256 : split ? 32 : 128;
    if (MODE == PF_GEMM_GATE_UP) {
        limit = inter;
        row_a = row_b = slab_rows * (int)slab + (split ? 0 : 32 * wave) + n;   // the unit's gate row and up row
        t1 = t0 + 1;
    } else {
        limit = a.hidden;
        row_a = 256 * (int)slab + 64 * wave + n;
        row_b = row_a + 32;
        t1 = t0;
    }
    if (slab_rows * (int)slab >= limit) return;   // the slab starts beyond the matrix: the whole workgroup
    const bool active = row_a - n < limit;        // this wave has rows (the others stay for the barriers)
    const int part = split ? wave : 0, parts = split ? 4 : 1;
    // the tile's activation rows (the all-zero row beyond the tile's last) and their scales
    const int a_cols = MODE == PF_GEMM_GATE_UP ? a.hidden : inter;
    const half_t *a16 = reinterpret_cast<const half_t *>(MODE == PF_GEMM_GATE_UP ? a.x16 : shared ? a.sact16 : a.act16);
    const float *a_scale = MODE == PF_GEMM_GATE_UP ? a.x_scale : shared ? a.sact_scale : a.act_scale;
    if (threadIdx.x < 32) {
        const int m = threadIdx.x;
        uint32_t src;
        if (m >= rows_here) src = MODE == PF_GEMM_GATE_UP || shared ? a.token_cap : a.token_cap * (uint32_t)K;
        else if (shared) src = (uint32_t)(m0 + m);
        else src = MODE == PF_GEMM_GATE_UP ? a.row_to_pair[first + m0 + m] / (uint32_t)K : (uint32_t)(first + m0 + m);
        src_row[m] = src;
        src_scale[m] = m < rows_here ? a_scale[src] : 0.0f;
    }
    __syncthreads();
    const PlainRow r0 = plain_row(a, t0, ex, min(row_a, limit - 1)), r1 = plain_row(a, t1, ex, min(row_b, limit - 1));
    const half_t *ahi = tile + (size_t)n * PLAIN_PITCH, *alo = ahi + 32 * PLAIN_PITCH;
    float16v acc0 = {0}, acc1 = {0};
    for (int c0 = 0; c0 < a_cols; c0 += PLAIN_CHUNK) {
        const int cols = min(PLAIN_CHUNK, a_cols - c0);
        if (c0) __syncthreads();   // the previous pass has been consumed
        // 64 row parts (32 rows, high and low) over the four waves; a lane moves 16 bytes of each
#pragma unroll 4
        for (int i = 0; i < 16; i++) {
            const int part = 16 * wave + i, row = part & 31, low = part >> 5;
            if (16 * lane < 2 * cols)
                to_lds(a16 + (size_t)src_row[row] * pf_half_row(a_cols) + (size_t)low * a_cols + c0 + 8 * lane,
                       reinterpret_cast<unsigned char *>(tile + ((size_t)low * 32 + row) * PLAIN_PITCH));
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (fmt == PF_Q2_K) {
            // sums of the staged rows over every 16 columns, as two-part halfs like the values themselves:
            // thread = (row, four neighbouring groups)
            const int row = threadIdx.x >> 3, g0 = 4 * (threadIdx.x & 7);
#pragma unroll
            for (int g = g0; g < g0 + 4; g++) {
                float total = 0.0f;
                if (16 * g < cols) {
                    const half_t *hi = tile + (size_t)row * PLAIN_PITCH + 16 * g, *lo = hi + 32 * PLAIN_PITCH;
                    const half8v a0 = *reinterpret_cast<const half8v *>(hi), a1 = *reinterpret_cast<const half8v *>(hi + 8);
                    const half8v b0 = *reinterpret_cast<const half8v *>(lo), b1 = *reinterpret_cast<const half8v *>(lo + 8);
#pragma unroll
                    for (int i = 0; i < 8; i++) total += ((float)a0[i] + (float)b0[i]) + ((float)a1[i] + (float)b1[i]);
                }
                const half_t top = (half_t)total;
                sums[(size_t)row * PLAIN_SUMS + g] = top;
                sums[(size_t)(32 + row) * PLAIN_SUMS + g] = (half_t)(total - (float)top);
            }
            __syncthreads();
        }
        if (active) {
            const half_t *mine = sums + (size_t)n * PLAIN_SUMS;
            if (fmt == PF_Q8_0) plain_product<PF_Q8_0>(r0, r1, ahi, alo, mine, 32 * PLAIN_SUMS, c0, cols, h, part, parts, acc0, acc1);
            else if (fmt == PF_MXFP4) plain_product<PF_MXFP4>(r0, r1, ahi, alo, mine, 32 * PLAIN_SUMS, c0, cols, h, part, parts, acc0, acc1);
            else plain_product<PF_Q2_K>(r0, r1, ahi, alo, mine, 32 * PLAIN_SUMS, c0, cols, h, part, parts, acc0, acc1);
        }
    }
    if (split) {   // every wave is active here: the partial sums of waves 1..3 go through LDS (over the staged columns)
        __syncthreads();
        float *partial = reinterpret_cast<float *>(plain_lds);
        if (wave) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                partial[((wave - 1) * 32 + r) * 64 + lane] = acc0[r];
                partial[((wave - 1) * 32 + 16 + r) * 64 + lane] = acc1[r];
            }
        }
        __syncthreads();
        if (wave) return;
#pragma unroll
        for (int w = 0; w < 3; w++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc0[r] += partial[(w * 32 + r) * 64 + lane];
                acc1[r] += partial[(w * 32 + 16 + r) * 64 + lane];
            }
        }
    }
    if (!active) return;
    // epilogue: the lane holds column n of its two tiles; register r is row 8 (r / 4) + 4 h + r % 4
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int m = 8 * (r >> 2) + 4 * h + (r & 3);
        if (m >= rows_here) continue;
        const float rs = src_scale[m];
        if (MODE == PF_GEMM_GATE_UP) {
            if (row_a >= limit) continue;
            const float v = pf_silu(acc0[r] * rs) * (acc1[r] * rs);
            if (shared) a.shared_act[(size_t)(m0 + m) * inter + row_a] = v;
            else a.act[(size_t)(first + m0 + m) * inter + row_a] = v;
        } else {
            float *out = a.down + (size_t)(first + m0 + m) * a.hidden;
            if (row_a < limit) out[row_a] = acc0[r] * rs;
            if (row_b < limit) out[row_b] = acc1[r] * rs;
        }
    }
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
    // four columns a thread; the rows of sixteen slots at a time are all requested before the first of their sums
    for (int c = 4 * threadIdx.x; c < H; c += 4 * blockDim.x) {
        PfOutputRegs out_regs[4];
#pragma unroll
        for (int j = 0; j < 4; j++) pf_output_prefetch(a, t, c + j, out_regs[j]);
        const float4 sh = *reinterpret_cast<const float4 *>(a.down + (size_t)(P + t) * H + c);
        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int s0 = 0; s0 < K; s0 += 16) {
            float4 v[16];
#pragma unroll
            for (int s = 0; s < 16; s++)
                if (s0 + s < K) v[s] = *reinterpret_cast<const float4 *>(a.down + (size_t)rows[s0 + s] * H + c);
#pragma unroll
            for (int s = 0; s < 16; s++) {
                if (s0 + s < K) {
                    const float w = weights[s0 + s];
                    sum[0] += w * v[s].x; sum[1] += w * v[s].y; sum[2] += w * v[s].z; sum[3] += w * v[s].w;
                }
            }
        }
        const float y[4] = {sum[0] + ss * sh.x, sum[1] + ss * sh.y, sum[2] + ss * sh.z, sum[3] + ss * sh.w};
#pragma unroll
        for (int j = 0; j < 4; j++) bad |= !pf_output_commit(a, t, c + j, y[j], out_regs[j]);
    }
    if (__any(bad) && pf_lane() == 0) atomicOr(a.error_word, PF_HIP_ERR_NONFINITE);
}

// ---- dispatch --------------------------------------------------------------------------------------
// Routed gate and up in Q4_K or IQ2_XXS (the ring kernel's operand paths); the routed down tensor and the
// shared expert's three tensors in that same format or in Q2_K, MXFP4, Q8_0 (the plain grouped product).
bool pf_prefill_supported(const PfHipMoeDesc &d) {
    const uint32_t g = d.type[1];
    auto covered = [&](uint32_t t) { return t == g || t == PF_Q8_0 || t == PF_Q2_K || t == PF_MXFP4; };
    if ((g != PF_Q4_K && g != PF_IQ2_XXS) || d.type[2] != g || !covered(d.type[3])) return false;
    if (d.type[5] != d.type[4] || !covered(d.type[4]) || !covered(d.type[6])) return false;
    // widths: whole 256-blocks where the ring kernel reads them; where the plain kernel takes a down projection, whole
    // 128-column halves (the checkpoints' 640), and only Q2_K may be stored wider than its logical width
    auto width_ok = [&](uint32_t type, uint32_t k) { return k % (type == g ? 256u : 128u) == 0; };
    if (d.hidden % 256 || d.inter % 32 || d.shared_inter % 32 || !width_ok(d.type[3], d.inter) || !width_ok(d.type[6], d.shared_inter))
        return false;
    if (d.down_physical < d.inter || (d.down_physical != d.inter && d.type[3] != PF_Q2_K) ||
        (d.type[3] == PF_Q2_K && d.down_physical % 256))
        return false;
    if (d.top_k > 64 || d.top_k >= d.experts || d.experts >= 65535) return false;
    return true;
}

size_t pf_prefill_half_row(int cols) { return pf_half_row(cols); }
// sum over experts of ceil(rows / 32) <= pairs / 32 + experts, plus the shared expert's tiles
int pf_prefill_max_tiles(int tokens, int experts, int top_k) {
    return (int)(((size_t)tokens * top_k) / 32 + experts + (tokens + 31) / 32 + 1);
}

template <int MODE, int FMT>
static void launch_gemm(const PfKernelArgs &a, int tokens, int slabs, hipStream_t stream) {
    const size_t lds = FMT == PF_IQ2_XXS ? GEMM_LDS_IQ2 : GEMM_LDS;
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    static int grid = 0;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_pf_gemm<MODE, FMT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        int device = 0, units = 0;
        (void)hipGetDevice(&device);
        (void)hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
        grid = units >= 8 ? units / 8 * 8 : 8;   // one workgroup per compute unit (its LDS), a multiple of the XCD count
        configured = true;
    }
    // the item count is only known on the device: every workgroup walks the list from its own index
    hipLaunchKernelGGL((pf_k_pf_gemm<MODE, FMT>), dim3(grid), dim3(64 * (NW + NL)), lds, stream, a, tokens, slabs);
}

template <int MODE>
static void launch_gemm_plain(const PfKernelArgs &a, int tokens, unsigned tile_cap, int slabs, int split, hipStream_t stream) {
    static bool configured = false;   // once per instantiation: more than the default 64 KB of dynamic LDS
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(pf_k_pf_gemm_plain<MODE>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, PLAIN_LDS);
        configured = true;
    }
    hipLaunchKernelGGL(pf_k_pf_gemm_plain<MODE>, dim3(tile_cap * slabs), dim3(256), PLAIN_LDS, stream, a, tokens, slabs, split);
}

void pf_launch_prefill(const PfKernelArgs &a, int tokens, hipStream_t stream, int stage_limit) {
    const int H = a.hidden, E = a.experts, K = a.top_k, I = a.inter, Is = a.shared_inter, P = tokens * K;
    const int last = stage_limit ? stage_limit : 4;
    // stage 1: fp16 parts of x, router logits
    // (the shared router's column rides with the conversion: as a column of the router product it cost a 17th column
    // tile of full depth, and 544 workgroups do not spread evenly over 256 compute units, 512 do)
    hipLaunchKernelGGL(pf_k_rows_to_half, dim3(tokens), dim3(256), 0, stream, a.x, a.x_pitch, H, (half_t *)a.x16, a.x_scale,
                       a.x_max2, a.error_word, reinterpret_cast<const float *>(a.w[7]), a.shared_scale);
    hipLaunchKernelGGL(pf_k_pf_router, dim3((tokens + 31) / 32, (E + 31) / 32), dim3(256), 0, stream, a, tokens);
    if (last < 2) return;
    // stage 2: routes and grouping
    pf_launch_route(a, tokens, stream);
    if (!pf_launch_group_fused(a.ids, P, E, tokens, a.offsets, a.tiles, a.pair_to_row, a.row_to_pair, stream)) {
        hipLaunchKernelGGL(pf_k_pf_count, dim3((P + 255) / 256), dim3(256), 0, stream, a.ids, P, E, a.counts);
        hipLaunchKernelGGL(pf_k_pf_scan_tiles, dim3(1), dim3(256), 0, stream, a.counts, E, tokens, a.offsets, a.tiles);
        pf_launch_group_place(a.ids, P, E, a.offsets, a.pair_to_row, a.row_to_pair, stream);
    }
    if (last < 3) return;
    // stage 3: gate/up + SwiGLU, then fp16 parts of the activation rows
    // the ring kernel takes the items whose tensors are in the routed gate's format, the plain kernel the rest
    const int gi = I > Is ? I : Is;
    const bool iq2 = a.type[1] == PF_IQ2_XXS;
    const uint32_t ring_fmt = a.type[1];
    const unsigned tile_cap = (unsigned)pf_prefill_max_tiles(tokens, E, K);
    if (iq2) launch_gemm<PF_GEMM_GATE_UP, PF_IQ2_XXS>(a, tokens, (gi + 32 * NW - 1) / (32 * NW), stream);
    else launch_gemm<PF_GEMM_GATE_UP, PF_Q4_K>(a, tokens, (gi + 32 * NW - 1) / (32 * NW), stream);
    // only the shared expert's tiles (tokens / 32 of them) are left for this launch: columns split over the waves
    if (a.type[4] != ring_fmt) launch_gemm_plain<PF_GEMM_GATE_UP>(a, tokens, tile_cap, (gi + 31) / 32, 1, stream);
    if (I <= 512 && Is <= 512 && P > 0 && tokens > 0) {
        const unsigned blocks_a = (unsigned)((P + 3) / 4), blocks_b = (unsigned)((tokens + 3) / 4);
        hipLaunchKernelGGL(pf_k_rows_to_half_short2, dim3(blocks_a + blocks_b), dim3(256), 0, stream, a.act, I, (size_t)P,
                           (half_t *)a.act16, a.act_scale, blocks_a, a.shared_act, Is, (size_t)tokens, (half_t *)a.sact16, a.sact_scale,
                           a.error_word);
    } else {
        launch_rows_to_half(a.act, (size_t)I, I, (size_t)P, (half_t *)a.act16, a.act_scale, nullptr, a.error_word, stream);
        launch_rows_to_half(a.shared_act, (size_t)Is, Is, (size_t)tokens, (half_t *)a.sact16, a.sact_scale, nullptr, a.error_word, stream);
    }
    if (last < 4) return;
    // stage 4: down and combine
    if (a.type[3] == ring_fmt || a.type[6] == ring_fmt) {
        if (iq2) launch_gemm<PF_GEMM_DOWN, PF_IQ2_XXS>(a, tokens, (H + 64 * NW - 1) / (64 * NW), stream);
        else launch_gemm<PF_GEMM_DOWN, PF_Q4_K>(a, tokens, (H + 64 * NW - 1) / (64 * NW), stream);
    }
    if (a.type[3] != ring_fmt || a.type[6] != ring_fmt) launch_gemm_plain<PF_GEMM_DOWN>(a, tokens, tile_cap, (H + 255) / 256, 0, stream);
    hipLaunchKernelGGL(pf_k_pf_combine, dim3(tokens), dim3(256), 0, stream, a, tokens);
}
