// Device layout of the weight tensors and the byte offsets the decode kernels read, as functions that
// compile for the host as well: the kernels call them for their addresses, pf_hip_moe_create for its
// allocation sizes, and a host-side test walks every (tensor, expert, row, segment) a launch can name and
// checks that each read ends inside the tensor's allocation.
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define PF_HD __host__ __device__ __forceinline__
#else
#define PF_HD static inline
#endif

// GGUF type ids and block geometry (src/gguf.c:12-16 of the reference).
enum { PF_F32 = 0, PF_F16 = 1, PF_Q8_0 = 8, PF_Q2_K = 10, PF_Q4_K = 12, PF_IQ2_XXS = 16, PF_BF16 = 30, PF_MXFP4 = 39 };

PF_HD bool pf_block_geometry(uint32_t type, size_t *block, size_t *bytes) {
    switch (type) {
    case PF_F32: *block = 1; *bytes = 4; return true;
    case PF_F16: case PF_BF16: *block = 1; *bytes = 2; return true;
    case PF_Q8_0: *block = 32; *bytes = 34; return true;
    case PF_Q2_K: *block = 256; *bytes = 84; return true;
    case PF_Q4_K: *block = 256; *bytes = 144; return true;
    case PF_IQ2_XXS: *block = 256; *bytes = 66; return true;
    case PF_MXFP4: *block = 32; *bytes = 17; return true;
    default: return false;
    }
}

// Formats stored split on the device (payloads, then scales): bytes of a block's leading scale, else 0.
PF_HD size_t pf_split_header_bytes(uint32_t type) {
    return type == PF_IQ2_XXS || type == PF_Q8_0 ? 2 : type == PF_MXFP4 ? 1 : 0;
}

struct PfTensorPlace {
    size_t row_bytes, expert_bytes;   // of the payload (split formats: without the scales)
    size_t scale_offset;              // split formats: byte offset of the scales in the tensor's buffer
    size_t bytes, gguf_bytes;         // of the device buffer; of the tensor as GGUF stores it
    int n_out, blocks_per_row;
};

// One tensor of k_storage x n_out x experts weights in the device layout.  False: unknown type or a row that is
// not whole blocks.
PF_HD bool pf_tensor_place(uint32_t type, size_t k_storage, size_t n_out, size_t experts, PfTensorPlace *p) {
    size_t block, size;
    if (!pf_block_geometry(type, &block, &size) || k_storage % block) return false;
    const size_t blocks_per_row = k_storage / block, rows = n_out * experts, head = pf_split_header_bytes(type);
    p->gguf_bytes = blocks_per_row * size * rows;
    p->n_out = (int)n_out;
    p->blocks_per_row = (int)blocks_per_row;
    if (head) {
        // every block's payload (64, 32 or 16 bytes), then every block's scale; four bytes of slack because the prefill
        // loader reads the dword around a scale
        const size_t payload = size - head;
        p->row_bytes = blocks_per_row * payload;
        p->scale_offset = (blocks_per_row * rows * payload + 255) & ~(size_t)255;
        p->bytes = p->scale_offset + blocks_per_row * rows * head + 4;
    } else {
        p->row_bytes = blocks_per_row * size;
        p->scale_offset = 0;
        p->bytes = p->gguf_bytes;
    }
    p->expert_bytes = p->row_bytes * n_out;
    return true;
}

// ---- launch geometry of the decode kernels --------------------------------------------------------
// Lanes that share one row of K values: the largest power of two that is at most K / 64 and at most 32.  A lane
// takes the 64-value segment `seg` of the row and, where K / 64 is not that power of two (K = 2560: 40 segments
// on 32 lanes, K = 640: 10 on 8), also segment seg + lanes if the row has one.
PF_HD int row_lanes(int K) {
    int l = 1;
    while (2 * l <= K / 64 && l < 32) l *= 2;
    return l;
}
PF_HD int row_passes(int K) { return (K / 64 + row_lanes(K) - 1) / row_lanes(K); }
// Rows of the down projection per workgroup of kernel 3: what one wave covers in a step, doubled until the row
// blocks of one token fit the 256 compute units (hidden 2560, intermediate 640: 16 rows, 160 blocks).
PF_HD int down_block_rows(int H, int I) {
    int rows = 64 / row_lanes(I);
    while ((H + rows - 1) / rows > 256 && rows < 64) rows *= 2;
    return rows;
}

// ---- what one lane reads of a row's 64-weight segment ------------------------------------------------
struct PfSpan { size_t at; uint32_t width; };   // bytes [at, at + width) of the tensor's buffer

// Row n of expert e; seg = the segment.  Returns the number of spans (at most 4).
PF_HD int pf_segment_spans(uint32_t type, const PfTensorPlace &p, size_t e, size_t n, int seg, PfSpan out[4]) {
    const size_t row = e * p.expert_bytes + n * p.row_bytes, block_index = (e * p.n_out + n) * p.blocks_per_row;
    switch (type) {
    case PF_Q4_K: {   // the block's 16-byte header, the 32 code bytes of the segment
        const size_t blk = row + (size_t)(seg >> 2) * 144;
        out[0] = {blk, 16};
        out[1] = {blk + 16 + 32 * (size_t)(seg & 3), 32};
        return 2;
    }
    case PF_IQ2_XXS:   // 16 payload bytes; the block's half scale
        out[0] = {row + 16 * (size_t)seg, 16};
        out[1] = {p.scale_offset + 2 * (block_index + (size_t)(seg >> 2)), 2};
        return 2;
    case PF_Q8_0:   // two blocks of 32 code bytes; their two half scales as one dword
        out[0] = {row + 64 * (size_t)seg, 64};
        out[1] = {p.scale_offset + 2 * (block_index + 2 * (size_t)seg), 4};
        return 2;
    case PF_MXFP4:   // two blocks of 16 nibble bytes; their two scale bytes
        out[0] = {row + 32 * (size_t)seg, 32};
        out[1] = {p.scale_offset + block_index + 2 * (size_t)seg, 2};
        return 2;
    case PF_Q2_K: {   // 84-byte blocks: 32 code bytes of the segment's half, four scale bytes, d and dmin
        const size_t blk = row + (size_t)(seg >> 2) * 84;
        out[0] = {blk + 16 + 32 * (size_t)((seg & 3) >> 1), 32};
        out[1] = {blk + 4 * (size_t)(seg & 3), 4};
        out[2] = {blk + 80, 4};
        return 3;
    }
    default: return 0;
    }
}

// The dword one thread of a warm-up workgroup touches: line l of the `lines` 128-byte steps over the rows
// [row0, row0 + rows) of expert e (the last step: the rows' scales where they are stored apart).  False: nothing.
PF_HD bool pf_warm_span(uint32_t type, const PfTensorPlace &p, size_t e, size_t row0, int rows, int l, int lines, PfSpan *out) {
    const size_t bytes = (size_t)rows * p.row_bytes;
    size_t at = e * p.expert_bytes + row0 * p.row_bytes;
    if (l == lines - 1) {
        if (!p.scale_offset) return false;
        const size_t each = type == PF_MXFP4 ? 1 : 2;
        at = p.scale_offset + (e * p.n_out + row0) * p.blocks_per_row * each;
    } else {
        const size_t step = (size_t)l * 128;
        at += step < bytes - 4 ? step : bytes - 4;
    }
    out->at = at & ~(size_t)3;   // buffers are 256-byte aligned: rounding the offset down is rounding the address down
    out->width = 4;
    return true;
}

// ---- tile-ordered Q4_K (32 rows x one 256-block = 4608 bytes: 32 headers, then per 64-weight run the rows' halves) ----
PF_HD size_t pf_q4t_chunk_at(size_t expert_bytes, size_t e, int row_tile, int kblocks, int kb) {
    return e * expert_bytes + ((size_t)row_tile * kblocks + kb) * 4608;
}
PF_HD size_t pf_q4t_header_at(int row_in_tile) { return 16 * (size_t)row_in_tile; }
PF_HD size_t pf_q4t_piece_at(int run, int half, int row_in_tile) { return 512 + (size_t)run * 1024 + (size_t)half * 512 + 16 * (size_t)row_in_tile; }

// ---- tile-ordered IQ2_XXS (32 rows x one 256-block = 2176 bytes: per 64-weight run the rows' 16-byte pieces -- two
// 32-groups of four grid indices and a sign/scale word each -- then the rows' 32 half scales and 64 bytes of padding
// that keep every piece group on whole 128-byte lines) ----
#define PF_I2T_CHUNK 2176
PF_HD size_t pf_i2t_expert_bytes(int n_out, int kblocks) { return (size_t)(n_out / 32) * kblocks * PF_I2T_CHUNK; }
PF_HD size_t pf_i2t_chunk_at(size_t expert_bytes, size_t e, int row_tile, int kblocks, int kb) {
    return e * expert_bytes + ((size_t)row_tile * kblocks + kb) * PF_I2T_CHUNK;
}
PF_HD size_t pf_i2t_scale_at(int row_in_tile) { return 2048 + 2 * (size_t)row_in_tile; }
PF_HD size_t pf_i2t_piece_at(int run, int row_in_tile) { return (size_t)run * 512 + 16 * (size_t)row_in_tile; }

// ---- tile-ordered Q8_0 (the shared expert of the checkpoint profiles; 32 rows x one 64-weight run = 2176 bytes: the
// rows' 64 code bytes as four 16-byte pieces, piece by piece, then the rows' two half scales each, then padding) ----
PF_HD size_t pf_q8t_expert_bytes(int n_out, int runs) { return (size_t)(n_out / 32) * runs * PF_I2T_CHUNK; }
PF_HD size_t pf_q8t_chunk_at(size_t expert_bytes, size_t e, int row_tile, int runs, int run) {
    return e * expert_bytes + ((size_t)row_tile * runs + run) * PF_I2T_CHUNK;
}
PF_HD size_t pf_q8t_piece_at(int piece, int row_in_tile) { return (size_t)piece * 512 + 16 * (size_t)row_in_tile; }
PF_HD size_t pf_q8t_scales_at(int row_in_tile) { return 2048 + 4 * (size_t)row_in_tile; }
