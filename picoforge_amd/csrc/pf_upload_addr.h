// What one thread of an upload kernel moves, as functions that compile for the host as well: the kernels that lay a
// layer's tensors out in device memory (the scale/payload split of IQ2_XXS, Q8_0 and MXFP4, the tile orders of Q4_K,
// IQ2_XXS and Q8_0) call them for their addresses, and a host-side test walks every thread of every launch and checks
// that each read ends inside the source buffer and each write inside the destination allocation.
#pragma once
#include "pf_decode_addr.h"

struct PfMove {
    bool active;        // false: the thread is beyond the work and moves nothing
    int to;             // 0: the destination's payload (or only) buffer, 1: its scales
    size_t src, dst;    // byte offsets
    uint32_t width;     // bytes moved (a second source of the same width at src2 where src2_used)
    bool src2_used;
    size_t src2;        // Q8_0 tile order: the second half scale of the pair
    int from;           // 0: the source's payload (or only) buffer, 1: its scales
};

// ---- Q4_K into tile order (pf_k_q4k_tile): one thread per 16-byte piece; rows a multiple of 32 ------------------------
PF_HD size_t pf_q4k_tile_threads(size_t rows, int blocks_per_row) { return rows * (size_t)blocks_per_row * 9; }
PF_HD PfMove pf_q4k_tile_move(size_t piece, size_t rows, int blocks_per_row) {
    PfMove m = {};
    if (piece >= pf_q4k_tile_threads(rows, blocks_per_row)) return m;
    const size_t chunk = piece / 288, tile = chunk / blocks_per_row, kb = chunk % blocks_per_row;
    const int p = (int)(piece % 288);
    size_t n, off;
    if (p < 32) {
        n = p; off = 0;
    } else {
        const int q = p - 32;
        n = q & 31; off = 16 + 32 * (size_t)(q >> 6) + 16 * (size_t)((q >> 5) & 1);
    }
    const size_t row_bytes = (size_t)blocks_per_row * 144;
    m.active = true; m.width = 16;
    m.src = (32 * tile + n) * row_bytes + 144 * kb + off;
    m.dst = 16 * piece;
    return m;
}

// ---- IQ2_XXS split (pf_k_iq2_split): one thread per 16-bit word of a 66-byte block ----------------------------------
PF_HD size_t pf_iq2_split_threads(size_t blocks) { return blocks * 33; }
PF_HD PfMove pf_iq2_split_move(size_t i, size_t blocks) {
    PfMove m = {};
    const size_t b = i / 33, h = i % 33;
    if (b >= blocks) return m;
    m.active = true; m.width = 2;
    m.src = 2 * (b * 33 + h);
    if (h == 0) { m.to = 1; m.dst = 2 * b; }
    else { m.to = 0; m.dst = 2 * (b * 32 + (h - 1)); }
    return m;
}

// ---- any format whose block leads with its scale (pf_k_block_split): one thread per byte ------------------------------
PF_HD size_t pf_block_split_threads(size_t blocks, int block_bytes) { return blocks * (size_t)block_bytes; }
PF_HD PfMove pf_block_split_move(size_t i, size_t blocks, int block_bytes, int header_bytes) {
    PfMove m = {};
    const size_t b = i / block_bytes;
    const int h = (int)(i % block_bytes);
    if (b >= blocks) return m;
    m.active = true; m.width = 1; m.src = i;
    if (h < header_bytes) { m.to = 1; m.dst = b * header_bytes + h; }
    else { m.to = 0; m.dst = b * (size_t)(block_bytes - header_bytes) + (h - header_bytes); }
    return m;
}

// ---- IQ2_XXS into tile order (pf_k_iq2_tile): per (32-row tile, 256-block) chunk 128 piece threads and 32 scale threads ----
PF_HD size_t pf_iq2_tile_threads(size_t rows, int blocks_per_row) { return rows / 32 * (size_t)blocks_per_row * 160; }
PF_HD PfMove pf_iq2_tile_move(size_t i, size_t rows, int blocks_per_row) {
    PfMove m = {};
    const size_t per_chunk = 128 + 32;
    const size_t chunk = i / per_chunk, tile = chunk / blocks_per_row, kb = chunk % blocks_per_row;
    if (chunk >= rows / 32 * (size_t)blocks_per_row) return m;
    const int p = (int)(i % per_chunk);
    m.active = true;
    if (p < 128) {
        const int run = p >> 5, row = p & 31;
        const size_t n = 32 * tile + row;
        m.width = 16; m.from = 0;
        m.src = (n * blocks_per_row + kb) * 64 + 16 * (size_t)run;
        m.dst = chunk * PF_I2T_CHUNK + pf_i2t_piece_at(run, row);
    } else {
        const int row = p - 128;
        const size_t n = 32 * tile + row;
        m.width = 2; m.from = 1;
        m.src = 2 * (n * blocks_per_row + kb);
        m.dst = chunk * PF_I2T_CHUNK + pf_i2t_scale_at(row);
    }
    return m;
}

// ---- Q8_0 into tile order (pf_k_q8_tile): per (32-row tile, 64-weight run) chunk 128 piece threads and 32 scale-pair threads ----
PF_HD size_t pf_q8_tile_threads(size_t rows, int blocks_per_row) { return rows / 32 * (size_t)(blocks_per_row / 2) * 160; }
PF_HD PfMove pf_q8_tile_move(size_t i, size_t rows, int blocks_per_row) {
    PfMove m = {};
    const size_t per_chunk = 128 + 32;
    const int runs = blocks_per_row / 2;
    const size_t chunk = i / per_chunk, tile = chunk / runs, run = chunk % runs;
    if (chunk >= rows / 32 * (size_t)runs) return m;
    const int p = (int)(i % per_chunk);
    m.active = true;
    if (p < 128) {
        const int piece = p >> 5, row = p & 31;
        const size_t n = 32 * tile + row;
        m.width = 16; m.from = 0;
        m.src = (n * blocks_per_row + 2 * run) * 32 + 16 * (size_t)piece;
        m.dst = chunk * PF_I2T_CHUNK + pf_q8t_piece_at(piece, row);
    } else {
        const int row = p - 128;
        const size_t n = 32 * tile + row, b = n * blocks_per_row + 2 * run;
        m.width = 2; m.from = 1;          // two half scales, 2 bytes each, written as one dword
        m.src = 2 * b; m.src2_used = true; m.src2 = 2 * (b + 1);
        m.dst = chunk * PF_I2T_CHUNK + pf_q8t_scales_at(row);
    }
    return m;
}
