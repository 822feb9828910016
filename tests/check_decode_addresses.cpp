// Host-side walk over every byte range the decode kernels can read from a layer's weight buffers.
// Compiled with g++ by tests/test_decode_addresses.py; includes the header the kernels take their offsets from
// (picoforge_amd/csrc/pf_decode_addr.h), so what is checked here is what the device executes.
//
// For a layer (hidden, experts, top_k, inter, shared_inter, down_physical, the tensors' types) it restates the
// launch geometry of the three decode kernels and of the warm-up workgroups -- which (tensor, expert, row,
// segment) each lane names -- and checks that every span ends inside the tensor's device allocation, that
// 16-byte reads are 16-byte aligned and dword reads 4-byte aligned.  Prints the number of spans checked;
// exit status 1 and the first offenders on a violation.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <initializer_list>
#include "../picoforge_amd/csrc/pf_decode_addr.h"

static long long checked = 0, bad = 0;

static void check(const char *what, int tensor, const PfTensorPlace &p, PfSpan s, unsigned align, size_t e, size_t n, int seg) {
    checked++;
    const bool inside = s.at + s.width <= p.bytes, aligned = s.at % align == 0;
    if (inside && aligned) return;
    if (bad++ < 10)
        fprintf(stderr, "%s: tensor %d expert %zu row %zu segment %d: [%zu, +%u) %s (buffer %zu bytes)\n", what, tensor, e, n, seg,
                s.at, s.width, inside ? "misaligned" : "beyond the buffer", p.bytes);
}

static unsigned span_alignment(uint32_t type, int index) {
    // what the loaders assume: 16-byte vector reads of headers and codes, dword or narrower reads of scales
    switch (type) {
    case PF_Q4_K: return 16;
    case PF_IQ2_XXS: return index == 0 ? 16 : 2;
    case PF_Q8_0: return index == 0 ? 16 : 4;
    case PF_MXFP4: return index == 0 ? 16 : 2;
    case PF_Q2_K: return 4;
    default: return 1;
    }
}

int main(int argc, char **argv) {
    if (argc != 15) {
        fprintf(stderr, "usage: %s hidden experts top_k inter shared_inter down_physical type0..type7\n", argv[0]);
        return 2;
    }
    const int H = atoi(argv[1]), E = atoi(argv[2]), I = atoi(argv[4]), Is = atoi(argv[5]), phys = atoi(argv[6]);
    uint32_t type[8];
    for (int a = 0; a < 8; a++) type[a] = (uint32_t)atoi(argv[7 + a]);
    const size_t k_storage[8] = {(size_t)H, (size_t)H, (size_t)H, (size_t)phys, (size_t)H, (size_t)H, (size_t)Is, (size_t)H};
    const size_t n_out[8] = {(size_t)E, (size_t)I, (size_t)I, (size_t)H, (size_t)Is, (size_t)Is, (size_t)H, 1};
    const size_t experts[8] = {1, (size_t)E, (size_t)E, (size_t)E, 1, 1, 1, 1};
    PfTensorPlace place[8];
    for (int a = 0; a < 8; a++)
        if (!pf_tensor_place(type[a], k_storage[a], n_out[a], experts[a], &place[a])) { fprintf(stderr, "tensor %d: no layout\n", a); return 2; }
    const size_t some_experts[4] = {0, 1, (size_t)E / 2, (size_t)E - 1};

    // kernel 2 (gate and up rows of a routed expert, of the shared expert): every unit, every segment of hidden,
    // including the second segment of the lanes that take two
    for (int a : {1, 2, 4, 5}) {
        const int rows = a <= 2 ? I : Is;
        for (size_t e : some_experts) {
            if (a >= 4 && e) continue;
            for (int n = 0; n < rows; n++)
                for (int seg = 0; seg < H / 64; seg++) {
                    PfSpan sp[4];
                    const int count = pf_segment_spans(type[a], place[a], e, (size_t)n, seg, sp);
                    if (!count) { fprintf(stderr, "tensor %d: a format without a decode loader\n", a); return 2; }
                    for (int i = 0; i < count; i++) check("gate/up", a, place[a], sp[i], span_alignment(type[a], i), e, n, seg);
                }
        }
    }
    // kernel 3 (down rows): the logical width only; rows clamp to hidden - 1
    for (int a : {3, 6}) {
        const int width = a == 3 ? I : Is;
        const int rows_per_block = down_block_rows(H, I), row_blocks = (H + rows_per_block - 1) / rows_per_block;
        const int LPR = row_lanes(width), per_step = 64 / LPR, steps = per_step >= rows_per_block ? 1 : rows_per_block / per_step;
        for (size_t e : some_experts) {
            if (a == 6 && e) continue;
            for (int nb = 0; nb < row_blocks; nb++)
                for (int st = 0; st < steps; st++)
                    for (int lane = 0; lane < 64; lane++) {
                        const int seg = lane & (LPR - 1), r = lane / LPR;
                        int n = nb * rows_per_block + st * per_step + r;
                        if (n > H - 1) n = H - 1;
                        for (int pass = 0; pass < row_passes(width); pass++) {
                            const int s = seg + pass * LPR;
                            if (s >= width / 64) continue;
                            PfSpan sp[4];
                            const int count = pf_segment_spans(type[a], place[a], e, (size_t)n, s, sp);
                            for (int i = 0; i < count; i++) check("down", a, place[a], sp[i], span_alignment(type[a], i), e, n, s);
                        }
                    }
        }
    }
    // the warm-up workgroups of kernel 2: every (slot, row block) item, every line
    {
        const int rows = down_block_rows(H, I), row_blocks = (H + rows - 1) / rows;
        const size_t widest = (size_t)rows * (place[3].row_bytes > place[6].row_bytes ? place[3].row_bytes : place[6].row_bytes);
        const int lines = (int)((widest + 127) / 128) + 1;
        for (int a : {3, 6})
            for (size_t e : some_experts) {
                if (a == 6 && e) continue;
                for (int nb = 0; nb < row_blocks; nb++)
                    for (int l = 0; l < lines; l++) {
                        PfSpan sp;
                        if (pf_warm_span(type[a], place[a], e, (size_t)nb * rows, rows, l, lines, &sp)) check("warm-up", a, place[a], sp, 4, e, nb * rows, l);
                    }
            }
    }
    // the tile-ordered Q4_K copies (same size as the row order): the row-as-lane kernels
    if (type[1] == PF_Q4_K && type[2] == PF_Q4_K && type[3] == PF_Q4_K && type[4] == PF_Q4_K && type[5] == PF_Q4_K && type[6] == PF_Q4_K &&
        H % 256 == 0 && I % 32 == 0 && Is % 32 == 0 && phys == I && I % 256 == 0 && Is % 256 == 0) {
        for (int a = 1; a <= 6; a++) {
            const int rows = (int)n_out[a], kblocks = (int)k_storage[a] / 256;
            for (size_t e : some_experts) {
                if (experts[a] == 1 && e) continue;
                for (int n = 0; n < rows; n++)
                    for (int kb = 0; kb < kblocks; kb++) {
                        const size_t chunk = pf_q4t_chunk_at(place[a].expert_bytes, e, n / 32, kblocks, kb);
                        check("tile header", a, place[a], {chunk + pf_q4t_header_at(n & 31), 16}, 16, e, n, kb);
                        for (int run = 0; run < 4; run++)
                            for (int h = 0; h < 2; h++)
                                check("tile piece", a, place[a], {chunk + pf_q4t_piece_at(run, h, n & 31), 16}, 16, e, n, 4 * kb + run);
                    }
            }
        }
    }
    // the tile-ordered IQ2_XXS copies (their own size: PF_I2T_CHUNK bytes per 32 rows and 256-block): every IQ2_XXS
    // expert tensor of a layer that is IQ2_XXS throughout, the routed gate and up tensors of the q2 profile
    for (int a = 1; a <= 6; a++) {
        if (type[a] != PF_IQ2_XXS || n_out[a] % 32 || k_storage[a] % 256) continue;
        const int rows = (int)n_out[a], kblocks = (int)k_storage[a] / 256;
        PfTensorPlace copy = place[a];
        copy.expert_bytes = pf_i2t_expert_bytes(rows, kblocks);
        copy.bytes = copy.expert_bytes * experts[a];
        for (size_t e : some_experts) {
            if (experts[a] == 1 && e) continue;
            for (int n = 0; n < rows; n++)
                for (int kb = 0; kb < kblocks; kb++) {
                    const size_t chunk = pf_i2t_chunk_at(copy.expert_bytes, e, n / 32, kblocks, kb);
                    check("tile scale", a, copy, {chunk + pf_i2t_scale_at(n & 31), 2}, 2, e, n, kb);
                    for (int run = 0; run < 4; run++)
                        check("tile piece", a, copy, {chunk + pf_i2t_piece_at(run, n & 31), 16}, 16, e, n, 4 * kb + run);
                }
        }
    }
    // the tile-ordered Q8_0 copies of the profiles' shared gate and up tensors: one chunk per 64-weight run, addressed by
    // the gate/up kernel as four chunks per 256-block
    for (int a : {4, 5}) {
        if (type[a] != PF_Q8_0 || n_out[a] % 32 || k_storage[a] % 256) continue;
        const int rows = (int)n_out[a], kblocks = (int)k_storage[a] / 256, runs = 4 * kblocks;
        PfTensorPlace copy = place[a];
        copy.expert_bytes = pf_q8t_expert_bytes(rows, runs);
        copy.bytes = copy.expert_bytes;
        for (int n = 0; n < rows; n++)
            for (int kb = 0; kb < kblocks; kb++)
                for (int run = 0; run < 4; run++) {
                    const size_t chunk = pf_q8t_chunk_at(0, 0, n / 32, runs, 4 * kb) + (size_t)run * PF_I2T_CHUNK;
                    check("tile scales", a, copy, {chunk + pf_q8t_scales_at(n & 31), 4}, 4, 0, n, 4 * kb + run);
                    for (int p = 0; p < 4; p++)
                        check("tile piece", a, copy, {chunk + pf_q8t_piece_at(p, n & 31), 16}, 16, 0, n, 4 * kb + run);
                }
    }
    printf("%lld spans checked, %lld outside or misaligned\n", checked, bad);
    return bad ? 1 : 0;
}
