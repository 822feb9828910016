// Host-side walk over every thread of every kernel that lays a layer's tensors out in device memory at
// pf_hip_moe_create (and when a pool stores an expert): the scale/payload split of IQ2_XXS, Q8_0 and MXFP4, the
// tile orders of Q4_K, IQ2_XXS and Q8_0.  Compiled with g++ by tests/test_upload_addresses.py; includes the
// header the kernels take their addresses from (picoforge_amd/csrc/pf_upload_addr.h), so what is checked here is
// what the device executes.  For each tensor of a layer it walks the launch as the library makes it -- every
// thread of the rounded-up grid -- and checks that each read ends inside the source buffer, each write inside the
// destination allocation (sizes as pf_hip_moe_create takes them: pf_tensor_place, pf_i2t_expert_bytes,
// pf_q8t_expert_bytes), that vector accesses are aligned, and that every byte of the destination that the decode
// and prefill kernels later read is written exactly once.  Prints the number of moves checked; exit status 1 on a
// violation.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "../picoforge_amd/csrc/pf_upload_addr.h"

static long long checked = 0, bad = 0;

struct Buffer { const char *name; size_t payload_bytes, scale_offset, scale_bytes, bytes; };   // one allocation: payload, then scales

static void complain(const char *kernel, const char *what, size_t thread, size_t at, unsigned width, size_t limit) {
    if (bad++ < 10) fprintf(stderr, "%s thread %zu: %s [%zu, +%u) against %zu bytes\n", kernel, thread, what, at, width, limit);
}

// walks `threads` rounded up to whole 256-thread workgroups
template <class MoveOf>
static void walk(const char *kernel, size_t threads, MoveOf move_of, const Buffer &src, const Buffer &dst, std::vector<unsigned char> *written) {
    const size_t launched = (threads + 255) / 256 * 256;
    for (size_t i = 0; i < launched; i++) {
        const PfMove m = move_of(i);
        if (!m.active) {
            if (i < threads) complain(kernel, "idle inside the work", i, 0, 0, threads);
            continue;
        }
        if (i >= threads) complain(kernel, "active beyond the work", i, 0, 0, threads);
        checked++;
        const size_t src_base = m.from ? src.scale_offset : 0, src_limit = m.from ? src.scale_offset + src.scale_bytes : src.payload_bytes;
        const size_t dst_base = m.to ? dst.scale_offset : 0, dst_limit = m.to ? dst.scale_offset + dst.scale_bytes : dst.payload_bytes;
        const unsigned wide = m.src2_used ? 2 * m.width : m.width;   // bytes written
        if (src_base + m.src + m.width > src_limit || src_limit > src.bytes) complain(kernel, "reads", i, src_base + m.src, m.width, src_limit);
        if (m.src2_used && src_base + m.src2 + m.width > src_limit) complain(kernel, "reads (second)", i, src_base + m.src2, m.width, src_limit);
        if (dst_base + m.dst + wide > dst_limit || dst_limit > dst.bytes) complain(kernel, "writes", i, dst_base + m.dst, wide, dst_limit);
        if ((src_base + m.src) % m.width || (dst_base + m.dst) % wide) complain(kernel, "misaligned", i, dst_base + m.dst, wide, 0);
        if (written && dst_base + m.dst + wide <= written->size())
            for (unsigned b = 0; b < wide; b++)
                if ((*written)[dst_base + m.dst + b]++) complain(kernel, "writes a byte twice", i, dst_base + m.dst + b, 1, 0);
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
    // routed tensors: a few experts' worth of rows stand for all of them where the kernel's addresses are linear in the row
    // (every kernel here is); the full expert count is walked for the first routed tensor
    for (int a = 1; a <= 6; a++) {
        const size_t experts = a <= 3 ? (a == 1 ? (size_t)E : 3) : 1;
        PfTensorPlace p;
        if (!pf_tensor_place(type[a], k_storage[a], n_out[a], experts, &p)) { fprintf(stderr, "tensor %d: no layout\n", a); return 2; }
        const size_t rows = n_out[a] * experts, head = pf_split_header_bytes(type[a]);
        size_t block = 1, size = 1;
        pf_block_geometry(type[a], &block, &size);
        const size_t blocks = rows * p.blocks_per_row;
        const Buffer gguf = {"gguf bytes", p.gguf_bytes, 0, 0, p.gguf_bytes};
        // the tensor's device buffer as pf_hip_moe_create allocates it
        const Buffer device = {"device tensor", head ? blocks * (size - head) : p.bytes, p.scale_offset, blocks * head, p.bytes};
        if (head) {   // split at upload
            std::vector<unsigned char> written(a == 1 && E > 64 ? 0 : p.bytes);   // (the large walk checks bounds only)
            if (type[a] == PF_IQ2_XXS)
                walk("pf_k_iq2_split", pf_iq2_split_threads(blocks), [&](size_t i) { return pf_iq2_split_move(i, blocks); }, gguf, device,
                     written.empty() ? nullptr : &written);
            else
                walk("pf_k_block_split", pf_block_split_threads(blocks, (int)size),
                     [&](size_t i) { return pf_block_split_move(i, blocks, (int)size, (int)head); }, gguf, device, written.empty() ? nullptr : &written);
        }
        if (n_out[a] % 32) continue;
        if (type[a] == PF_Q4_K) {   // second copy in tile order: the same size as the tensor
            const Buffer tiled = {"tile-ordered Q4_K", p.bytes, 0, 0, p.bytes};
            std::vector<unsigned char> written(a == 1 && E > 64 ? 0 : p.bytes);
            walk("pf_k_q4k_tile", pf_q4k_tile_threads(rows, p.blocks_per_row), [&](size_t i) { return pf_q4k_tile_move(i, rows, p.blocks_per_row); },
                 device, tiled, written.empty() ? nullptr : &written);
            for (size_t b = 0; b < written.size(); b++)
                if (written[b] != 1) { complain("pf_k_q4k_tile", "leaves a byte unwritten", 0, b, 1, p.bytes); break; }
        } else if (type[a] == PF_IQ2_XXS) {
            const size_t bytes = pf_i2t_expert_bytes((int)n_out[a], p.blocks_per_row) * experts;
            const Buffer tiled = {"tile-ordered IQ2_XXS", bytes, 0, 0, bytes};
            walk("pf_k_iq2_tile", pf_iq2_tile_threads(rows, p.blocks_per_row), [&](size_t i) { return pf_iq2_tile_move(i, rows, p.blocks_per_row); },
                 device, tiled, nullptr);
        } else if (type[a] == PF_Q8_0 && experts == 1 && k_storage[a] % 64 == 0 && (a == 4 || a == 5)) {
            const size_t bytes = pf_q8t_expert_bytes((int)n_out[a], (int)(k_storage[a] / 64));
            const Buffer tiled = {"tile-ordered Q8_0", bytes, 0, 0, bytes};
            walk("pf_k_q8_tile", pf_q8_tile_threads(n_out[a], p.blocks_per_row), [&](size_t i) { return pf_q8_tile_move(i, n_out[a], p.blocks_per_row); },
                 device, tiled, nullptr);
        }
    }
    printf("%lld moves checked, %lld out of bounds or misaligned\n", checked, bad);
    return bad ? 1 : 0;
}
